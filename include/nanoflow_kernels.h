/*
 * nanoflow_kernels.h -- C ABI of the MI355X (gfx950) kernel layer.
 *
 * One entry point per operator of the reference's single-device nano-batch
 * pipeline.  Every function takes raw DEVICE pointers, plain sizes and a HIP
 * stream (as void*; NULL = the default stream), enqueues its kernels on that
 * stream without synchronising, and returns 0 on success or a negative
 * NF_ERR_* code (nf_last_error() gives the text).  fp16 tensors are IEEE
 * binary16 bit patterns (uint16_t).  No function allocates device memory.
 *
 * Each declaration cites the reference interface it replaces
 * (paths relative to the reference checkout).
 */
#ifndef NANOFLOW_KERNELS_H
#define NANOFLOW_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* nf_stream_t; /* hipStream_t */

/* Exported symbols (the library is built with hidden default visibility). */
#define NF_API __attribute__((visibility("default")))

#define NF_OK 0
#define NF_ERR_INVALID_ARGUMENT (-1) /* shape/pointer rejected before any launch */
#define NF_ERR_UNSUPPORTED (-2)      /* valid request this build has no kernel for */
#define NF_ERR_RUNTIME (-3)          /* HIP runtime reported an error */
#define NF_ERR_WORKSPACE (-4)        /* caller's workspace is too small */

/* ABI version of this header (bumped on any signature change). */
NF_API int nf_abi_version(void);
/* Text of the last error raised on the calling thread ("" if none). */
NF_API const char* nf_last_error(void);

/* x[t,:] = table[tokens[t],:]; hidden % 8 == 0.
 * Replaces genEmbedding<<<>>> as launched by GenEmbedding::work
 * (pipeline/src/small_cuda_operator.cu:9-24, pipeline/include/otherWrapper.cuh:166-171). */
NF_API int nf_embedding_f16(const int32_t* tokens, const uint16_t* table, uint16_t* out, int n_tokens,
                     int hidden, nf_stream_t stream);

/* Moves the KV pages of the listed requests between one layer's pool and a staging buffer laid
 * out like kv_indices: for every r = req_idx[i], i < req_num, and every
 * j in [kv_indptr[r], kv_indptr[r+1]): staging page j <- pool page kv_indices[j] (to_pool == 0,
 * offloading) or pool page kv_indices[j] <- staging page j (to_pool != 0, loading back).  A page
 * is page_bytes bytes (K and V halves together: vortexModelConfig::page_mem_size), a multiple
 * of 16.  All pointers are device (or device-accessible pinned) memory.
 * Replaces moveKVcacheKernel (pipeline/src/offloadKernel.cu:17-34) behind PageAggregator /
 * PageDispatcher (pipeline/include/otherWrapper.cuh:413-472). */
NF_API int nf_move_kv_pages(int req_num, const int32_t* req_idx, const int32_t* kv_indptr, const int32_t* kv_indices,
                            uint16_t* staging, uint16_t* kv_data, size_t page_bytes, int to_pool, nf_stream_t stream);

/* out = half(x * rsqrt(mean(x^2) + eps) * weight), fp32 math; hidden % 8 == 0.
 * Replaces rms_norm() (pipeline/include/rms_norm.cuh:48-127,210-233) called by
 * LayerNorm::work (pipeline/include/otherWrapper.cuh:94-102). */
NF_API int nf_rmsnorm_f16(uint16_t* out, const uint16_t* in, const uint16_t* weight, int rows, int hidden,
                   float eps, nf_stream_t stream);
/* nf_rmsnorm_f16 whose result is also written in the form an fp8-weight GEMM takes: out_q [rows,
 * hidden] e4m3 bytes and row_scale [rows], bit for bit what nf_quantize_rows_e4m3 makes of `out`
 * (which is written as well), in the same launch.  hidden % 16 == 0, hidden <= 8192.  No counterpart
 * in the reference (its GEMMs are fp16 only). */
NF_API int nf_rmsnorm_quantize_e4m3(uint16_t* out, const uint16_t* in, const uint16_t* weight, uint8_t* out_q,
                                    float* row_scale, int rows, int hidden, float eps, nf_stream_t stream);

/* D = half(alpha * A.B + beta * C), fp16 operands, fp32 accumulate on MFMA.
 * A [M,K] row-major; B [K,N] row-major when b_col_major == 0, [N,K] row-major
 * (K contiguous) when 1; C and D [M,N] row-major; C may alias D or be NULL when
 * beta == 0.  K % 8 == 0, N % 8 == 0.
 * Replaces CutlassGEMMWrapper::work / cutlass::gemm::device::Gemm
 * (pipeline/include/cutlassGemmWrapperImpl.cuh:68-166). */
NF_API int nf_gemm_f16(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int M, int N,
                int K, float alpha, float beta, int b_col_major, nf_stream_t stream);

/* nf_gemm_f16 with scratch: a GEMM of at most 512 rows whose output tiles would leave most of the
 * chip idle (few rows against a narrow N: the QKV, O and down projections of a small decode batch;
 * up to 320 rows any contraction of 1024 or more, from 321 to 512 rows contractions of 12288 or
 * more) is split over K into shares that fill it, summed in fp32 through `workspace`
 * (nf_gemm_workspace_bytes(M, N, K) bytes, 16-byte aligned; 0 = this shape is not split).  With a
 * null or short workspace, or a shape that does not profit, it is nf_gemm_f16.  The sum over k is
 * then taken share by share, so results differ from nf_gemm_f16 in fp32 rounding only.
 * nf_gemm_workspace_bytes_upto(max_M, N, K): the largest requirement over 1..max_M rows.
 * No counterpart in the reference (its serial split-K is a tag field of the CUTLASS kernel,
 * pipeline/include/gemmShape.cuh:5-6). */
NF_API size_t nf_gemm_workspace_bytes(int M, int N, int K);
NF_API size_t nf_gemm_workspace_bytes_upto(int max_M, int N, int K);
NF_API int nf_gemm_f16_ws(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int M, int N, int K,
                          float alpha, float beta, int b_col_major, void* workspace, size_t workspace_bytes,
                          nf_stream_t stream);
/* nf_gemm_f16_ws for callers that cannot allocate or pass a workspace (code under hipGraph
 * capture, serving loops and harnesses that forbid hipMalloc): the partial sums of a launch split
 * over K go to a static device array inside the library, nf_gemm_noalloc_scratch_bytes() = 32 MiB,
 * which every device the library runs on holds until the process ends.  Calls no hipMalloc / hipFree
 * or any allocating routine; the first call on a device looks up the array's address
 * (hipGetSymbolAddress), so make that call outside a capture.  A shape whose split needs more than
 * the array holds is rejected (NF_ERR_INVALID_ARGUMENT, nothing launched); shapes that are not
 * split run as nf_gemm_f16 and never touch the array.  Nothing in the array has to start at zero
 * (every share overwrites its sums before the reduction reads them), but all calls on one device
 * share it: calls that overlap in time on one device (two streams) race.
 * Results are bit-identical to nf_gemm_f16_ws with a workspace of nf_gemm_workspace_bytes().
 * No counterpart in the reference. */
NF_API int nf_gemm_f16_noalloc(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int M, int N,
                               int K, float alpha, float beta, int b_col_major, nf_stream_t stream);
NF_API size_t nf_gemm_noalloc_scratch_bytes(void);
/* the same for the fused gate/up pair: both products are split, their fp32 sums rounded to fp16 and
 * put through SiLU-mul by the reduction (workspace: nf_dual_swiglu_workspace_bytes(M, N, K)) */
NF_API size_t nf_dual_swiglu_workspace_bytes(int M, int N, int K);
NF_API size_t nf_dual_swiglu_workspace_bytes_upto(int max_M, int N, int K);
NF_API int nf_dual_swiglu_f16_ws(const uint16_t* A, const uint16_t* Bgate, const uint16_t* Bup, uint16_t* out,
                                 int M, int N, int K, int b_col_major, void* workspace, size_t workspace_bytes,
                                 nf_stream_t stream);
/* nf_gemm_f16 / nf_gemm_bias_f16 (c_is_row != 0: C is one row [N] added to every row) on a tile and
 * a split over K of the CALLER's choosing: what the cta_m, cta_n and split_k fields of the reference's
 * GEMM tag select (pipeline/include/gemmShape.cuh:5-6; there one CUTLASS instantiation per tag,
 * pipeline/include/gemmFactory.in:7-16).  The tile is the entry of the library's menu closest to
 * tile_m x tile_n (nf_gemm_tile_menu enumerates it: index 0 .. count-1 -> tile sizes and whether the
 * entry takes k-contiguous weights only; returns the count); split_k > 1 cuts K into that many shares
 * (at most 16, each at least 64 deep) whose fp32 sums go through `workspace`
 * (nf_gemm_tiled_workspace_bytes(M, N, K, split_k) bytes, 16-byte aligned) and are added by a second
 * launch.  Results agree with nf_gemm_f16 to fp32 summation order. */
NF_API int nf_gemm_tile_menu(int index, int* tile_m, int* tile_n, int* k_contiguous_weights_only);
NF_API size_t nf_gemm_tiled_workspace_bytes(int M, int N, int K, int split_k);
NF_API int nf_gemm_f16_tiled(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int M, int N, int K,
                             float alpha, float beta, int b_col_major, int c_is_row, int tile_m, int tile_n,
                             int split_k, void* workspace, size_t workspace_bytes, nf_stream_t stream);
/* the same for nf_gemm_bias_f16 (declared below) */
NF_API int nf_gemm_bias_f16_ws(const uint16_t* A, const uint16_t* B, const uint16_t* bias, uint16_t* D, int M, int N,
                               int K, float alpha, float beta, int b_col_major, void* workspace,
                               size_t workspace_bytes, nf_stream_t stream);

/* D = half(alpha * A.B + beta * bias[n]): nf_gemm_f16 with one row, bias [N], added to every row
 * of the product, read in the epilogue instead of from an [M,N] copy of it.
 * Replaces the QKV GEMM of the *_KQVBIAS pipelines, whose C operand is the bias replicated over
 * max-batch rows by replicateKQVBias (pipeline/src/small_cuda_operator.cu:254-292; used at
 * pipeline/src/pipeline.cu:520-533,1048-1058, pipeline_nonoverlap.cu:163-168,209-211). */
NF_API int nf_gemm_bias_f16(const uint16_t* A, const uint16_t* B, const uint16_t* bias, uint16_t* D, int M,
                     int N, int K, float alpha, float beta, int b_col_major, nf_stream_t stream);

/* out = half(silu(float(half(A.Bgate))) * float(half(A.Bup))); A [M,K] and out [M,N] row-major;
 * Bgate/Bup [K,N] row-major (b_col_major = 0, the orientation the reference's weight files use)
 * or [N,K], k contiguous (b_col_major = 1: the layout a GEMM tag calls ColumnMajor for B,
 * pipeline/src/generate-gemm/genGEMM.py:44-49).  K % 8 == 0, N % 8 == 0.
 * Replaces DualWrapper::work / cutlass DualGemm + LeftSiLUAndMul
 * (pipeline/include/dualWrapper.cuh:95-144,192-194). */
NF_API int nf_dual_swiglu_f16(const uint16_t* A, const uint16_t* Bgate, const uint16_t* Bup, uint16_t* out,
                       int M, int N, int K, int b_col_major, nf_stream_t stream);

/* The same two operators on bfloat16 storage (bf16 x bf16 -> fp32 -> bf16, products rounded to bf16
 * before SiLU-mul): same kernels, other element type.  The reference's wrappers are fp16 only
 * (cutlassGemmWrapperImpl.cuh:24-27); these have no counterpart there and the pipeline does not
 * use them. */
NF_API int nf_gemm_bf16(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int M, int N,
                 int K, float alpha, float beta, int b_col_major, nf_stream_t stream);
NF_API int nf_dual_swiglu_bf16(const uint16_t* A, const uint16_t* Bgate, const uint16_t* Bup, uint16_t* out,
                        int M, int N, int K, nf_stream_t stream);

/* fp8 GEMM family (OCP e4m3: bias 7, no infinities, max 448) on the fp8 matrix cores.  No
 * counterpart in the reference (its GEMM wrappers are half-only,
 * pipeline/include/cutlassGemmWrapperImpl.cuh:24-27); operand roles as in nf_gemm_f16.
 *
 * nf_quantize_rows_e4m3: row_scale[m] = max_k |X[m][k]| / 448 (1 for an all-zero row),
 *   Xq[m][k] = e4m3(X[m][k] / row_scale[m]), round to nearest even.  X fp16 [M,K], K % 16 == 0.
 * nf_gemm_f8_f16: D = half(alpha * a_scale[m] * b_scale[n] * sum_k Aq[m][k] * Bq[n][k] + beta * C)
 *   with Aq [M,K] and Bq [N,K] e4m3 bytes (weights stored one row per output channel, k
 *   contiguous), fp32 accumulation.  K % 16 == 0, N % 8 == 0.
 * nf_gemm_f8w_f16: fp16 activations against fp8 weights = the two calls above, the quantised
 *   activations and their scales living in `workspace` (nf_gemm_f8w_workspace_bytes(M, K)
 *   bytes, 16-byte aligned).
 * nf_quantize_weight_e4m3: a weight in the pipeline's orientation, W fp16 [K,N] row-major, to the
 *   form the two GEMMs above take: Wq [N,K] e4m3 with col_scale[n] = max_k |W[k][n]| / 448 (1 for
 *   an all-zero column), Wq[n][k] = e4m3(W[k][n] / col_scale[n]): the row quantiser applied to the
 *   transpose.  K % 16 == 0, N % 8 == 0.
 * nf_dual_swiglu_f8_f16: out = half(silu(g) * u) with g = half(a_scale[m] * g_scale[n] * sum_k
 *   Aq[m][k] * Gq[n][k]) and u likewise from Uq, u_scale: nf_dual_swiglu_f16 on fp8 operands
 *   (products rounded to fp16 before SiLU-mul, as there).  nf_dual_swiglu_f8w_f16: the same from
 *   fp16 activations, quantised into `workspace` (nf_gemm_f8w_workspace_bytes(M, K) bytes).
 * nf_gemm_f8q_f16 / nf_dual_swiglu_f8q_f16: nf_gemm_f8w_f16 / nf_dual_swiglu_f8w_f16 on activations
 *   that are quantised already (Aq, a_scale: by nf_quantize_rows_e4m3 or nf_rmsnorm_quantize_e4m3);
 *   `workspace` (may be NULL) is the one the f8w form would be given and is used, at the same
 *   offsets, for the sums of a launch split over K only. */
/* nf_gemm_f8w_f16 and nf_dual_swiglu_f8w_f16 split launches of at most 256 rows over K, like
 * nf_gemm_f16_ws, when the workspace also has room for the fp32 sums behind the quantised rows:
 * nf_gemm_f8w_split_workspace_bytes(M, N, K) / nf_dual_swiglu_f8w_split_workspace_bytes(M, N, K)
 * bytes (equal to nf_gemm_f8w_workspace_bytes(M, K) for shapes that are not split); *_upto: the
 * largest requirement over 1..max_M rows. */
NF_API size_t nf_gemm_f8w_split_workspace_bytes(int M, int N, int K);
NF_API size_t nf_gemm_f8w_split_workspace_bytes_upto(int max_M, int N, int K);
NF_API size_t nf_dual_swiglu_f8w_split_workspace_bytes(int M, int N, int K);
NF_API size_t nf_dual_swiglu_f8w_split_workspace_bytes_upto(int max_M, int N, int K);
NF_API int nf_quantize_weight_e4m3(const uint16_t* W, uint8_t* Wq, float* col_scale, int K, int N,
                                   nf_stream_t stream);
NF_API int nf_dual_swiglu_f8_f16(const uint8_t* Aq, const float* a_scale, const uint8_t* Gq, const float* g_scale,
                                 const uint8_t* Uq, const float* u_scale, uint16_t* out, int M, int N, int K,
                                 nf_stream_t stream);
NF_API int nf_dual_swiglu_f8w_f16(const uint16_t* A, const uint8_t* Gq, const float* g_scale, const uint8_t* Uq,
                                  const float* u_scale, uint16_t* out, int M, int N, int K, void* workspace,
                                  size_t workspace_bytes, nf_stream_t stream);
NF_API int nf_quantize_rows_e4m3(const uint16_t* X, uint8_t* Xq, float* row_scale, int M, int K,
                                 nf_stream_t stream);
NF_API int nf_gemm_f8_f16(const uint8_t* Aq, const float* a_scale, const uint8_t* Bq, const float* b_scale,
                          const uint16_t* C, uint16_t* D, int M, int N, int K, float alpha, float beta,
                          nf_stream_t stream);
NF_API int nf_gemm_f8q_f16(const uint8_t* Aq, const float* a_scale, const uint8_t* Bq, const float* b_scale,
                           const uint16_t* C, uint16_t* D, int M, int N, int K, float alpha, float beta,
                           void* workspace, size_t workspace_bytes, nf_stream_t stream);
NF_API int nf_dual_swiglu_f8q_f16(const uint8_t* Aq, const float* a_scale, const uint8_t* Gq, const float* g_scale,
                                  const uint8_t* Uq, const float* u_scale, uint16_t* out, int M, int N, int K,
                                  void* workspace, size_t workspace_bytes, nf_stream_t stream);
NF_API size_t nf_gemm_f8w_workspace_bytes(int M, int K);
NF_API int nf_gemm_f8w_f16(const uint16_t* A, const uint8_t* Bq, const float* b_scale, const uint16_t* C,
                           uint16_t* D, int M, int N, int K, float alpha, float beta, void* workspace,
                           size_t workspace_bytes, nf_stream_t stream);

/* Per token t of kqv [n_tokens,(Hq+2Hkv)*d] (columns K | V | Q): request
 * r = rev_input_indptr[t], position p = per_token_offset[t],
 * page = kv_indices[kv_indptr[r] + p / page_size], entry = p % page_size;
 * K heads -> rotate-half RoPE at p -> kv_data[page][0][entry]; V heads -> copied to
 * kv_data[page][1][entry]; Q heads -> RoPE -> q_out[t].  kv_data is one layer's pool
 * [pages][2][page_size][Hkv][d].  head_dim must be 128.
 * rope_scale / smooth_a / smooth_b implement the Llama-3.1 frequency rule; pass
 * 1, 0, 0 for plain RoPE.
 * Replaces flashinfer::splitRopeAppend (pipeline/include/small_cuda_operator.cuh:21-133)
 * called by RoPEAppend::work (pipeline/include/otherWrapper.cuh:345-380). */
NF_API int nf_rope_append_f16(const uint16_t* kqv, uint16_t* q_out, uint16_t* kv_data,
                       const int32_t* kv_indices, const int32_t* kv_indptr,
                       const int32_t* rev_input_indptr, const int32_t* per_token_offset,
                       int n_tokens, int num_qo_heads, int num_kv_heads, int head_dim,
                       int page_size, float rope_scale, float rope_theta, float smooth_a,
                       float smooth_b, nf_stream_t stream);

/* Bytes of device workspace nf_attention_paged_f16 needs for this problem size. */
NF_API size_t nf_attention_workspace_bytes(int batch, int max_qo_rows, int num_qo_heads);

/* Batched attention over a paged KV pool.  For request i in [0,batch): query rows
 * qo_indptr[i]..qo_indptr[i+1] of q/o (ABSOLUTE row indices into buffers of row
 * width Hq*d), keys/values = pages kv_indices[kv_indptr[i]..kv_indptr[i+1]) with
 * kv_last_page_len[i] valid entries in the last page.  causal != 0: row j of a
 * request with qo_len rows sees keys <= kv_len - qo_len + j.  sm_scale = 1/sqrt(d),
 * no position encoding inside.  head_dim 128, page_size 16, Hq/Hkv in {1,2,4,8}.
 * max_qo_rows: an upper bound on the total number of query rows of the batch
 * (sizes the launch; a bound that is too small is an error the kernel cannot see).
 * num_blocks > 0 caps the number of workgroups (the reference's sm_blk); 0 = fill
 * the device.  workspace: nf_attention_workspace_bytes() bytes of device scratch.
 * Replaces BatchPrefillWithPagedKVCacheWrapper as used by DecodeGemvWrapper::work
 * (causal=false, pipeline/include/gemvWrapper.cuh:201-228) and PrefillGemvWrapper::work
 * (causal=true, :322-374), including the planning done by BatchPrefillHandler::BeginForward
 * (gemv/include/attention/handler.cuh:557-595), which here runs on the device. */
NF_API int nf_attention_paged_f16(const uint16_t* q, uint16_t* o, const int32_t* qo_indptr,
                           const uint16_t* kv_data, const int32_t* kv_indptr,
                           const int32_t* kv_indices, const int32_t* kv_last_page_len, int batch,
                           int max_qo_rows, int num_qo_heads, int num_kv_heads, int head_dim,
                           int page_size, int causal, int num_blocks, void* workspace,
                           size_t workspace_bytes, nf_stream_t stream);

/* The smaller operators of the reference's vocabulary; none is on a single-device schedule's path.
 * nf_split_kqv_f16: k, q, v [rows, *_dim] = the three column ranges of kqv [rows, k_dim + q_dim +
 *   v_dim], in that order (splitKQVOutput, pipeline/src/small_cuda_operator.cu:27-59; SplitKQVOutput,
 *   pipeline/include/otherWrapper.cuh:183-232); widths % 8 == 0, a zero width takes a null pointer.
 * nf_extract_rank_columns_f16: out [rows, cols] = columns [rank * cols, (rank + 1) * cols) of in
 *   [rows, nranks * cols] (extractRankSubmatrixHalfDevice, small_cuda_operator.cu:133-161;
 *   SplitTensor, otherWrapper.cuh:235-263); cols % 8 == 0.
 * nf_silu_mul_f16: out [rows, cols] = in[:, :cols] * silu(in[:, cols:]) of in [rows, 2 * cols], fp32
 *   arithmetic, one rounding (silu_and_multiply, small_cuda_operator.cu:100-129; Activation,
 *   otherWrapper.cuh:268-287); cols % 8 == 0.
 * nf_transpose_f16: out [cols, rows] = in [rows, cols] transposed, any shape, not in place
 *   (transpose, small_cuda_operator.cu:64-97; Transpose, otherWrapper.cuh:395-411).
 * nf_sleep_us: a kernel that occupies the stream for `us` microseconds (at most 1 s) by the device's
 *   real-time counter (cudaSleep, pipeline/src/sleep.cu:5-11; SleepWrapper, otherWrapper.cuh:290-300). */
NF_API int nf_split_kqv_f16(const uint16_t* kqv, uint16_t* k, uint16_t* q, uint16_t* v, int rows, int k_dim, int q_dim,
                            int v_dim, nf_stream_t stream);
NF_API int nf_extract_rank_columns_f16(const uint16_t* in, uint16_t* out, int rows, int cols, int nranks, int rank,
                                       nf_stream_t stream);
NF_API int nf_silu_mul_f16(const uint16_t* in, uint16_t* out, int rows, int cols, nf_stream_t stream);
NF_API int nf_transpose_f16(const uint16_t* in, uint16_t* out, int rows, int cols, nf_stream_t stream);
NF_API int nf_sleep_us(int us, nf_stream_t stream);

/* out[r,:] = in[input_indptr[r+1]-1,:] (last token of each request); hidden % 8 == 0.
 * Replaces copySelectedRows (pipeline/src/small_cuda_operator.cu:217-251) called by
 * KeepToken::work (pipeline/include/otherWrapper.cuh:521-523). */
NF_API int nf_keep_token_f16(const uint16_t* in, uint16_t* out, const int32_t* input_indptr, int req_num,
                      int hidden, nf_stream_t stream);

/* Row argmax over fp16 logits [rows, cols] -> argmax[rows] (and max_vals[rows] when not
 * NULL), with the tie order of the reference kernel (values <= -10000 never win;
 * equal maxima: smallest bit-reversed (col mod 1024), then smallest col).
 * Replaces computeRowMax (pipeline/src/small_cuda_operator.cu:165-214) called by
 * MaxSampling::work (pipeline/include/otherWrapper.cuh:489-491). */
NF_API int nf_argmax_f16(const uint16_t* logits, uint16_t* max_vals, int32_t* argmax, int rows, int cols,
                  nf_stream_t stream);

/* Calibration micro-benchmarks: ceilings measured on the device the library runs on, beside which
 * the kernels' rates are reported.  Each call launches, waits for and times its own kernels (HIP
 * events on `stream`); `scratch` is at least 8192 bytes of device memory the kernels may write.
 * nf_calibrate_mfma: a register-only loop of independent 32x32 MFMA instructions (fp8 == 0:
 *   v_mfma_f32_32x32x16_f16; else the 32x32x64 fp8 form), one wavefront per SIMD, `iters` x 16
 *   instructions per wavefront, on zero operands (random_operands == 0), on pseudo-random ones
 *   (1), or (2, fp16 only) on pseudo-random operands that each wavefront re-reads from LDS before
 *   every 16 instructions, the way the main loop of the 256x256 GEMM tile is fed, or (3, fp16
 *   only; `scratch` then holds 8192 + 8 MiB bytes) with that tile's operand loads beside them as
 *   well, from a window of scratch the L2 holds straight into LDS, or (4) as 1 with the 16x16
 *   instruction of the type instead (16x16x32 f16, 16x16x128 fp8; the same flops per pass on 64
 *   accumulators);
 *   *tflops = the rate, *clock_mhz = shader clock the wavefronts saw while running.
 * nf_calibrate_hbm_read: all CUs stream `bytes` of `buf` (16-byte aligned, much larger than the
 *   last-level cache) `reps` times; *gbps = the read rate.
 * nf_calibrate_paged_read: the access pattern of paged decode attention (arguments as
 *   nf_attention_paged_f16's: page size 16, head_dim 128) without its arithmetic;
 *   *gbps = kv_bytes_per_launch x reps / time.
 * No counterpart in the reference, whose benchmarks divide by vendor peaks. */
NF_API int nf_calibrate_mfma(int fp8, int random_operands, int iters, void* scratch, size_t scratch_bytes,
                             double* tflops, double* clock_mhz, nf_stream_t stream);
NF_API int nf_calibrate_hbm_read(const void* buf, size_t bytes, int reps, void* scratch, size_t scratch_bytes,
                                 double* gbps, nf_stream_t stream);
NF_API int nf_calibrate_paged_read(const uint16_t* kv_data, const int32_t* kv_indptr, const int32_t* kv_indices,
                                   const int32_t* kv_last_page_len, int batch, int num_kv_heads,
                                   size_t kv_bytes_per_launch, int reps, void* scratch, size_t scratch_bytes,
                                   double* gbps, nf_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* NANOFLOW_KERNELS_H */
