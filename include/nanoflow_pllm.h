/*
 * nanoflow_pllm.h -- C ABI of the pipeline control plane (host library libnf_pipeline.so).
 *
 * Flat-C mirror of what the reference exports to its Python frontend through the
 * pybind11 module `pllm_python` (pipeline/src/pybind.cu:189-284) and to C++ callers
 * through pipeline/include/computeBound.cuh:76-87: one pipeline on one GPU, driven
 * by init -> config -> (update -> run | run_async .. run_async_wait)* -> finalize.
 * Structs have the reference's fields in the reference's order
 * (pipeline/include/vortexData.cuh:7-111) with std::vector / std::string members
 * replaced by pointer + count.  fp16 data is uint16_t bit patterns.
 *
 * Every function returns 0 on success and a negative NF_PLLM_ERR_* code otherwise
 * (pllm_last_error() gives the text).  As in the reference, a failing GPU runtime
 * call inside the pipeline terminates the process.
 */
#ifndef NANOFLOW_PLLM_H
#define NANOFLOW_PLLM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NF_PLLM_API __attribute__((visibility("default")))

#define NF_PLLM_OK 0
#define NF_PLLM_ERR_INVALID_ARGUMENT (-1)
#define NF_PLLM_ERR_STATE (-2)       /* call out of order (e.g. update before config) */
#define NF_PLLM_ERR_UNSUPPORTED (-3) /* more than one rank, a model shape the kernels are not built for */

/* Worker::PipelineType (pipeline/include/computeBound.cuh:22-34). */
enum nf_pipeline_type {
  /* The reference's main Pipeline (pipeline/src/pipeline.cu): QKV projection, RoPE-append and
   * decode attention as four nano-batches (sizes kqv1, nano1 - kqv1, kqv3, T - nano1 - kqv3), O and
   * the FFN as two, attention on a stream of its own; on this one rank without its exchange steps. */
  NF_PIPE_PLLM = 0,
  NF_PIPE_NONOVERLAP = 1,  /* its sequential schedule: runs as NON_OVERLAP_LOCAL */
  NF_PIPE_NANOBATCH = 2,   /* PLLM's nano-batches on one stream */
  /* PLLM plus the KV offload round trip of pipeline.cu:37-59,701-726: every layer the pages of the
   * iteration's first two requests are gathered, copied to pinned host memory, copied back and
   * scattered into the pool again (results are PLLM's). */
  NF_PIPE_PLLMOFFLOAD = 3,
  /* models with a bias on the q/k/v projections (Qwen2; pipeline/src/computeBound.cu:234-242):
   * on this one device they run as LOCAL / NON_OVERLAP_LOCAL / NANOBATCH_LOCAL with
   * vortexLayerWeight::B_KQV added by the QKV GEMMs */
  NF_PIPE_KQVBIAS = 4,
  NF_PIPE_NONOVERLAP_KQVBIAS = 5,
  NF_PIPE_NANOBATCH_KQVBIAS = 6,
  NF_PIPE_LOCAL = 7,             /* two nano-batches, GEMM and attention streams overlapped */
  NF_PIPE_NON_OVERLAP_LOCAL = 8, /* sequential baseline */
  NF_PIPE_NANOBATCH_LOCAL = 9    /* nano-batched, single stream */
};

/* vortexWeight (vortexData.cuh:7-12) */
typedef struct nf_vortex_weight {
  uint16_t* ptr;
  int N;
  int K;
} nf_vortex_weight;

/* vortexLayerWeight (vortexData.cuh:14-25).  Weights are K x N row-major; W_KQV columns are
 * ordered K | V | Q (pipeline/utils/weightSaver.py:118). */
typedef struct nf_vortex_layer_weight {
  nf_vortex_weight W_O1, W_O2, W_U, W_G, W_D, W_KQV, B_KQV, W_LN_Attention, W_LN_FFN, W_ROT;
} nf_vortex_layer_weight;

/* vortexModelWeight (vortexData.cuh:27-32) */
typedef struct nf_vortex_model_weight {
  nf_vortex_weight lm_head;
  nf_vortex_weight embedding;
  nf_vortex_weight model_layernorm;
  const nf_vortex_layer_weight* layer_weight;
  int num_layers;
} nf_vortex_model_weight;

/* vortexInitData (vortexData.cuh:35-53).  All pointers are DEVICE memory owned by the caller
 * for the life of the pipeline. */
typedef struct nf_vortex_init_data {
  uint16_t** kv_data; /* host array of num_layers device pools [pages,2,page,Hkv,d] */
  nf_vortex_model_weight weight;
  size_t weight_size;
  uint16_t* tmp_buffer;
  size_t tmp_buffer_size; /* in halves */
} nf_vortex_init_data;

/* vortexUpdateData (vortexData.cuh:55-90).  All arrays are HOST memory (pinned or not); they
 * are staged during pllm_update and may be reused when it returns. */
typedef struct nf_vortex_update_data {
  int decodePrefillBorder;
  int prefillNum;
  int prefillTokensNum;
  int keepTokenListLength;
  int* input_tokens; /* the prefill tokens only; decode tokens come from the last samples */
  int32_t* input_indptr;
  int32_t* rev_input_indptr;
  int32_t* keep_token_list;
  int32_t* kv_indptr;
  int32_t* kv_indices;
  int32_t* kv_last_page_len;
  int32_t* per_token_offset;
  int32_t* gemv_batch_size; /* [4] */
  int32_t* gemv_num_blocks; /* [4] */
} nf_vortex_update_data;

/* vortexConfigData (vortexData.cuh:104-110) */
typedef struct nf_vortex_config_data {
  const char* const* gemm_op_tag;
  int num_gemm_op_tag;
  int global_batch_size;
  int nanobatch_1_size;
  int kqv1_size;
  int kqv3_size;
} nf_vortex_config_data;

NF_PLLM_API const char* pllm_last_error(void);

/* setModelConfig (pybind.cu:154-156 -> updateVortexModelConfig, load_config.cu:11-112). */
NF_PLLM_API int pllm_set_model_config(const char* json_path);
/* setRank (pybind.cu:10-13); only nranks == 1 is accepted. */
NF_PLLM_API int pllm_set_rank(int nranks, int vnranks);
/* Size of the tmp buffer (in halves) and of one layer's KV pool (in pages) that the current
 * model configuration asks for (ModelConfig.k_temp_size / max_page_num, config.h:99-100). */
NF_PLLM_API size_t pllm_tmp_buffer_halves(void);
NF_PLLM_API size_t pllm_max_page_num(void);
/* pllm_python.init (pybind.cu:73-98) with weights already on the device
 * (the C++ init(), computeBound.cu:65-113).  Spawns the worker thread. */
NF_PLLM_API int pllm_init(const nf_vortex_init_data* input, int pipeline_type);
/* modelWeightToGPU (vortexData.cu:340-373): uploads a host-resident weight set; the device
 * copies are written to *device_weight / device_layers[num_layers]. */
NF_PLLM_API int pllm_model_weight_to_gpu(const nf_vortex_model_weight* host_weight,
                                         nf_vortex_model_weight* device_weight,
                                         nf_vortex_layer_weight* device_layers);
/* pllm_python.createModelWeight (pybind.cu:228, vortexData.cu:386-406): device memory for every
 * weight of the configured model (zero-filled here; the reference leaves it as allocated), never
 * freed.  layers must have room for the model's layer count; *weight points at it. */
NF_PLLM_API int pllm_create_model_weight(nf_vortex_model_weight* weight, nf_vortex_layer_weight* layers,
                                         int layers_capacity);
/* createModelWeightCPU (vortexData.cu:375-384), which is what the reference's Python module exports
 * as createModelWeight (pybind.cu:281): HOST memory for every weight of the configured model
 * (zero-filled, never freed), to be uploaded by pllm_model_weight_to_gpu as pllm_python.init does. */
NF_PLLM_API int pllm_create_model_weight_host(nf_vortex_model_weight* weight, nf_vortex_layer_weight* layers,
                                              int layers_capacity);
/* Layers of the configured model (0 before pllm_set_model_config): the capacity the builders ask for. */
NF_PLLM_API int pllm_num_layers(void);
/* pllm_python.createInitData (pybind.cu:229, vortexData.cu:33-56): the tmp buffer and one zeroed
 * KV pool per layer for the configured model (never freed) around the given weights.  kv_data
 * must have room for the model's layer count. */
NF_PLLM_API int pllm_create_init_data(nf_vortex_init_data* data, uint16_t** kv_data, int layers_capacity,
                                      const nf_vortex_model_weight* weight);
/* pllm_python.config (pybind.cu:106-108). */
NF_PLLM_API int pllm_config(const nf_vortex_config_data* config);
/* What pllm_config checks before it builds anything, callable on its own (no state, no device):
 * 0 < global_batch_size <= max_batch_size; for the nano-batched types 0 < nanobatch_1_size <
 * global_batch_size; for the types that run the four-way schedule (PLLM, NANOBATCH, PLLMOFFLOAD,
 * KQVBIAS, NANOBATCH_KQVBIAS: pipeline/src/computeBound.cu:234-247) also 0 <= kqv1_size <=
 * nanobatch_1_size and 0 <= kqv3_size <= global_batch_size - nanobatch_1_size.  The reference
 * checks none of this (pipeline/src/pipeline.cu:279-470 sizes its buffers from the fields as given). */
NF_PLLM_API int pllm_check_nanobatch_split(int pipeline_type, int max_batch_size, int global_batch_size,
                                           int nanobatch_1_size, int kqv1_size, int kqv3_size);
/* What pllm_update checks of gemv_batch_size[4] (serve_8B.py:391-394 produces it): the groups sum
 * to the decode rows; nano-batched types: groups 0+1 = the decode rows of nano-batch 1; four-way
 * types: the rows of groups 0..i lie inside QKV pieces 0..i (decode attention of group i starts as
 * soon as QKV piece i and its RoPE-append are done, pipeline/src/pipeline.cu:640-676; a group that
 * reaches further would read rows not yet written).  No state, no device. */
NF_PLLM_API int pllm_check_gemv_split(int pipeline_type, int nanobatch_1_size, int kqv1_size, int kqv3_size,
                                      int decode_rows, const int32_t* gemv_batch_size);
/* pllm_python.update (pybind.cu:100-104 -> update(), computeBound.cu:115-161). */
NF_PLLM_API int pllm_update(const nf_vortex_update_data* update);
/* run / run_async / run_async_wait (computeBound.cu:27-61). */
NF_PLLM_API int pllm_run(void);
NF_PLLM_API int pllm_run_async(void);
NF_PLLM_API int pllm_run_async_wait(void);
/* getPipelineOutput (pybind.cu:158-186): non-owning view of the sampled token ids of the
 * last completed run, valid until the next run_async_wait. */
NF_PLLM_API int pllm_get_pipeline_output(const int32_t** tokens, int* count);
/* finalize (computeBound.cu:180-193). */
NF_PLLM_API int pllm_finalize(void);

/* The decode-token feed that update() applies before uploading (computeBound.cu:121-150),
 * exposed for host-side tests: out = [prev_output[i] for kept slots i] ++ prefill_tokens;
 * prev_count == 0 feeds token id 1 to every kept slot.  Returns the count written. */
NF_PLLM_API int pllm_build_input_tokens(const int32_t* prev_output, int prev_count,
                                        const int32_t* keep_token_list, int keep_token_list_length,
                                        const int32_t* prefill_tokens, int prefill_tokens_num,
                                        int32_t* out);

/* ---- CPU batch formation and the asynchronous serving loop ------------------------------
 * Replaces the Python scheduler that drives pllm_python in the reference:
 * DistKVPool / DistKVCache / BatchedDistKVCache (pipeline/utils/kv_cache.py:20-135) and
 * Scheduler.schedule_req / bench_text_gen (pipeline/utils/serve_8B.py:177-569).  The former
 * owns request queue, worksets and page tables; pllm_sched_form fills a
 * nf_vortex_update_data whose arrays stay valid until the next form call. */
typedef struct nf_batch_former nf_batch_former;

/* Scheduler(memory_pool, ..., decode_length, prefill_length) + init_pipe's batch sizes
 * (serve_8B.py:104-146); kv_pages = DistKVPool capacity (serve_8B.py:643). */
NF_PLLM_API nf_batch_former* pllm_sched_create(int kv_pages, int page_size, int global_batch_size,
                                               int nanobatch_1_size, int kqv1_size, int kqv3_size,
                                               int average_prefill_length,
                                               int average_decode_length);
NF_PLLM_API void pllm_sched_destroy(nf_batch_former* f);
/* NewRequestQueue.put (pipeline/utils/request_info.py:13-31). */
NF_PLLM_API int pllm_sched_add_request(nf_batch_former* f, int req_idx, const int32_t* prompt,
                                       int prompt_len, int output_len, double start_time);
/* schedule_req (serve_8B.py:212-346). */
NF_PLLM_API int pllm_sched_schedule(nf_batch_former* f);
/* bench_text_gen up to initUpdateData (serve_8B.py:356-451). */
NF_PLLM_API int pllm_sched_form(nf_batch_former* f, nf_vortex_update_data* out);
/* back-fill of the outputs of the iteration that just completed (serve_8B.py:499-520);
 * n == 0 when none has. */
NF_PLLM_API int pllm_sched_harvest(nf_batch_former* f, const int32_t* ids, int n);
/* predict_output (serve_8B.py:523-569): length-only retirement, keep list, next worksets.
 * placeholder_zero != 0 is the skip-cycle mode.  *n_retired = requests retired by this call. */
NF_PLLM_API int pllm_sched_advance(nf_batch_former* f, double now, int placeholder_zero,
                                   int* n_retired);
/* counts[0..4] = queued requests, decoding requests, prefilling requests, free pages,
 * retired requests so far. */
NF_PLLM_API int pllm_sched_state(nf_batch_former* f, int counts[5]);
/* Copies the outputs of retired request number `which` (retirement order): returns the number
 * of tokens written (<= cap), *req_idx its id; negative on error. */
NF_PLLM_API int pllm_sched_retired_output(nf_batch_former* f, int which, int* req_idx, int32_t* out,
                                          int cap);
/* check_future_page_usage (serve_8B.py:177-203): out[0..n) pages in use i iterations ahead;
 * returns the forecast length (average_prefill + average_decode + 2). */
/* Bookkeeping of retired request `which` as the reference writes it to its .req_time file
 * (serve_8B.py:795-797): times = {request_comein_time, encode_latency, decode_start_at,
 * decode_latency}, in the seconds of the `now` values passed to pllm_sched_advance (pllm_serve
 * uses a monotonic clock). */
NF_PLLM_API int pllm_sched_retired_info(nf_batch_former* f, int which, int* req_idx, int* input_len,
                                        int* output_len, double times[4]);
NF_PLLM_API int pllm_sched_future_page_usage(nf_batch_former* f, int64_t* out, int cap);

/* What the reference prints to its .stat file (serve_8B.py:755-793) plus the CPU-side split
 * of a cycle. */
typedef struct nf_serve_stats {
  int cycles;
  int retired;
  double wall_s;
  double tokens_per_s; /* retired * (average_prefill + average_decode) / wall_s */
  double cycle_ms;
  double form_ms;     /* CPU: schedule + form per cycle (overlaps the GPU run) */
  double wait_ms;     /* blocked in run_async_wait per cycle */
  double update_ms;   /* update() per cycle */
  double gpu_iter_ms; /* device time of an iteration */
  long long tokens_processed;
} nf_serve_stats;
/* The serving loop of serve_8B.py:655-700 over an initialised and configured pipeline:
 * skip_cycles simulated cycles (scheduler only), warmup_cycles executed but untimed cycles,
 * then run_cycles executed and timed cycles; batch i+1 is formed on the CPU while the GPU runs
 * batch i.  The timed region starts and ends with the GPU idle and resets the accumulated
 * pipeline timings at its start. */
NF_PLLM_API int pllm_serve(nf_batch_former* f, int skip_cycles, int warmup_cycles, int run_cycles,
                           nf_serve_stats* stats);

/* Measurement (no counterpart in the reference, which only logs the iteration time,
 * pipeline_local.cu:444-463).  pllm_set_profiling level 1 brackets every attention launch with
 * events on its own stream; level 2 also every dense GEMM launch; 0 switches it off.
 * Schedules of 8 or more layers time every 4th layer only (the event records cost device
 * time); the launch counts returned are the launches actually timed.  pllm_get_timings returns the last iteration's time and the
 * durations accumulated since the last pllm_reset_timings. */
typedef struct nf_pipeline_timings {
  double iter_ms;
  double decode_attn_ms;
  long decode_attn_launches;
  double prefill_attn_ms;
  long prefill_attn_launches;
  double gemm_ms;    /* dense GEMM launches (level 2): summed duration, count, flops */
  long gemm_launches;
  double gemm_flop;
  int layer_stride;  /* every layer_stride-th layer is timed: totals per iteration = sums * layer_stride */
} nf_pipeline_timings;
/* Storage of the five per-layer GEMM weights (W_KQV, W_O1/W_O2, W_G, W_U, W_D) in the init data
 * the next pllm_init is given; everything else (embedding, norms, B_KQV, LM head) is fp16 in both.
 * No counterpart in the reference, whose wrappers are half-only
 * (pipeline/include/cutlassGemmWrapperImpl.cuh:24-27).
 *   NF_WEIGHTS_F16:  ptr -> fp16 [K][N] row-major, as in the reference (the default).
 *   NF_WEIGHTS_E4M3: ptr -> N*K OCP e4m3 bytes [N][K] (one row per output channel), followed at byte
 *     pllm_e4m3_weight_scale_offset(N, K) by N fp32 per-output-channel scales;
 *     pllm_e4m3_weight_bytes(N, K) bytes in all, 16-byte aligned.  N and K keep their meaning.
 *     pllm_quantize_weight_e4m3 writes that form from a device-resident fp16 [K][N] weight
 *     (scale[n] = max_k |w[k][n]| / 448).  The GEMMs then quantise their input rows per launch and
 *     run on the fp8 matrix cores; the QKV bias pipeline types are not available in this format. */
enum nf_weight_format { NF_WEIGHTS_F16 = 0, NF_WEIGHTS_E4M3 = 1 };
NF_PLLM_API int pllm_set_weight_format(int format);
NF_PLLM_API int pllm_get_weight_format(void);
NF_PLLM_API size_t pllm_e4m3_weight_bytes(int N, int K);
NF_PLLM_API size_t pllm_e4m3_weight_scale_offset(int N, int K);
NF_PLLM_API int pllm_quantize_weight_e4m3(const uint16_t* w_f16, void* out, int N, int K, void* stream);

NF_PLLM_API int pllm_set_profiling(int on);
/* Time every stride-th launch of each operator (0 = automatic: 4 on schedules of 8 or more layers,
 * else 1).  Takes effect at the next pllm_set_profiling / pllm_init.  pllm_get_timings reports the
 * stride in use as layer_stride. */
NF_PLLM_API int pllm_set_profiling_stride(int stride);
NF_PLLM_API int pllm_get_timings(nf_pipeline_timings* out);
/* hipGraph replay (the reference carries a graph switch that is compiled off, `constexpr bool
 * enableGraph = false`, pipeline_local.cu:319-327, and only its capture events remain).  With graph mode on, an iteration whose launch signature
 * (decode rows, prefill requests and tokens, the four attention group sizes and block caps) has
 * been seen before is captured once and replayed afterwards; the first occurrence of a
 * signature runs eagerly.  Profiling (level > 0) takes precedence and disables replay.
 * counters = {iterations run eagerly, graphs captured, iterations replayed}. */
NF_PLLM_API int pllm_set_graph_mode(int on);
NF_PLLM_API int pllm_get_graph_counters(long counters[3]);
NF_PLLM_API int pllm_reset_timings(void);
/* Device address of an intermediate of the current pipeline, for parity checks:
 * name in {"hidden" (residual stream after the last layer, [T, hidden]),
 *          "logits" ([T, vocab])}; for PLLMOFFLOAD also "offload_host" (PINNED HOST memory,
 *          [pages moved, halves per page]: what the last layer's offload round trip left); for the non-overlap pipeline also the last layer's operator
 *          inputs and outputs: "ln_attn" (QKV input), "kqv", "attn_out" (O input), "o_out",
 *          "ln_ffn" (gate/up input), "act" (down input). */
NF_PLLM_API int pllm_debug_buffer(const char* name, uint16_t** ptr, int* rows, int* cols);

#ifdef __cplusplus
}
#endif
#endif /* NANOFLOW_PLLM_H */
