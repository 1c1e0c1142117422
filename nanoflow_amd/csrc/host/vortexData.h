// Plain structs crossing the caller <-> pipeline boundary.  Field order and meaning are the
// reference's (pipeline/include/vortexData.cuh:7-111); `half` is the fp16 bit pattern.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "tensor.h"

struct vortexWeight {
  half* ptr = nullptr;
  int N = 0;
  int K = 0;
  size_t size() const { return (size_t)N * K; }
};

// Storage of the five per-layer GEMM weights (W_KQV, W_O1/W_O2, W_G, W_U, W_D); embedding, norms,
// B_KQV and the LM head are fp16 in both.  The reference knows fp16 only.
//   F16:  ptr -> fp16 [K][N] row-major (K = input features), as in the reference.
//   E4M3: ptr -> N*K OCP e4m3 bytes [N][K] (one row per output channel, k contiguous), followed at
//         byte e4m3WeightScaleOffset(N, K) by N fp32 per-output-channel scales
//         (w[k][n] ~ scale[n] * e4m3[n][k]); e4m3WeightBytes(N, K) bytes in all, 16-byte aligned.
//         N and K keep their meaning, so size() still checks the shape.
enum class WeightFormat { F16 = 0, E4M3 = 1 };
inline size_t e4m3WeightScaleOffset(size_t N, size_t K) { return (N * K + 255) / 256 * 256; }
inline size_t e4m3WeightBytes(size_t N, size_t K) { return e4m3WeightScaleOffset(N, K) + N * sizeof(float); }

// The format of the init data the next init() is given (process-wide, F16 unless set).
void setWeightFormat(WeightFormat format);
WeightFormat getWeightFormat();

struct vortexLayerWeight {
  vortexWeight W_O1, W_O2, W_U, W_G, W_D, W_KQV, B_KQV, W_LN_Attention, W_LN_FFN, W_ROT;
};

struct vortexModelWeight {
  vortexWeight lm_head;
  vortexWeight embedding;
  vortexWeight model_layernorm;
  std::vector<vortexLayerWeight> layer_weight;
};

struct vortexInitData {
  half** kv_data = nullptr;  // per layer: [max_pages, 2, page_size, num_head, head_dim]
  vortexModelWeight weight;  // device pointers
  size_t weight_size = 0;
  half* tmp_buffer = nullptr;  // device
  size_t tmp_buffer_size = 0;  // in halves
};

struct vortexUpdateData {
  int decodePrefillBorder = 0;  // rows [border, end) of the dense batch are prefill tokens
  int prefillNum = 0;           // prefill requests
  int prefillTokensNum = 0;     // prefill tokens
  int keepTokenListLength = 0;
  int* input_tokens = nullptr;
  int32_t* input_indptr = nullptr;      // [req+1]
  int32_t* rev_input_indptr = nullptr;  // [tokens] request of each token
  int32_t* keep_token_list = nullptr;   // [keepTokenListLength] 1 = slot keeps decoding
  int32_t* kv_indptr = nullptr;         // [req+1]
  int32_t* kv_indices = nullptr;        // [used pages]
  int32_t* kv_last_page_len = nullptr;  // [req]
  int32_t* per_token_offset = nullptr;  // [tokens] position of each token in its request
  int32_t* gemv_batch_size = nullptr;   // host, [4]
  int32_t* gemv_num_blocks = nullptr;   // host, [4]
};

struct vortexOutputData {
  int32_t* sampled_token_array = nullptr;  // host, one token per request
  int sampled_tokens = 0;
  half* offload_kv_cache = nullptr;
  int global_batch_size = 0;
};

struct vortexConfigData {
  std::vector<std::string> gemm_op_tag;
  int global_batch_size = 0;
  int nanobatch_1_size = 0;
  int kqv1_size = 0;
  int kqv3_size = 0;
};

// Builders used by the synthetic end-to-end run (reference: pipeline/src/vortexData.cu).
vortexModelWeight modelWeightToGPU(vortexModelWeight& modelWeight, int rank);
void createInitData(vortexInitData& data, vortexModelWeight& weight, int rank);
void createUpdateData(vortexUpdateData& data, int rank, int global_batch_size, int avg_prefill_length,
                      int avg_decode_length);
void createModelWeight(vortexModelWeight& data, int rank);
void createModelWeightCPU(vortexModelWeight& data, int rank);
void allocateKVData(vortexInitData& data, int rank);
bool readConfigData(vortexConfigData& data, int rank, const std::string& filename);
