// Row-wise operators of the pipeline: RMSNorm, embedding gather, split+RoPE+paged-KV append,
// last-token gather, greedy sampler.  Interfaces of pipeline/include/otherWrapper.cuh:17-540
// (only the operators the single-device pipelines use).
#pragma once
#include "config.h"
#include "nanoflow_kernels.h"
#include "operatorWrapper.h"
#include "vortexData.h"

class OtherWrapper : public OperatorWrapper {};

// input_size / output_size == I_O_Ratio
template <size_t I_O_Ratio = 1>
class VectorOpWrapper : public OtherWrapper {
public:
  using Element = half;
  Element* input = nullptr;
  Element* output = nullptr;
  pllmTensor<Element> pllm_tensor_input, pllm_tensor_output;
  size_t input_size = 0, output_size = 0;

  VectorOpWrapper& setInput(pllmTensor<Element> t) {
    input = t.ptr;
    input_size = t.size();
    pllm_tensor_input = t;
    assert(output_size == 0 || input_size == output_size * I_O_Ratio);
    return *this;
  }
  VectorOpWrapper& setOutput(pllmTensor<Element> t) {
    output = t.ptr;
    output_size = t.size();
    pllm_tensor_output = t;
    assert(input_size == 0 || input_size == output_size * I_O_Ratio);
    return *this;
  }
  pllmTensor<Element> getOutput() { return pllm_tensor_output; }
  pllmTensor<Element> getInput() { return pllm_tensor_input; }
  OperatorWrapper& logImpl() override {
    logTensor("input", pllm_tensor_input, 10, 20);
    logTensor("output", pllm_tensor_output, 10, 20);
    return *this;
  }
};

// RMSNorm over rows of model_hidden_dim (the reference's class name is LayerNorm).
class LayerNorm : public VectorOpWrapper<1> {
public:
  Element* weight = nullptr;
  pllmTensor<half> pllm_tensor_weight;

  LayerNorm& setWeight(Element* w) {
    weight = w;
    return *this;
  }
  bool setWeight(vortexWeight w) {
    weight = w.ptr;
    pllm_tensor_weight = pllmTensor<half>(w.ptr, size_t(1), w.size(), PllmLayout::ROW_MAJOR);
    return true;
  }
  OperatorWrapper& logImpl() override {
    logTensor("weight", pllm_tensor_weight, 1, 20);
    logTensor("input", pllm_tensor_input, 10, 20);
    logTensor("output", pllm_tensor_output, 10, 20);
    return *this;
  }
  // rows that hold tokens in this iteration (-1: all rows of the input); the rest is left as it was
  int live_rows = -1;
  void set_live_rows(int r) { live_rows = r; }
  // Not in the reference's interface: the output rows also as e4m3 bytes [rows, hidden] with one
  // fp32 scale per row, for a consumer GEMM on e4m3 weights (BaseGEMMWrapper::setQuantizedA); the
  // fp16 output is written all the same.  Hidden sizes the fused kernel does not take are refused.
  uint8_t* output_q = nullptr;
  float* output_q_scale = nullptr;
  static bool canQuantize() { return ModelConfig.model_hidden_dim % 16 == 0 && ModelConfig.model_hidden_dim <= 8192; }
  bool setQuantOutput(uint8_t* q, float* scale) {
    if (!canQuantize() || !q || !scale) return false;
    output_q = q;
    output_q_scale = scale;
    return true;
  }
  void work() override {
    assert(pllm_tensor_input.dim2 == (size_t)ModelConfig.model_hidden_dim);
    const int all = (int)(input_size / ModelConfig.model_hidden_dim);
    const int rows = live_rows >= 0 && live_rows < all ? live_rows : all;
    if (output_q) {
      NF_KERNEL_CHECK(nf_rmsnorm_quantize_e4m3(output, input, weight, output_q, output_q_scale, rows,
                                               ModelConfig.model_hidden_dim, ModelConfig.rms_norm_eps, stream));
      return;
    }
    NF_KERNEL_CHECK(nf_rmsnorm_f16(output, input, weight, rows, ModelConfig.model_hidden_dim,
                                   ModelConfig.rms_norm_eps, stream));
  }
};

class GenEmbedding : public OtherWrapper {
public:
  half* weight = nullptr;
  int* tokens = nullptr;
  half* output = nullptr;
  pllmTensor<int> pllm_tensor_tokens;
  pllmTensor<half> pllm_tensor_output, pllm_tensor_weight;
  int input_size = 0, output_size = 0;

  bool setWeight(vortexWeight w) {
    weight = w.ptr;
    pllm_tensor_weight = pllmTensor<half>(w.ptr, w.K, w.N, PllmLayout::ROW_MAJOR);
    return true;
  }
  void setInput(pllmTensor<int> t) {
    tokens = t.ptr;
    input_size = (int)t.size();
    pllm_tensor_tokens = t;
    if (output_size) assert(input_size * ModelConfig.model_hidden_dim == output_size);
  }
  pllmTensor<half> getOutput() { return pllm_tensor_output; }
  void setOutput(pllmTensor<half> o) {
    output = o.ptr;
    output_size = (int)o.size();
    pllm_tensor_output = o;
    if (input_size) assert(input_size * ModelConfig.model_hidden_dim == output_size);
  }
  // rows that hold tokens in this iteration (-1: all); ids beyond them are not uploaded, so
  // their rows are left as they were
  int live_rows = -1;
  void set_live_rows(int r) { live_rows = r; }
  void work() override {
    const int rows = live_rows >= 0 && live_rows < input_size ? live_rows : input_size;
    if (rows == 0) return;
    NF_KERNEL_CHECK(nf_embedding_f16(tokens, weight, output, rows, ModelConfig.model_hidden_dim, stream));
  }
  OperatorWrapper& logImpl() override {
    logTensor("weight", pllm_tensor_weight, 1, 20);
    logTensor("tokens", pllm_tensor_tokens, 1, 20);
    logTensor("output", pllm_tensor_output, 10, 20);
    return *this;
  }
};

// The smaller operators of the reference's vocabulary (pipeline/include/otherWrapper.cuh:183-301,
// 395-412, 542-568).  The single-device schedules do not use them (the gate/up pair is fused, nothing
// is exchanged between ranks); they are here for schedules written against the reference's interface.

// kqv [rows, k_dim + q_dim + v_dim] copied apart into k, q, v (in that column order).
class SplitKQVOutput : public OtherWrapper {
public:
  half* kqv = nullptr;
  half* k = nullptr;
  half* q = nullptr;
  half* v = nullptr;
  pllmTensor<half> pllm_tensor_kqv, pllm_tensor_k, pllm_tensor_q, pllm_tensor_v;
  int k_dim = 0, q_dim = 0, v_dim = 0, batch_size = 0;

  void init(pllmTensor<half> kqv, pllmTensor<half> k, pllmTensor<half> q, pllmTensor<half> v, int batch_size, int k_dim,
            int q_dim, int v_dim) {
    assert((int)k.dimC() == k_dim && (int)q.dimC() == q_dim && (int)v.dimC() == v_dim);
    pllm_tensor_kqv = kqv;
    pllm_tensor_k = k;
    pllm_tensor_q = q;
    pllm_tensor_v = v;
    this->kqv = kqv.ptr;
    this->k = k.ptr;
    this->q = q.ptr;
    this->v = v.ptr;
    this->k_dim = k_dim;
    this->q_dim = q_dim;
    this->v_dim = v_dim;
    this->batch_size = batch_size;
  }
  void work() override {
    NF_KERNEL_CHECK(nf_split_kqv_f16(kqv, k, q, v, batch_size, k_dim, q_dim, v_dim, stream));
  }
  OperatorWrapper& logImpl() override {
    logTensor("kqv", pllm_tensor_kqv, 10, 20);
    logTensor("k", pllm_tensor_k, 10, 20);
    logTensor("q", pllm_tensor_q, 10, 20);
    logTensor("v", pllm_tensor_v, 10, 20);
    return *this;
  }
};

// output [M, N] = the rank's N columns of input [M, nranks * N].
class SplitTensor : public OtherWrapper {
public:
  pllmTensor<half> input, output;
  int nranks = 1, rank = 0, N = 0;

  void init(pllmTensor<half> input, pllmTensor<half> output, int nranks, int rank) {
    this->input = input;
    this->output = output;
    this->nranks = nranks;
    this->rank = rank;
    this->N = (int)output.dim2;
  }
  void work() override {
    NF_KERNEL_CHECK(nf_extract_rank_columns_f16(input.ptr, output.ptr, (int)input.dim1, N, nranks, rank, stream));
  }
  OperatorWrapper& logImpl() override {
    logTensor("input", input, 10, 20);
    logTensor("output", output, 10, 20);
    return *this;
  }
};

// output [M, N] = input[:, :N] * silu(input[:, N:]) of input [M, 2 N]: the activation between separate
// gate / up and down projections (the schedules here use the fused pair, DualWrapper, instead).
class Activation : public VectorOpWrapper<2> {
  int M = 0, N = 0;

public:
  void init(Element* input, Element* output, int input_size, int output_size) {
    this->input = input;
    this->output = output;
    this->input_size = input_size;
    this->output_size = output_size;
  }
  void config(int M, int N) {
    this->M = M;
    this->N = N;
  }
  void work() override { NF_KERNEL_CHECK(nf_silu_mul_f16(input, output, M, N, stream)); }
};

// Occupies its stream for a while: a stand-in operator for experiments with schedules.
class SleepWrapper : public OtherWrapper {
public:
  void work() override { NF_KERNEL_CHECK(nf_sleep_us(10, stream)); }
  void sleep(hipStream_t stream, int us = 10) { NF_KERNEL_CHECK(nf_sleep_us(us, stream)); }
};

// output [cols, rows] = input [rows, cols] transposed; the two tensors carry opposite layouts.
class Transpose : public VectorOpWrapper<1> {
  int rows = 0, cols = 0;

public:
  void config(int rows, int cols) {
    this->rows = rows;
    this->cols = cols;
  }
  void work() override {
    assert(static_cast<int>(getInput().layout) == 1 - static_cast<int>(getOutput().layout));
    NF_KERNEL_CHECK(nf_transpose_f16(input, output, rows, cols, stream));
  }
};

class CopyTensor : public OtherWrapper {
public:
  pllmTensor<half> input, output;

  void work() override {
    if (input.size())
      HIP_CHECK(hipMemcpyAsync(output.ptr, input.ptr, input.size() * sizeof(half), hipMemcpyDeviceToDevice, stream));
  }
  OperatorWrapper& logImpl() override {
    logTensor("input", input, 10, 20);
    logTensor("output", output, 10, 20);
    return *this;
  }
  CopyTensor& setOutput(pllmTensor<half> output) {
    this->output = output;
    return *this;
  }
  CopyTensor& setInput(pllmTensor<half> input) {
    this->input = input;
    return *this;
  }
};

class RoPEAppend : public OtherWrapper {
public:
  pllmTensor<half> kqv_input, q_out;
  pllmTensor<int32_t> rev_input_indptr, per_token_offset;
  int dense_batch_size = 0;
  pllmTensor<half> kv_data;
  pllmTensor<int32_t> kv_indices, kv_indptr, kv_last_page_len;
  int* kqv_ready_counter = nullptr;

  void setKVData(half* kv) {
    kv_data = pllmTensor<half>(kv, size_t(ModelConfig.max_page_num * ModelConfig.frame_page_size * 2),
                               size_t(ModelConfig.model_head_dim * ModelConfig.model_kv_heads_gpu),
                               PllmLayout::ROW_MAJOR);
  }
  void setKVData(pllmTensor<half> kv) { kv_data = kv; }

  // kqv_input / q_out / rev_input_indptr / per_token_offset are the nano-batch's slices;
  // the kv_* arrays are the whole iteration's.
  void update(int dense_batch_size, pllmTensor<half> kqv_input, pllmTensor<half> q_out,
              pllmTensor<int32_t> rev_input_indptr, pllmTensor<int32_t> per_token_offset,
              pllmTensor<int32_t> kv_indices, pllmTensor<int32_t> kv_indptr,
              pllmTensor<int32_t> kv_last_page_len, int* kqv_ready_counter = nullptr) {
    this->kqv_input = kqv_input;
    this->q_out = q_out;
    this->rev_input_indptr = rev_input_indptr;
    this->per_token_offset = per_token_offset;
    this->dense_batch_size = dense_batch_size;
    this->kv_indices = kv_indices;
    this->kv_indptr = kv_indptr;
    this->kv_last_page_len = kv_last_page_len;
    this->kqv_ready_counter = kqv_ready_counter;
  }
  void work() override {
    NF_KERNEL_CHECK(nf_rope_append_f16(
        kqv_input.ptr, q_out.ptr, kv_data.ptr, kv_indices.ptr, kv_indptr.ptr, rev_input_indptr.ptr,
        per_token_offset.ptr, dense_batch_size, ModelConfig.model_qo_heads_gpu,
        ModelConfig.model_kv_heads_gpu, ModelConfig.model_head_dim, ModelConfig.frame_page_size,
        ModelConfig.factor, ModelConfig.rope_theta, ModelConfig.smooth_a, ModelConfig.smooth_b,
        stream));
  }
  OperatorWrapper& logImpl() override {
    logTensor("kqv", kqv_input, 10, 20);
    logTensor("q_out", q_out, 10, 20);
    logTensor("rev_input_indptr", rev_input_indptr, 1, 512);
    logTensor("per_token_offset", per_token_offset, 1, 512);
    logTensor("kv_indices", kv_indices, 1, 512);
    logTensor("kv_indptr", kv_indptr, 1, 512);
    logTensor("kv_last_page_len", kv_last_page_len, 1, 512);
    return *this;
  }
};

class MaxSampling : public OtherWrapper {
public:
  pllmTensor<half> d_matrix, d_maxVals;
  pllmTensor<int> d_argMax;
  int batch_size = 0;

  void init(pllmTensor<half> d_matrix, pllmTensor<half> d_maxVals, pllmTensor<int> d_argMax) {
    this->d_matrix = d_matrix;
    this->d_maxVals = d_maxVals;
    this->d_argMax = d_argMax;
  }
  void work() override {
    NF_KERNEL_CHECK(nf_argmax_f16(d_matrix.ptr, d_maxVals.ptr, d_argMax.ptr, batch_size,
                                  (int)d_matrix.dim2, stream));
  }
  OperatorWrapper& set_batch_size(int b) {
    batch_size = b;
    return *this;
  }
  OperatorWrapper& logImpl() override {
    logTensor("d_matrix", d_matrix, 10, 20);
    logTensor("d_maxVals", d_maxVals, 1, 20);
    logTensor("d_argMax", d_argMax, 1, (size_t)batch_size);
    return *this;
  }
};

class KeepToken : public OtherWrapper {
public:
  int req_num = 0;
  pllmTensor<half> input, output;
  int32_t* input_indptr = nullptr;

  void update(int req_num, int32_t* input_indptr) {
    this->req_num = req_num;
    this->input_indptr = input_indptr;
  }
  void work() override {
    NF_KERNEL_CHECK(nf_keep_token_f16(input.ptr, output.ptr, input_indptr, req_num,
                                      (int)input.dim2, stream));
  }
  KeepToken& setOutput(pllmTensor<half> o) {
    output = o;
    return *this;
  }
  KeepToken& setInput(pllmTensor<half> i) {
    input = i;
    return *this;
  }
  OperatorWrapper& logImpl() override {
    logTensor("input", input, 10, 20);
    logTensor("output", output, 10, 20);
    return *this;
  }
};

// KV offload operators (pipeline/include/otherWrapper.cuh:413-472).  PageAggregator gathers the
// pages of the listed (finished) requests from one layer's pool into a staging buffer laid out
// like kv_indices, ready for one contiguous copy to host memory; PageDispatcher scatters a staging
// buffer loaded from host memory back into the pages the requests now own.  The reference wires
// them only into its tensor-parallel offload pipeline, with fixed request lists as a cost model
// (pipeline/src/pipeline.cu:37-59,701-726,915-931); here they are free-standing operators.
class PageAggregator : public OtherWrapper {
public:
  int finished_req_num = 0;
  int32_t* finished_idx = nullptr;
  int32_t* kv_indptr = nullptr;
  int32_t* kv_indices = nullptr;
  half* output = nullptr;
  half* kv_data = nullptr;

  void init(int finished_req_num, int32_t* finished_idx, int32_t* kv_indptr, int32_t* kv_indices, half* output) {
    this->finished_req_num = finished_req_num;
    this->finished_idx = finished_idx;
    this->kv_indptr = kv_indptr;
    this->kv_indices = kv_indices;
    this->output = output;
  }
  void setKVData(half* kv_data) { this->kv_data = kv_data; }
  void work() override {
    NF_KERNEL_CHECK(nf_move_kv_pages(finished_req_num, finished_idx, kv_indptr, kv_indices, output, kv_data,
                                     ModelConfig.page_mem_size, 0, stream));
  }
};

class PageDispatcher : public OtherWrapper {
public:
  int load_req_num = 0;
  int32_t* load_idx = nullptr;
  int32_t* kv_indptr = nullptr;
  int32_t* kv_indices = nullptr;
  half* host_input = nullptr;  // the staging buffer the host copy was loaded into (device memory)
  half* kv_data = nullptr;

  void init(int load_req_num, int32_t* load_idx, int32_t* kv_indptr, int32_t* kv_indices, half* host_input) {
    this->load_req_num = load_req_num;
    this->load_idx = load_idx;
    this->kv_indptr = kv_indptr;
    this->kv_indices = kv_indices;
    this->host_input = host_input;
  }
  void setKVData(half* kv_data) { this->kv_data = kv_data; }
  void work() override {
    NF_KERNEL_CHECK(nf_move_kv_pages(load_req_num, load_idx, kv_indptr, kv_indices, host_input, kv_data,
                                     ModelConfig.page_mem_size, 1, stream));
  }
};
