// Attention operators ("GEMV" in the reference's vocabulary = decode attention).
// Interfaces of pipeline/include/gemvWrapper.cuh:17-385.  Planning that the reference does on
// the host in init() (BatchPrefillHandler::BeginForward plus its H2D copies) happens inside
// the kernel layer on the device, so init() only records arguments and never synchronises.
#pragma once
#include "config.h"
#include "nanoflow_kernels.h"
#include "operatorWrapper.h"

class GemvWrapper : public OperatorWrapper {
public:
  using Element = half;
  uint32_t batch_size = 0;
  int32_t block_num = 0;

  Element* kv_data = nullptr;           // [max_pages, 2, page_size, num_head, head_dim]
  int32_t* kv_indptr = nullptr;         // [batch_size + 1]
  int32_t* kv_indices = nullptr;        // [used_pages]
  int32_t* kv_last_page_len = nullptr;  // [batch_size]
  int32_t* qo_indptr = nullptr;         // [batch_size + 1], absolute rows of q / o
  Element* q = nullptr;
  Element* o = nullptr;

  pllmTensor<int32_t> qo_indptr_tensor, kv_indptr_tensor, kv_last_page_len_tensor;
  pllmTensor<half> input_tensor, output_tensor;
  int* device_KQV_ready = nullptr;   // accepted for interface parity; unused
  int* device_GEMV_ready = nullptr;

  GemvWrapper(bool causal) : OperatorWrapper(false, true), causal_(causal) {
    workspace_bytes_ = nf_attention_workspace_bytes(ModelConfig.max_batch_size + 1,
                                                    ModelConfig.max_batch_size,
                                                    ModelConfig.model_qo_heads_gpu);
    HIP_CHECK(hipMalloc(&workspace_, workspace_bytes_));
  }
  ~GemvWrapper() override { (void)hipFree(workspace_); }

  void setKVData(Element* kv) { kv_data = kv; }

  static size_t getInputSize(uint32_t batch_size) {
    return (size_t)(2 * ModelConfig.model_kv_heads_gpu + ModelConfig.model_qo_heads_gpu) *
           ModelConfig.model_head_dim * batch_size;
  }
  static size_t getOutputSize(uint32_t batch_size) {
    return (size_t)ModelConfig.model_qo_heads_gpu * ModelConfig.model_head_dim * batch_size;
  }

  void init(uint32_t batch_size, int32_t block_num, pllmTensor<int32_t> qo_indptr,
            pllmTensor<int32_t> kv_indptr, int32_t* kv_indices,
            pllmTensor<int32_t> kv_last_page_len, pllmTensor<half> input, pllmTensor<half> output,
            int* device_KQV_ready = nullptr, int* device_GEMV_ready = nullptr) {
    this->batch_size = batch_size;
    this->block_num = block_num;
    assert(kv_indptr.layout == PllmLayout::ROW_MAJOR);
    assert(batch_size == 0 || kv_indptr.size() == batch_size + 1);
    assert(batch_size == 0 || kv_last_page_len.size() == batch_size);
    assert(input.size() == 0 ||
           input.dim2 == (size_t)ModelConfig.model_qo_heads_gpu * ModelConfig.model_head_dim);
    this->kv_indptr = kv_indptr.ptr;
    this->kv_indices = kv_indices;
    this->kv_last_page_len = kv_last_page_len.ptr;
    this->qo_indptr = qo_indptr.ptr;
    this->q = input.ptr;
    this->o = output.ptr;
    this->device_KQV_ready = device_KQV_ready;
    this->device_GEMV_ready = device_GEMV_ready;
    qo_indptr_tensor = qo_indptr;
    kv_indptr_tensor = kv_indptr;
    kv_last_page_len_tensor = kv_last_page_len;
    input_tensor = input;
    output_tensor = output;
    // q/o are passed as the base of the whole iteration buffer, so any dense-batch row may
    // be addressed: bound the launch by the largest dense batch.
    max_rows_ = ModelConfig.max_batch_size;
  }

  void work() override {
    // decode: one row per request; prefill: at most every row of the shared q buffer
    const int max_rows = causal_ ? max_rows_ : (int)batch_size;
    int rc = nf_attention_paged_f16(q, o, qo_indptr, kv_data, kv_indptr, kv_indices,
                                    kv_last_page_len, (int)batch_size, max_rows,
                                    ModelConfig.model_qo_heads_gpu, ModelConfig.model_kv_heads_gpu,
                                    ModelConfig.model_head_dim, ModelConfig.frame_page_size,
                                    causal_ ? 1 : 0, causal_ ? 0 : block_num, workspace_,
                                    workspace_bytes_, stream);
    if (rc != 0)  // the reference throws on an attention failure (gemvWrapper.cuh:195-200)
      throw std::invalid_argument(std::string("paged attention failed with error: ") +
                                  nf_last_error());
  }

  OperatorWrapper& logImpl() override {
    logTensor("kv_indptr", kv_indptr_tensor, 1, 20);
    logTensor("kv_last_page_len", kv_last_page_len_tensor, 1, 20);
    logTensor("input", input_tensor, 10, 20);
    logTensor("output", output_tensor, 10, 20);
    return *this;
  }

private:
  bool causal_;
  int max_rows_ = 0;
  void* workspace_ = nullptr;
  size_t workspace_bytes_ = 0;
};

// Decode attention: non-causal, one query row per request, workgroup count capped by
// block_num (the reference's sm_blk knob).
class DecodeGemvWrapper : public GemvWrapper {
public:
  DecodeGemvWrapper() : GemvWrapper(false) {}
};

// Chunked-prefill attention: causal with the kv_len - qo_len offset; block_num is ignored
// (the reference launches these with all blocks).
class PrefillGemvWrapper : public GemvWrapper {
public:
  PrefillGemvWrapper() : GemvWrapper(true) {}
};
