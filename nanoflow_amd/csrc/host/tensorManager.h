// TensorManager: device mirrors of the per-iteration update data.
// Interface of the reference's pipeline/include/tensorManager.cuh:7-90.  Differences on
// purpose: the caller's arrays are first copied into pinned staging owned here (so the caller
// may reuse its buffers as soon as update() returns), the host-to-device copies are
// stream-ordered on the pipeline's stream instead of ending in a device-wide synchronise, and
// the staged host copy stays readable so the pipeline can plan without device-to-host reads.
#pragma once
#include <cstring>
#include <vector>

#include "config.h"
#include "helper.h"
#include "vortexData.h"

class TensorManager {
  TensorManager() = default;
  std::vector<vortexUpdateData> gpu_update_datas;
  std::vector<vortexUpdateData> host_update_datas;  // pinned staging, same layout
  int nranks = 0;
  int vnranks = 0;
  bool inited = false;
  size_t cap_batch = 0, cap_pages = 0;  // sizes the mirrors were allocated for

  template <typename T>
  static void alloc_pair(T*& dev, T*& host, size_t n) {
    HIP_CHECK(hipMalloc(&dev, n * sizeof(T)));
    HIP_CHECK(hipMemset(dev, 0, n * sizeof(T)));  // entries past an iteration's live ones stay valid indices
    HIP_CHECK(hipHostMalloc(&host, n * sizeof(T), hipHostMallocDefault));
    std::memset(host, 0, n * sizeof(T));
  }
  template <typename T>
  static void stage(T* host_stage, T* dev, const T* src, size_t n, hipStream_t s) {
    if (n == 0) return;
    std::memcpy(host_stage, src, n * sizeof(T));
    HIP_CHECK(hipMemcpyAsync(dev, host_stage, n * sizeof(T), hipMemcpyHostToDevice, s));
  }

public:
  static TensorManager& getInstance() {
    static TensorManager instance;
    return instance;
  }
  bool isInited() const { return inited; }

  void release() {
    for (size_t i = 0; i < gpu_update_datas.size(); ++i) {
      auto& g = gpu_update_datas[i];
      auto& h = host_update_datas[i];
      int32_t* dev[] = {g.input_tokens, g.input_indptr, g.kv_indptr, g.kv_indices, g.kv_last_page_len,
                        g.per_token_offset, g.rev_input_indptr, g.keep_token_list};
      int32_t* hst[] = {h.input_tokens, h.input_indptr, h.kv_indptr, h.kv_indices, h.kv_last_page_len,
                        h.per_token_offset, h.rev_input_indptr, h.keep_token_list};
      for (auto p : dev) (void)hipFree(p);
      for (auto p : hst) (void)hipHostFree(p);
      delete[] g.gemv_batch_size;
      delete[] g.gemv_num_blocks;
    }
    gpu_update_datas.clear();
    host_update_datas.clear();
    inited = false;
  }

  // Idempotent for an unchanged configuration; reallocates when the limits changed.
  void init(int nranks, int vnranks) {
    if (inited && cap_batch == (size_t)ModelConfig.max_batch_size && cap_pages == ModelConfig.max_page_num)
      return;
    if (inited) release();
    cap_batch = ModelConfig.max_batch_size;
    cap_pages = ModelConfig.max_page_num;
    this->nranks = nranks;
    this->vnranks = vnranks;
    gpu_update_datas.resize(nranks);
    host_update_datas.resize(nranks);
    const size_t mb = ModelConfig.max_batch_size;
    for (int i = 0; i < nranks; i++) {
      HIP_CHECK(hipSetDevice(i));
      auto& g = gpu_update_datas[i];
      auto& h = host_update_datas[i];
      alloc_pair(g.input_tokens, h.input_tokens, mb);
      alloc_pair(g.input_indptr, h.input_indptr, mb + 1);
      alloc_pair(g.kv_indptr, h.kv_indptr, mb + 1);
      alloc_pair(g.kv_indices, h.kv_indices, ModelConfig.max_page_num);
      alloc_pair(g.kv_last_page_len, h.kv_last_page_len, mb);
      alloc_pair(g.per_token_offset, h.per_token_offset, mb);
      alloc_pair(g.rev_input_indptr, h.rev_input_indptr, mb);
      alloc_pair(g.keep_token_list, h.keep_token_list, mb);
      g.gemv_batch_size = new int32_t[4];
      g.gemv_num_blocks = new int32_t[4];
      h.gemv_batch_size = g.gemv_batch_size;
      h.gemv_num_blocks = g.gemv_num_blocks;
    }
    inited = true;
  }

  // Validates sizes against the mirrors; returns nullptr (with a logged error) when the
  // iteration does not fit.
  vortexUpdateData* update_data_to_gpu(const vortexUpdateData& u, int rank, hipStream_t s) {
    auto& g = gpu_update_datas[rank];
    auto& h = host_update_datas[rank];
    const int total_batch = u.decodePrefillBorder + u.prefillNum;
    const int total_token = u.input_indptr[total_batch];
    const int used_pages = u.kv_indptr[total_batch];
    if (total_batch > ModelConfig.max_batch_size || total_token > ModelConfig.max_batch_size ||
        (size_t)used_pages > ModelConfig.max_page_num ||
        u.keepTokenListLength > ModelConfig.max_batch_size ||
        total_token != u.decodePrefillBorder + u.prefillTokensNum) {
      NF_LOG_ERROR("update data does not fit: requests %d tokens %d (max %d), pages %d (max %zu), "
                   "border %d + prefill tokens %d",
                   total_batch, total_token, ModelConfig.max_batch_size, used_pages,
                   ModelConfig.max_page_num, u.decodePrefillBorder, u.prefillTokensNum);
      return nullptr;
    }
    g.decodePrefillBorder = h.decodePrefillBorder = u.decodePrefillBorder;
    g.prefillNum = h.prefillNum = u.prefillNum;
    g.prefillTokensNum = h.prefillTokensNum = u.prefillTokensNum;
    g.keepTokenListLength = h.keepTokenListLength = u.keepTokenListLength;
    stage(h.input_tokens, g.input_tokens, u.input_tokens, total_token, s);
    stage(h.input_indptr, g.input_indptr, u.input_indptr, total_batch + 1, s);
    stage(h.kv_indptr, g.kv_indptr, u.kv_indptr, total_batch + 1, s);
    stage(h.kv_indices, g.kv_indices, u.kv_indices, used_pages, s);
    stage(h.kv_last_page_len, g.kv_last_page_len, u.kv_last_page_len, total_batch, s);
    std::memcpy(g.gemv_batch_size, u.gemv_batch_size, 4 * sizeof(int32_t));
    std::memcpy(g.gemv_num_blocks, u.gemv_num_blocks, 4 * sizeof(int32_t));
    stage(h.per_token_offset, g.per_token_offset, u.per_token_offset, total_token, s);
    stage(h.rev_input_indptr, g.rev_input_indptr, u.rev_input_indptr, total_token, s);
    stage(h.keep_token_list, g.keep_token_list, u.keep_token_list, u.keepTokenListLength, s);
    return &g;
  }

  // Host-side copy of the last update of this rank (valid until the next update).
  const vortexUpdateData& host_data(int rank) const { return host_update_datas[rank]; }
};
