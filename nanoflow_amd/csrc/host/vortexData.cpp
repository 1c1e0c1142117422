// Synthetic data builders for the end-to-end run (reference: pipeline/src/vortexData.cu).
#include "vortexData.h"

#include <cstring>

#include "config.h"
#include "helper.h"
#include "mini_json.h"

void allocateKVData(vortexInitData& data, int rank) {
  HIP_CHECK(hipSetDevice(rank));
  const size_t page_halves = (size_t)2 * ModelConfig.model_kv_heads_gpu * ModelConfig.frame_page_size *
                             ModelConfig.model_head_dim;
  const size_t num_pages = ModelConfig.max_page_num;
  half** kv_datas = new half*[ModelConfig.model_layer];
  NF_LOG_INFO("allocate kv data: %.2f GB", num_pages * page_halves * 2.0 * ModelConfig.model_layer / 1e9);
  for (int i = 0; i < ModelConfig.model_layer; i++) {
    HIP_CHECK(hipMalloc(&kv_datas[i], num_pages * page_halves * sizeof(half)));
    // zero-fill: unwritten entries must at least be finite numbers
    HIP_CHECK(hipMemset(kv_datas[i], 0, num_pages * page_halves * sizeof(half)));
  }
  data.kv_data = kv_datas;
}

void createInitData(vortexInitData& data, vortexModelWeight& weight, int rank) {
  HIP_CHECK(hipSetDevice(rank));
  half* temp = nullptr;
  const size_t kTempSize = ModelConfig.k_temp_size;
  HIP_CHECK(hipMalloc(&temp, kTempSize * sizeof(half)));
  data.weight = weight;
  data.weight_size = (size_t)ModelConfig.model_hidden_dim * ModelConfig.model_hidden_dim * 3;
  data.tmp_buffer = temp;
  data.tmp_buffer_size = kTempSize;
  allocateKVData(data, rank);
}

static vortexWeight device_weight(int N, int K) {
  vortexWeight w;
  w.N = N;
  w.K = K;
  HIP_CHECK(hipMalloc(&w.ptr, w.size() * sizeof(half)));
  HIP_CHECK(hipMemset(w.ptr, 0, w.size() * sizeof(half)));
  return w;
}
// One of the five per-layer GEMM weights in the current weight format (zero-filled).
static vortexWeight device_gemm_weight(int N, int K) {
  if (getWeightFormat() != WeightFormat::E4M3) return device_weight(N, K);
  vortexWeight w;
  w.N = N;
  w.K = K;
  const size_t bytes = e4m3WeightBytes((size_t)N, (size_t)K);
  HIP_CHECK(hipMalloc(&w.ptr, bytes));
  HIP_CHECK(hipMemset(w.ptr, 0, bytes));
  return w;
}
static vortexWeight host_weight(int N, int K) {
  vortexWeight w;
  w.N = N;
  w.K = K;
  w.ptr = new half[w.size()]();
  return w;
}
static vortexWeight host_gemm_weight(int N, int K) {
  if (getWeightFormat() != WeightFormat::E4M3) return host_weight(N, K);
  vortexWeight w;
  w.N = N;
  w.K = K;
  w.ptr = new half[(e4m3WeightBytes((size_t)N, (size_t)K) + 1) / 2]();
  return w;
}

template <typename MakeWeight, typename MakeGemmWeight>
static void fill_model_weight(vortexModelWeight& data, MakeWeight make, MakeGemmWeight make_gemm) {
  const int H = ModelConfig.model_hidden_dim, Hg = ModelConfig.model_hidden_dim_pergpu;
  const int F = ModelConfig.model_ff_dim_gpu;
  const int kqv_n = (2 * ModelConfig.model_kv_heads_gpu + ModelConfig.model_qo_heads_gpu) *
                    ModelConfig.model_head_dim;
  // (N, K) pairs as the reference's createModelWeight passes them; only N*K is checked
  data.lm_head = make(H, (int)ModelConfig.vocab_size);
  data.embedding = make((int)ModelConfig.vocab_size, H);
  data.model_layernorm = make(H, 1);
  data.layer_weight.resize(ModelConfig.model_layer);
  for (auto& lw : data.layer_weight) {
    lw.W_O1 = make_gemm(Hg, H);
    lw.W_O2 = make_gemm(H, Hg);
    lw.W_U = make_gemm(F, H);
    lw.W_G = make_gemm(F, H);
    lw.W_D = make_gemm(H, F);
    lw.W_KQV = make_gemm(kqv_n, H);
    lw.B_KQV = make(1, kqv_n);
    lw.W_LN_Attention = make(H, 1);
    lw.W_LN_FFN = make(H, 1);
    lw.W_ROT = make(64, 1);
  }
}

void createModelWeight(vortexModelWeight& data, int rank) {
  HIP_CHECK(hipSetDevice(rank));
  fill_model_weight(data, device_weight, device_gemm_weight);
}
void createModelWeightCPU(vortexModelWeight& data, int rank) {
  (void)rank;
  fill_model_weight(data, host_weight, host_gemm_weight);
}

static vortexWeight upload(const vortexWeight& h, bool gemm_weight = false) {
  vortexWeight d = h;
  if (!h.ptr || h.size() == 0) return d;
  const size_t bytes = gemm_weight && getWeightFormat() == WeightFormat::E4M3
                           ? e4m3WeightBytes((size_t)h.N, (size_t)h.K)
                           : h.size() * sizeof(half);
  HIP_CHECK(hipMalloc(&d.ptr, bytes));
  HIP_CHECK(hipMemcpy(d.ptr, h.ptr, bytes, hipMemcpyHostToDevice));
  return d;
}

vortexModelWeight modelWeightToGPU(vortexModelWeight& hw, int rank) {
  HIP_CHECK(hipSetDevice(rank));
  vortexModelWeight d;
  d.lm_head = upload(hw.lm_head);
  d.embedding = upload(hw.embedding);
  d.model_layernorm = upload(hw.model_layernorm);
  d.layer_weight.resize(hw.layer_weight.size());
  for (size_t i = 0; i < hw.layer_weight.size(); ++i) {
    const auto& s = hw.layer_weight[i];
    auto& t = d.layer_weight[i];
    t.W_O1 = upload(s.W_O1, true);
    t.W_O2 = s.W_O2.ptr == s.W_O1.ptr ? t.W_O1 : upload(s.W_O2, true);
    t.W_U = upload(s.W_U, true);
    t.W_G = upload(s.W_G, true);
    t.W_D = upload(s.W_D, true);
    t.W_KQV = upload(s.W_KQV, true);
    t.B_KQV = upload(s.B_KQV);
    t.W_LN_Attention = upload(s.W_LN_Attention);
    t.W_LN_FFN = upload(s.W_LN_FFN);
    t.W_ROT = upload(s.W_ROT);
  }
  return d;
}

template <typename T>
static T* pinned_copy(const std::vector<T>& v, size_t min_elems = 1) {
  T* p = nullptr;
  HIP_CHECK(hipHostMalloc(&p, std::max(v.size(), min_elems) * sizeof(T), hipHostMallocDefault));
  if (!v.empty()) std::memcpy(p, v.data(), v.size() * sizeof(T));
  return p;
}

// A self-consistent synthetic iteration: decode requests with a full 1024-token history and
// prefill chunks starting at position 0, contiguous page ids.  Same split of the dense batch
// as the reference (decode share = avg_decode / (avg_decode + avg_prefill) of the batch,
// prefill requests of avg_prefill_length tokens, pipeline/src/vortexData.cu:61-204); unlike
// the reference the append positions and KV lengths agree with each other.
void createUpdateData(vortexUpdateData& data, int rank, int global_batch_size, int avg_prefill_length,
                      int avg_decode_length) {
  HIP_CHECK(hipSetDevice(rank));
  const int page = ModelConfig.frame_page_size;
  const int dpb = static_cast<int>(global_batch_size * static_cast<float>(avg_decode_length) /
                                   (avg_decode_length + avg_prefill_length));
  const int prefillNum = (global_batch_size - dpb + avg_prefill_length - 1) / avg_prefill_length;
  std::vector<int32_t> qo_len(dpb, 1);
  for (int i = 0; i < prefillNum - 1; i++) qo_len.push_back(avg_prefill_length);
  if (prefillNum > 0) qo_len.push_back(global_batch_size - dpb - (prefillNum - 1) * avg_prefill_length);
  const int req = (int)qo_len.size();
  const int decode_hist = 1023;  // decode requests append their 1024th token
  std::vector<int32_t> tokens(global_batch_size), indptr{0}, rev, off, keep(dpb, 1), kv_indptr{0},
      kv_indices, kv_last;
  for (int i = 0; i < global_batch_size; i++) tokens[i] = i % (int)ModelConfig.vocab_size;
  for (int r = 0; r < req; ++r) {
    const int prev = r < dpb ? decode_hist : 0;
    indptr.push_back(indptr.back() + qo_len[r]);
    for (int j = 0; j < qo_len[r]; ++j) {
      rev.push_back(r);
      off.push_back(prev + j);
    }
    const int kv_len = prev + qo_len[r];
    const int pages = (kv_len + page - 1) / page;
    for (int p = 0; p < pages; ++p) kv_indices.push_back((int32_t)kv_indices.size());
    kv_indptr.push_back(kv_indptr.back() + pages);
    kv_last.push_back((kv_len - 1) % page + 1);
  }
  if (kv_indices.size() > ModelConfig.max_page_num) {
    std::fprintf(stderr, "createUpdateData: needs %zu pages, the pool has %zu (raise allocate_kv_data_batch)\n",
                 kv_indices.size(), ModelConfig.max_page_num);
    std::exit(EXIT_FAILURE);
  }
  data.decodePrefillBorder = dpb;
  data.prefillNum = prefillNum;
  data.prefillTokensNum = global_batch_size - dpb;
  data.keepTokenListLength = dpb;
  // host arrays: update() stages them to the device.  input_tokens holds the prefill tokens
  // only; the decode tokens come from the previous iteration's samples.
  std::vector<int32_t> prefill_tokens(tokens.begin() + dpb, tokens.end());
  data.input_tokens = pinned_copy(prefill_tokens);
  data.input_indptr = pinned_copy(indptr);
  data.rev_input_indptr = pinned_copy(rev);
  data.keep_token_list = pinned_copy(keep);
  data.kv_indptr = pinned_copy(kv_indptr);
  data.kv_indices = pinned_copy(kv_indices);
  data.kv_last_page_len = pinned_copy(kv_last);
  data.per_token_offset = pinned_copy(off);
  data.gemv_batch_size = new int32_t[4]{std::min(256, dpb), std::max(dpb - 256, 0), 0, 0};
  data.gemv_num_blocks = new int32_t[4]{0, 0, 0, 0};
}

bool readConfigData(vortexConfigData& data, int rank, const std::string& filename) {
  (void)rank;
  try {
    mini_json::Value j = mini_json::parse_file(filename);
    const auto& pc = j.at("pipeline_configs");
    data.gemm_op_tag.clear();
    if (pc.contains("gemm_op_tag") && pc.at("gemm_op_tag").is_array())
      for (const auto& t : pc.at("gemm_op_tag").arr) data.gemm_op_tag.push_back(t.str);
    data.global_batch_size = (int)pc.at("global_batch_size").number();
    data.nanobatch_1_size = (int)pc.at("nanobatch_1_size").number();
    data.kqv1_size = (int)pc.at("kqv1_size").number();
    data.kqv3_size = (int)pc.at("kqv3_size").number();
  } catch (const std::exception& e) {
    std::fprintf(stderr, "readConfigData(%s): %s\n", filename.c_str(), e.what());
    return false;
  }
  return true;
}
