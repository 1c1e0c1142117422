// Pipeline schedules for one GPU.
//   PipelineBase              config / update / run interface (pipeline/include/pipeline.h:22-51)
//   LocalPipeline             two nano-batches; dense ops on stream_gemm, attention on
//                             stream_gemv, cross-stream edges are event waits
//                             (pipeline/include/pipeline.h:322-403, pipeline/src/pipeline_local.cu)
//   NonOverlapLocalPipeline   same math on one stream, no nano-batching
//                             (pipeline/include/pipeline.h:405-465,
//                              pipeline/src/pipeline_nonoverlap_local.cu)
//   Pipeline                  the reference's main schedule (pipeline/include/pipeline.h:53-170,
//                             pipeline/src/pipeline.cu) on one device: the QKV projection, RoPE-append
//                             and decode attention run as FOUR nano-batches, O / FFN as two; its
//                             all-gather / all-reduce steps have nothing to move on one rank and are
//                             left out.  With enable_offload it also round-trips KV pages through host
//                             memory every layer (pipeline.cu:37-59,701-726).
// More than one rank (the collectives) is outside this build.
#pragma once
#include <array>
#include <cstdarg>
#include <string>
#include <memory>

#include "allocManager.h"
#include "config.h"
#include "dualWrapper.h"
#include "eventManager.h"
#include "gemmWrapper.h"
#include "gemvWrapper.h"
#include "otherWrapper.h"
#include "vortexData.h"

#include <map>
#include <set>

#define SET_NAME_PTR(var) (var)->name = #var;
#define SET_NAME_REF(var) (var).name = #var;
#define GEMM_ALIAS(x) BaseGEMMWrapper*& x = gemms[static_cast<int>(GEMM_NAME::x)]

// Accumulated per-iteration timings (filled when profiling is on).
struct PipelineTimings {
  double iter_ms = 0;        // last iteration, start of first op to end of sampler
  double decode_attn_ms = 0; // sum of decode-attention launch durations
  long decode_attn_launches = 0;
  double prefill_attn_ms = 0;
  long prefill_attn_launches = 0;
  double gemm_ms = 0;        // sum of dense GEMM launch durations (profiling level 2)
  long gemm_launches = 0;
  double gemm_flop = 0;      // flops of those launches (2*M*N*K each; the fused gate/up pair 4*M*N*K)
  int layer_stride = 1;      // every layer_stride-th layer's launches are the timed ones
};

class PipelineBase {
public:
  PipelineBase(vortexInitData* input_data, int nrank, int nranks, int vnranks);
  virtual ~PipelineBase() = default;

protected:
  vortexInitData* input_data;
  vortexUpdateData update_data;       // device pointers
  vortexUpdateData host_update_data;  // same iteration, host (staged) pointers
  vortexConfigData config_data;
  int rank;
  int nranks;
  int vnranks;
  AllocationManager<half> tmpBufferM;
  EventManager ev;
  std::vector<hipEvent_t>& events = ev.events;
  bool profiling = false;
  bool profile_gemms = false;
  PipelineTimings timings;
  // The *_KQVBIAS pipeline types (models whose q/k/v projections have a bias, Qwen2): the QKV
  // GEMMs add vortexLayerWeight::B_KQV ([1, kqv_n], columns K|V|Q) to every row, beta = 1
  // (pipeline/src/pipeline.cu:520-533, pipeline_nonoverlap.cu:209-211).
  WeightFormat weight_format = getWeightFormat();  // of the five per-layer GEMM weights
  // config() reports what it cannot build here and returns early instead of ending the process
  // (the reference dereferences the null wrapper, pipeline_local.cu:850); the control plane turns
  // it into an error code.
  std::string config_error;
  void configFail(const char* fmt, ...) __attribute__((format(printf, 2, 3))) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    config_error = buf;
    std::fprintf(stderr, "%s\n", buf);
  }
  bool kqv_bias = false;
  bool bindKQVBias(BaseGEMMWrapper* kqv, vortexWeight& bias) {
    if (!kqv_bias) return true;
    if (!bias.ptr || bias.size() != kqv->N) {
      std::fprintf(stderr, "KQV bias size mismatch  %zu %zu\n", bias.size(), kqv->N);
      return false;
    }
    kqv->setCRow(pllmTensor<half>(bias.ptr, 1, (int)kqv->N, PllmLayout::ROW_MAJOR));
    return true;
  }

  // The weight layout the gate/up pair is given (it has no tag of its own): [N][K] when every
  // per-layer GEMM tag says ColumnMajor for B, the reference's [K][N] otherwise.
  template <class Gemms>
  static PllmLayout pairWeightLayout(const Gemms& gemms, int logits_index) {
    for (int i = 0; i < (int)gemms.size(); ++i)
      if (i != logits_index && gemms[i]->weightLayout() != PllmLayout::COL_MAJOR) return PllmLayout::ROW_MAJOR;
    return PllmLayout::COL_MAJOR;
  }

  // e4m3 weights: the RMSNorm in front of the QKV and of the gate/up projection writes its rows
  // as e4m3 bytes + one fp32 scale per row as well, into a [rows, hidden] image carved from the tmp
  // buffer, and the GEMMs read their rows there instead of launching a quantiser of their own.
  struct QuantRows {
    uint8_t* q = nullptr;
    float* scale = nullptr;
    QuantRows at(size_t row) const { return {q + row * (size_t)ModelConfig.model_hidden_dim, scale + row}; }
    explicit operator bool() const { return q != nullptr; }
  };
  QuantRows allocQuantRows(size_t rows) {
    if (weight_format != WeightFormat::E4M3 || !LayerNorm::canQuantize() || rows == 0) return {};
    QuantRows r;
    r.q = static_cast<uint8_t*>(tmpBufferM.allocBytes(rows * (size_t)ModelConfig.model_hidden_dim));
    r.scale = static_cast<float*>(tmpBufferM.allocBytes(rows * sizeof(float)));
    return r;
  }

  // hipGraph replay of an iteration.  Everything that shapes a launch (grid sizes, row counts,
  // which operators are skipped) is a function of the configuration and of a few integers of
  // the update data; those integers form the signature a captured graph is filed under.  A
  // signature runs eagerly the first time it is seen (one-time kernel attribute calls must not
  // happen inside a capture), is captured the second time, and is replayed from then on.
  // Per-launch profiling brackets cannot be read back from a replay, so profiling disables it.
  // So do CU-masked streams: a replayed graph runs its kernel nodes without the capture stream's
  // CU mask and a kernel node has no mask attribute, so a pipeline built on masked streams
  // (NANOFLOW_GEMM_CUS / NANOFLOW_GEMV_CUS) keeps launching eagerly whatever the graph mode says.
  bool graph_mode = false;
  bool masked_streams = false;
  std::map<std::vector<int>, hipGraphExec_t> graph_execs;
  std::set<std::vector<int>> graph_seen;
  long graph_replays = 0, graph_captures = 0, graph_eager = 0;
  static constexpr size_t kMaxGraphs = 64;
  static constexpr size_t kMaxSeen = 4096;

  template <class F>
  void runIteration(hipStream_t origin, const std::vector<int>& sig, F&& enqueue) {
    if (!graph_mode || profiling || masked_streams) {
      ++graph_eager;
      enqueue();
      return;
    }
    auto it = graph_execs.find(sig);
    if (it == graph_execs.end()) {
      if (!graph_seen.count(sig) || graph_execs.size() >= kMaxGraphs) {
        if (graph_seen.size() >= kMaxSeen) graph_seen.clear();  // bounded: forgetting only delays a capture
        graph_seen.insert(sig);
        ++graph_eager;
        enqueue();
        return;
      }
      hipGraph_t graph = nullptr;
      HIP_CHECK(hipStreamBeginCapture(origin, hipStreamCaptureModeRelaxed));
      enqueue();
      HIP_CHECK(hipStreamEndCapture(origin, &graph));
      hipGraphExec_t exec = nullptr;
      HIP_CHECK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
      HIP_CHECK(hipGraphDestroy(graph));
      it = graph_execs.emplace(sig, exec).first;
      ++graph_captures;
    }
    HIP_CHECK(hipGraphLaunch(it->second, origin));
    ++graph_replays;
  }
  void clearGraphs() {
    for (auto& kv : graph_execs) (void)hipGraphExecDestroy(kv.second);
    graph_execs.clear();
    graph_seen.clear();
  }
  std::vector<int> baseSignature() const {
    std::vector<int> s = {host_update_data.decodePrefillBorder, host_update_data.prefillNum,
                          host_update_data.prefillTokensNum};
    for (int i = 0; i < 4; ++i) {
      s.push_back(host_update_data.gemv_batch_size ? host_update_data.gemv_batch_size[i] : 0);
      s.push_back(host_update_data.gemv_num_blocks ? host_update_data.gemv_num_blocks[i] : 0);
    }
    return s;
  }

public:
  virtual vortexOutputData run() = 0;
  virtual void update(vortexUpdateData* update_data) = 0;
  virtual void config(vortexConfigData* config_data) = 0;
  virtual void setName() {}
  // stream on which update data must be uploaded so that it is ordered before run()
  virtual hipStream_t uploadStream() = 0;
  // level 0: off; 1: attention launches; 2: attention and dense GEMM launches
  // empty when the last config() built its schedule
  const std::string& configError() const { return config_error; }
  virtual void setProfiling(int level) { profiling = level > 0; profile_gemms = level > 1; }
  // every stride-th launch of an operator is timed: the override, else 4 on schedules of 8 or
  // more layers (the event records themselves cost device time), else 1
  static inline int profile_stride_override = 0;
  static unsigned profileStride() {
    if (profile_stride_override > 0) return (unsigned)profile_stride_override;
    return ModelConfig.run_layer >= 8 ? 4u : 1u;
  }
  int profilingLevel() const { return profiling ? (profile_gemms ? 2 : 1) : 0; }
  const PipelineTimings& getTimings() const { return timings; }
  void resetTimings() {
    const int stride = timings.layer_stride;
    timings = PipelineTimings();
    timings.layer_stride = stride;
  }
  void setGraphMode(bool on) {
    graph_mode = on;
    if (!on) clearGraphs();
  }
  void graphCounters(long out[3]) const {
    out[0] = graph_eager;
    out[1] = graph_captures;
    out[2] = graph_replays;
  }
  void setHostUpdate(const vortexUpdateData& h) { host_update_data = h; }
};

class LocalPipeline : public PipelineBase {
public:
  void assignSameStream();
  enum class GEMM_NAME { O1 = 0, O2, D1, D2, KQV1, KQV2, LOGITS, NUM };
  static constexpr std::array gemmConfig = {
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // O1
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // O2
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // D1
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // D2
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // KQV1
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // KQV2
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // LOGITS
  };
  static constexpr int gemmNum = static_cast<int>(GEMM_NAME::NUM);
  std::array<BaseGEMMWrapper*, gemmNum> gemms{};
  GEMM_ALIAS(O1);
  GEMM_ALIAS(O2);
  GEMM_ALIAS(D1);
  GEMM_ALIAS(D2);
  GEMM_ALIAS(KQV1);
  GEMM_ALIAS(KQV2);
  GEMM_ALIAS(LOGITS);

  DualWrapper dual1, dual2;
  GenEmbedding genEmbedding1, genEmbedding2;
  DecodeGemvWrapper GEMV1, GEMV2, GEMV3, GEMV4;
  std::array<DecodeGemvWrapper*, 4> gemvs{&GEMV1, &GEMV2, &GEMV3, &GEMV4};
  LayerNorm layerNormAttention1, layerNormAttention2;
  LayerNorm layerNormFFN1, layerNormFFN2;
  LayerNorm layerNormModel;
  RoPEAppend roPEAppends[2];
  PrefillGemvWrapper prefill1, prefill2;
  MaxSampling maxSampler;
  KeepToken keepToken;

  pllmTensor<half> gemvQ1, gemvQ2;
  pllmTensor<half> gemvAggregateOutput1, gemvAggregateOutput2;
  pllmTensor<half> KQV_output1, KQV_output2;
  BaseGEMMWrapper* KQV_ptrs[2] = {nullptr, nullptr};
  vortexOutputData output_data;
  hipStream_t stream_gemm = nullptr;
  hipStream_t stream_gemv = nullptr;
  hipStream_t stream_other = nullptr;
  int update_token_num = 0;
  int border_request = -1;  // the prefill request cut by the nano-batch border in this iteration (-1: none)
  vortexUpdateData prefill1_update;   // device copies patched for a prefill request that
  vortexUpdateData prefill1_staging;  // straddles the nano-batch border (+ pinned staging)
  bool nanobatch_only = false;

  LocalPipeline(vortexInitData* input_data, int nrank, int nranks, int vnranks,
                bool nanobatch_only = false, bool kqv_bias = false);
  ~LocalPipeline() override;
  void ScheduleInit();
  void GEMMOpInit();
  void GEMVOpInit();
  void OtherOpInit();
  void setWeight(int layer);
  void setWeight_group_O(int layer);
  void setWeight_group_LN(int layer);
  vortexOutputData run() override;
  void update(vortexUpdateData* update_data) override;
  void config(vortexConfigData* config_data) override;
  void GEMVOpUpdate();
  void setName() override;
  hipStream_t uploadStream() override { return stream_gemm; }
  void setProfiling(int level) override;

private:
  void init();
  double totalCompute();
  void enqueueIteration();
};

class NonOverlapLocalPipeline : public PipelineBase {
public:
  enum class GEMM_NAME { O = 0, D, KQV, LOGITS, NUM };
  static constexpr std::array gemmConfig = {
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // O
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // D
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // KQV
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // LOGITS
  };
  static constexpr int gemmNum = static_cast<int>(GEMM_NAME::NUM);
  std::array<BaseGEMMWrapper*, gemmNum> gemms{};
  GEMM_ALIAS(O);
  GEMM_ALIAS(D);
  GEMM_ALIAS(KQV);
  GEMM_ALIAS(LOGITS);

  DualWrapper dual;
  GenEmbedding genEmbedding;
  DecodeGemvWrapper GEMV;
  LayerNorm layerNormAttention, layerNormFFN, layerNormModel;
  RoPEAppend roPEAppend;
  PrefillGemvWrapper prefill;
  MaxSampling maxSampler;
  KeepToken keepToken;

  pllmTensor<half> gemvInput, gemvOutput;
  vortexOutputData output_data;
  hipStream_t stream_all = nullptr;
  // Chunked-prefill attention runs beside decode attention (different requests, disjoint rows):
  // it is bound by the latency of its longest tile, not by bandwidth, and a prefill workgroup
  // (32 KB of LDS) fits on a CU next to two decode-attention workgroups.
  hipStream_t stream_prefill = nullptr;
  hipEvent_t prefill_fork = nullptr, prefill_join = nullptr;
  int update_token_num = 0;

  NonOverlapLocalPipeline(vortexInitData* input_data, int nrank, int nranks, int vnranks,
                          bool kqv_bias = false);
  ~NonOverlapLocalPipeline() override;
  void ScheduleInit();
  void GEMMOpInit();
  void GEMVOpInit();
  void OtherOpInit();
  void setWeight(int layer);
  vortexOutputData run() override;
  void update(vortexUpdateData* update_data) override;
  void config(vortexConfigData* config_data) override;
  void GEMVOpUpdate();
  void setName() override;
  hipStream_t uploadStream() override { return stream_all; }
  void setProfiling(int level) override;

private:
  double totalCompute();
};

class Pipeline : public PipelineBase {
public:
  enum class GEMM_NAME { O1 = 0, O2, D1, D2, KQV1, KQV2, KQV3, KQV4, LOGITS, NUM };
  static constexpr std::array gemmConfig = {
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // O1
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // O2
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // D1
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // D2
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",   // KQV1
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // KQV2
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // KQV3
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",   // KQV4
      "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor",  // LOGITS
  };
  static constexpr int gemmNum = static_cast<int>(GEMM_NAME::NUM);
  std::array<BaseGEMMWrapper*, gemmNum> gemms{};
  GEMM_ALIAS(O1);
  GEMM_ALIAS(O2);
  GEMM_ALIAS(D1);
  GEMM_ALIAS(D2);
  GEMM_ALIAS(KQV1);
  GEMM_ALIAS(KQV2);
  GEMM_ALIAS(KQV3);
  GEMM_ALIAS(KQV4);
  GEMM_ALIAS(LOGITS);

  DualWrapper dual1, dual2;
  GenEmbedding genEmbedding1, genEmbedding2_1, genEmbedding2_2;
  DecodeGemvWrapper GEMV1, GEMV2, GEMV3, GEMV4;
  std::array<DecodeGemvWrapper*, 4> gemvs{&GEMV1, &GEMV2, &GEMV3, &GEMV4};
  PrefillGemvWrapper prefill;
  LayerNorm layerNormAttention1, layerNormAttention2_1, layerNormAttention2_2;
  LayerNorm layerNormFFN1, layerNormFFN2;
  LayerNorm layerNormModel1;
  BaseGEMMWrapper* KQV_ptrs[4] = {nullptr, nullptr, nullptr, nullptr};
  RoPEAppend roPEAppends[4];
  PageAggregator pageAgg;
  PageDispatcher pageDisp;
  MaxSampling maxSampler;
  KeepToken keepToken;

  pllmTensor<half> gemvQ, gemvAggregateOutput, KQV_output;
  vortexOutputData output_data;
  hipStream_t stream_gemm = nullptr, stream_gemv = nullptr, stream_cpy = nullptr;
  int update_token_num = 0;
  bool enable_offload = false;
  bool nanobatch_only = false;

  // KV offload round trip (enable_offload): the pages of the iteration's first offload_reqs
  // requests are gathered from the layer's pool into deviceOffloadKVCache, copied to the pinned
  // host buffer offloadKVCache, copied back into deviceLoadKVCache and scattered into the pages
  // the requests own -- the data path of evicting and re-admitting a request, paid every layer
  // as in the reference (whose lists and copy sizes are fixed constants: a cost model).
  static constexpr int kOffloadReqs = 2;
  half* offloadKVCache = nullptr;        // pinned host
  half* deviceOffloadKVCache = nullptr;  // device staging, laid out like kv_indices
  half* deviceLoadKVCache = nullptr;
  int32_t* finished_idx = nullptr;       // device: 0, 1, 2, ...
  int32_t* load_idx = nullptr;
  size_t offload_pages_cap = 0;          // pages the staging buffers hold
  size_t offload_pages = 0;              // pages moved per layer in this iteration
  int offload_reqs = 0;
  hipEvent_t offload_done = nullptr;

  Pipeline(vortexInitData* input_data, int nrank, int nranks, int vnranks, bool enable_offload = false,
           bool nanobatch_only = false, bool kqv_bias = false);
  ~Pipeline() override;
  void ScheduleInit();
  void GEMMOpInit();
  void GEMVOpInit();
  void OtherOpInit();
  void setWeight(int layer);
  vortexOutputData run() override;
  void update(vortexUpdateData* update_data) override;
  void config(vortexConfigData* config_data) override;
  void GEMVOpUpdate();
  void setName() override;
  hipStream_t uploadStream() override { return stream_gemm; }
  void setProfiling(int level) override;

private:
  void enqueueIteration();
};

// Creates a stream restricted to `num_cus` compute units starting at CU `first_cu` of every
// XCD-interleaved numbering (0 = no restriction, plain stream).
hipStream_t createPipelineStream(int first_cu, int num_cus);
