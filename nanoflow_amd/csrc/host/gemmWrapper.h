// GEMM operator wrappers over the kernel layer's C ABI.
//   BaseGEMMWrapper  -- same virtual interface as the reference's
//                       pipeline/include/cutlassGemmWrapperImpl.cuh:23-66;
//   HipGEMMWrapper   -- D = alpha*A.B + beta*C on the MFMA kernel; takes the place of
//                       CutlassGEMMWrapper<...> (:68-437).  The tag's cta_m x cta_n selects the
//                       closest tile of the kernel layer's menu and its split_k a split over K
//                       for launches of more than 512 live rows (the dense regime a tag is tuned
//                       for; shorter launches keep the few-row plan); cta_m = 0 leaves both to the
//                       kernel layer's cost model.  The warp and stage fields are recorded only
//                       (wavefront grid and LDS ring follow from the tile).  The three layout
//                       fields are honoured (A and output RowMajor, B Row- or ColumnMajor);
//   generateGEMM(tag) -- tag -> wrapper factory (pipeline/include/gemmFactory.cuh).
#pragma once
#include <algorithm>
#include <string>

#include "nanoflow_kernels.h"
#include "operatorWrapper.h"
#include "vortexData.h"

struct BaseGEMMWrapper : public OperatorWrapper {
  using ElementInputA = half;
  using ElementInputB = half;
  using ElementOutput = half;
  using ElementAccumulator = float;

  size_t M = 0, N = 0, K = 0;
  void set_shape(int m, int n, int k) {
    M = m;
    N = n;
    K = k;
    NF_LOG_INFO("name:%s M:%zu, N:%zu, K:%zu", name.c_str(), M, N, K);
  }
  // Rows of A that hold tokens in this iteration; the launch and the flop count cover only
  // those.  The reference's GEMMs always run their configured M (a dense batch is assumed full);
  // when admission is limited by KV memory the batch is not, and the padding rows would cost as
  // much as live ones.  Not in the reference's interface.
  size_t live_rows = (size_t)-1;
  void set_live_rows(size_t r) { live_rows = r; }
  size_t rows() const { return live_rows < M ? live_rows : M; }
  size_t mk() const { return M * K; }
  size_t kn() const { return K * N; }
  size_t mn() const { return M * N; }

  virtual void init(ElementAccumulator beta_ = ElementAccumulator(0)) = 0;
  virtual void profile() = 0;
  virtual double totalCompute() = 0;
  virtual float gflops(double runtime_ms) = 0;
  virtual bool checkResult() = 0;
  virtual ~BaseGEMMWrapper() = default;
  virtual void set_weight(ElementInputB* data_b) = 0;
  virtual bool set_weight(vortexWeight& weight) = 0;
  virtual BaseGEMMWrapper& setOutput(pllmTensor<ElementOutput> data) = 0;
  virtual BaseGEMMWrapper& setA(pllmTensor<ElementInputA> data_a) = 0;
  virtual BaseGEMMWrapper& setB(pllmTensor<ElementInputB> data_b) = 0;
  virtual BaseGEMMWrapper& setC(pllmTensor<ElementOutput> data_c) = 0;
  virtual BaseGEMMWrapper& setD(pllmTensor<ElementOutput> data_d) = 0;
  virtual pllmTensor<ElementInputA> getA() = 0;
  virtual pllmTensor<ElementOutput> getD() = 0;
  virtual pllmTensor<ElementInputB> getB() = 0;
  virtual pllmTensor<ElementOutput> getC() = 0;
  virtual void set_alpha(float alpha_) = 0;
  virtual void set_beta(float beta_) = 0;
  // Not in the reference's interface: the rows of A as e4m3 bytes [M, K] with one fp32 scale per
  // row, written by the producer of A (nf_rmsnorm_quantize_e4m3) at the same row positions.  A
  // wrapper on e4m3 weights then skips its own quantiser launch and returns true; others ignore it.
  virtual bool setQuantizedA(const uint8_t* a_q, const float* a_scale) {
    (void)a_q;
    (void)a_scale;
    return false;
  }
  // Not in the reference's interface: C = one row [1, N] added (times beta) to every row of the
  // product, read by the kernel's epilogue.  Takes the place of setC() with the bias replicated
  // over max-batch rows (replicateKQVBias, pipeline/src/pipeline.cu:520-533,1048-1058).
  virtual BaseGEMMWrapper& setCRow(pllmTensor<ElementOutput> row) = 0;
  // Also not in the reference's interface: device scratch a wrapper needs per launch (the
  // quantised activations of the fp8-weight wrapper), handed out by the pipeline's buffer plan
  // once the shape is set.  Zero for the fp16 wrapper.
  virtual size_t workspaceBytes() const { return 0; }
  virtual void setWorkspace(void* ptr, size_t bytes) {
    (void)ptr;
    (void)bytes;
  }
  // The layout of B the wrapper was built for (the tag's second layout field): ROW_MAJOR = [K][N],
  // COL_MAJOR = [N][K].  Not in the reference's interface (there it is a template argument).
  virtual PllmLayout weightLayout() const { return PllmLayout::ROW_MAJOR; }
};

struct GemmTag {
  int cta_m = 0, cta_n = 0, cta_k = 0, warp_m = 0, warp_n = 0, warp_k = 0, split_k = 1, stages = 0;
  PllmLayout layout_a = PllmLayout::ROW_MAJOR, layout_b = PllmLayout::ROW_MAJOR,
             layout_out = PllmLayout::ROW_MAJOR;
};
// Parses the tag grammar; returns false on malformed input.
bool parseGemmTag(const std::string& tag, GemmTag& out);

struct HipGEMMWrapper : public BaseGEMMWrapper {
  GemmTag tag;
  pllmTensor<half> pllm_tensor_a, pllm_tensor_b, pllm_tensor_c, pllm_tensor_d;
  float alpha = 1.f, beta = 0.f;
  bool inited = false;
  // scratch for the fp32 partial sums of launches that are split over K (few live rows against a
  // narrow N would otherwise leave most of the chip idle); sized for the worst case up to M rows
  void* splitk_workspace = nullptr;
  size_t splitk_workspace_bytes = 0;
  // the tag names a tile (cta_m, cta_n > 0): it applies to launches of more than kTagMinRows live rows
  static constexpr size_t kTagMinRows = 512;
  bool tagChoosesTile() const { return tag.cta_m > 0 && tag.cta_n > 0 && rows() > kTagMinRows; }
  // The tag's split over K, lowered to what fits the partial-sum scratch the tmp buffer reserves per
  // wrapper (ModelConfig.k_temp_size: 256 x 65536 floats, 67 MB): 2 shares of 2048 x 4096 fit, the
  // LM head's never do.
  static constexpr size_t kSplitScratchBytes = (size_t)256 * 65536 * sizeof(float);
  int taggedSplit() const {
    if (tag.split_k <= 1 || M == 0 || N == 0) return 1;
    const size_t fit = kSplitScratchBytes / (M * N * sizeof(float));
    return (int)std::max<size_t>(1, std::min<size_t>((size_t)tag.split_k, fit));
  }
  size_t workspaceBytes() const override {
    const size_t few = nf_gemm_workspace_bytes_upto((int)M, (int)N, (int)K);
    const size_t tagged = tag.cta_m > 0 && tag.cta_n > 0 && M > kTagMinRows
                              ? nf_gemm_tiled_workspace_bytes((int)M, (int)N, (int)K, taggedSplit()) : 0;
    return few > tagged ? few : tagged;
  }
  void setWorkspace(void* ptr, size_t bytes) override {
    splitk_workspace = ptr;
    splitk_workspace_bytes = bytes;
  }
  bool c_is_row = false;  // pllm_tensor_c is a [1, N] row added to every row

  explicit HipGEMMWrapper(const GemmTag& t) : tag(t) {}
  PllmLayout weightLayout() const override { return tag.layout_b; }

  void work() override;
  // operands as cutlassGemmWrapperImpl.cuh's logImpl prints them: 10 rows x 20 columns each
  OperatorWrapper& logImpl() override {
    logTensor("input", pllm_tensor_a, 10, 20);
    if (weightIsHalf()) logTensor("weight", pllm_tensor_b, 10, 20);
    if (pllm_tensor_c.ptr && beta != 0.f) logTensor("C", pllm_tensor_c, 10, 20);
    logTensor("output", pllm_tensor_d, 10, 20);
    return *this;
  }
  virtual bool weightIsHalf() const { return true; }

  HipGEMMWrapper& setOutput(pllmTensor<half> data) override { return setD(data); }
  HipGEMMWrapper& setA(pllmTensor<half> a) override {
    assert(a.layout == PllmLayout::ROW_MAJOR && a.dim1 == M && a.dim2 == K);
    pllm_tensor_a = a;
    return *this;
  }
  HipGEMMWrapper& setB(pllmTensor<half> b) override {
    pllm_tensor_b = b;
    return *this;
  }
  HipGEMMWrapper& setC(pllmTensor<half> c) override {
    assert(c.layout == PllmLayout::ROW_MAJOR && c.dim1 == M && c.dim2 == N);
    pllm_tensor_c = c;
    c_is_row = false;
    return *this;
  }
  HipGEMMWrapper& setCRow(pllmTensor<half> row) override {
    assert(row.dim1 == 1 && row.dim2 == N);
    pllm_tensor_c = row;
    c_is_row = true;
    return *this;
  }
  HipGEMMWrapper& setD(pllmTensor<half> d) override {
    assert(d.layout == PllmLayout::ROW_MAJOR && d.dim1 == M && d.dim2 == N);
    pllm_tensor_d = d;
    return *this;
  }
  pllmTensor<half> getA() override { return pllm_tensor_a; }
  pllmTensor<half> getB() override { return pllm_tensor_b; }
  pllmTensor<half> getC() override { return pllm_tensor_c; }
  pllmTensor<half> getD() override { return pllm_tensor_d; }

  // All operands are expected to be set; (re)binds the problem size and beta.
  void init(float beta_ = 0.f) override {
    beta = beta_;
    inited = true;
  }
  void set_weight(half* data_b) override {
    pllm_tensor_b = tag.layout_b == PllmLayout::ROW_MAJOR
                        ? pllmTensor<half>(data_b, K, N, PllmLayout::ROW_MAJOR)
                        : pllmTensor<half>(data_b, N, K, PllmLayout::COL_MAJOR);
  }
  bool set_weight(vortexWeight& weight) override {
    if (weight.size() != K * N) {
      std::fprintf(stderr, "Weight size mismatch  %zu %zu %zu\n", weight.size(), K, N);
      return false;
    }
    set_weight(weight.ptr);
    return true;
  }
  void set_alpha(float a) override { alpha = a; }
  void set_beta(float b) override { beta = b; }

  double totalCompute() override { return 2.0 * (double)rows() * (double)N * (double)K; }
  float gflops(double runtime_ms) override { return float(totalCompute() / 1e9 / (runtime_ms / 1e3)); }
  void profile() override;      // times 100 launches on the op's stream, logs GFLOP/s
  bool checkResult() override;  // spot-checks D against a host fp64 dot product
};

// fp16 activations against an e4m3 weight with per-output-channel scales (WeightFormat::E4M3):
// each launch quantises the rows of A into the workspace (per-row scale) and multiplies on the
// fp8 matrix cores, D = half(alpha * sa[m] * sb[n] * sum_k Aq.Bq + beta * C).  No counterpart in
// the reference (its wrappers are half-only, cutlassGemmWrapperImpl.cuh:24-27).
struct HipGEMMWrapperF8W : public HipGEMMWrapper {
  void* workspace = nullptr;
  size_t workspace_bytes = 0;
  const uint8_t* a_q = nullptr;   // rows of A quantised by their producer (setQuantizedA), or null
  const float* a_q_scale = nullptr;
  explicit HipGEMMWrapperF8W(const GemmTag& t) : HipGEMMWrapper(t) {}
  bool setQuantizedA(const uint8_t* q, const float* scale) override {
    a_q = q;
    a_q_scale = scale;
    return q && scale;
  }
  void work() override;
  bool weightIsHalf() const override { return false; }  // e4m3 bytes and scales: not dumped
  void set_weight(half* blob) override {  // see WeightFormat::E4M3
    pllm_tensor_b = pllmTensor<half>(blob, N, K, PllmLayout::COL_MAJOR);
  }
  using HipGEMMWrapper::set_weight;
  HipGEMMWrapperF8W& setCRow(pllmTensor<half> row) override {
    (void)row;
    std::fprintf(stderr, "%s: a bias row is not implemented for e4m3 weights\n", name.c_str());
    std::exit(EXIT_FAILURE);
  }
  // quantised input rows, and the fp32 sums of launches of few rows that are split over K
  size_t workspaceBytes() const override { return nf_gemm_f8w_split_workspace_bytes_upto((int)M, (int)N, (int)K); }
  void setWorkspace(void* ptr, size_t bytes) override {
    workspace = ptr;
    workspace_bytes = bytes;
  }
  bool checkResult() override;  // against the dequantised weight
};

// Unknown or unsupported tags are an error here (nullptr + logged message) rather than the
// reference's null dereference (pipeline/include/gemmFactory.cuh, pipeline_local.cu:850).
BaseGEMMWrapper* generateGEMM(const std::string& tag, WeightFormat format = WeightFormat::F16);
