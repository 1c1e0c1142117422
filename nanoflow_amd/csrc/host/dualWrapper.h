// DualWrapper: fused gate/up projection with the SwiGLU epilogue,
// D2 = silu(A.B0) * (A.B1); the two plain products are not stored (kStoreD0/kStoreD1 are
// false in the reference).  Interface of pipeline/include/dualWrapper.cuh:47-321; the tile
// template parameters of the reference type are dropped (tiling is the kernel layer's).
#pragma once
#include "nanoflow_kernels.h"
#include "operatorWrapper.h"
#include "vortexData.h"

struct DualWrapper : public OperatorWrapper {
  int M = 0, N = 0, K = 0;
  pllmTensor<half> pllm_tensor_a, pllm_tensor_b1, pllm_tensor_b2, pllm_tensor_c;
  pllmTensor<half> pllm_tensor_d0, pllm_tensor_d1, pllm_tensor_d2;
  bool inited = false;
  // WeightFormat::E4M3: b1 / b2 point at e4m3 weights with their scales behind them; the rows of A
  // are quantised into the workspace on every launch (nf_dual_swiglu_f8w_f16)
  int live_rows = -1;  // rows of A that hold tokens in this iteration (see BaseGEMMWrapper::live_rows)
  void set_live_rows(int r) { live_rows = r; }
  int rows() const { return live_rows >= 0 && live_rows < M ? live_rows : M; }
  bool e4m3 = false;
  // e4m3 weights: the rows of A as e4m3 bytes [M, K] + one fp32 scale per row, when the producer
  // of A has written them (nf_rmsnorm_quantize_e4m3); the launch then skips its quantiser
  const uint8_t* a_q = nullptr;
  const float* a_q_scale = nullptr;
  bool setQuantizedA(const uint8_t* q, const float* scale) {
    a_q = q;
    a_q_scale = scale;
    return e4m3 && q && scale;
  }
  void* workspace = nullptr;
  size_t workspace_bytes = 0;
  void setWeightFormat(WeightFormat f) { e4m3 = f == WeightFormat::E4M3; }
  // fp16 weights: ROW_MAJOR = [K][N] as the reference's weight files hold them, COL_MAJOR = [N][K],
  // k contiguous (what a GEMM tag calls ColumnMajor for B).  The reference's DualWrapper takes its
  // layouts as template arguments (dualWrapper.cuh:47-60) and the pipeline JSON has no tag for it:
  // the pipelines give the pair the layout that ALL per-layer GEMM tags agree on, RowMajor otherwise.
  PllmLayout weight_layout = PllmLayout::ROW_MAJOR;
  void setWeightLayout(PllmLayout l) { weight_layout = l; }
  // fp16 weights: scratch for launches of few rows that are split over K (nf_dual_swiglu_f16_ws)
  size_t workspaceBytes() const {
    return e4m3 ? nf_dual_swiglu_f8w_split_workspace_bytes_upto(M, N, K) : nf_dual_swiglu_workspace_bytes_upto(M, N, K);
  }
  void setWorkspace(void* ptr, size_t bytes) {
    workspace = ptr;
    workspace_bytes = bytes;
  }

  void set_shape(int m, int n, int k) {
    M = m;
    N = n;
    K = k;
    NF_LOG_INFO("name:%s M:%d, N:%d, K:%d", name.c_str(), M, N, K);
  }
  void work() override {
    if (e4m3) {
      const uint8_t* g = reinterpret_cast<const uint8_t*>(pllm_tensor_b1.ptr);
      const uint8_t* u = reinterpret_cast<const uint8_t*>(pllm_tensor_b2.ptr);
      const size_t so = e4m3WeightScaleOffset((size_t)N, (size_t)K);
      if (a_q && a_q_scale) {
        NF_KERNEL_CHECK(nf_dual_swiglu_f8q_f16(a_q, a_q_scale, g, reinterpret_cast<const float*>(g + so), u,
                                               reinterpret_cast<const float*>(u + so), pllm_tensor_d2.ptr, rows(), N, K,
                                               workspace, workspace_bytes, stream));
        return;
      }
      NF_KERNEL_CHECK(nf_dual_swiglu_f8w_f16(pllm_tensor_a.ptr, g, reinterpret_cast<const float*>(g + so), u,
                                             reinterpret_cast<const float*>(u + so), pllm_tensor_d2.ptr, rows(), N, K,
                                             workspace, workspace_bytes, stream));
      return;
    }
    NF_KERNEL_CHECK(nf_dual_swiglu_f16_ws(pllm_tensor_a.ptr, pllm_tensor_b1.ptr, pllm_tensor_b2.ptr, pllm_tensor_d2.ptr,
                                          rows(), N, K, weight_layout == PllmLayout::COL_MAJOR ? 1 : 0, workspace,
                                          workspace_bytes, stream));
  }
  OperatorWrapper& logImpl() override {
    logTensor("input", pllm_tensor_a, 10, 20);
    if (!e4m3) {  // e4m3 weights are bytes with their scales behind them: not dumped
      logTensor("weight0", pllm_tensor_b1, 10, 20);
      logTensor("weight1", pllm_tensor_b2, 10, 20);
    }
    logTensor("output2", pllm_tensor_d2, 128, 20);
    return *this;
  }
  DualWrapper& setA(pllmTensor<half> a) {
    assert(a.layout == PllmLayout::ROW_MAJOR && (int)a.dim1 == M && (int)a.dim2 == K);
    pllm_tensor_a = a;
    return *this;
  }
  DualWrapper& setC(pllmTensor<half> c) {  // bias operand; unused (kUseBias is false)
    pllm_tensor_c = c;
    return *this;
  }
  DualWrapper& setD(pllmTensor<half> d0, pllmTensor<half> d1, pllmTensor<half> d2) {
    pllm_tensor_d0 = d0;
    pllm_tensor_d1 = d1;
    pllm_tensor_d2 = d2;
    return *this;
  }
  pllmTensor<half> getA() { return pllm_tensor_a; }
  pllmTensor<half> getD() { return pllm_tensor_d2; }
  pllmTensor<half> getC() { return pllm_tensor_c; }
  void init() { inited = true; }
  // weight1 = gate (goes through SiLU), weight2 = up
  bool set_weight(vortexWeight& weight1, vortexWeight& weight2) {
    if (weight1.size() != (size_t)K * N || weight2.size() != (size_t)K * N) {
      std::fprintf(stderr, "Dual weight size mismatch %zu %zu vs %d x %d\n", weight1.size(),
                   weight2.size(), K, N);
      return false;
    }
    if (weight_layout == PllmLayout::COL_MAJOR && !e4m3) {
      pllm_tensor_b1 = pllmTensor<half>(weight1.ptr, N, K, PllmLayout::COL_MAJOR);
      pllm_tensor_b2 = pllmTensor<half>(weight2.ptr, N, K, PllmLayout::COL_MAJOR);
    } else {
      pllm_tensor_b1 = pllmTensor<half>(weight1.ptr, K, N, PllmLayout::ROW_MAJOR);
      pllm_tensor_b2 = pllmTensor<half>(weight2.ptr, K, N, PllmLayout::ROW_MAJOR);
    }
    return true;
  }
  double totalCompute() { return 4.0 * (double)rows() * (double)N * (double)K; }
};
