#include "gemmWrapper.h"

#include <cmath>
#include <cstring>
#include <sstream>
#include <vector>

bool parseGemmTag(const std::string& tag, GemmTag& out) {
  std::vector<std::string> parts;
  std::stringstream ss(tag);
  std::string tok;
  while (std::getline(ss, tok, '_')) parts.push_back(tok);
  if (parts.size() != 11) return false;
  int* fields[8] = {&out.cta_m, &out.cta_n, &out.cta_k, &out.warp_m,
                    &out.warp_n, &out.warp_k, &out.split_k, &out.stages};
  for (int i = 0; i < 8; ++i) {
    char* end = nullptr;
    long v = std::strtol(parts[i].c_str(), &end, 10);
    if (end == parts[i].c_str() || *end != '\0' || v < 0) return false;  // 0: left to the library
    *fields[i] = (int)v;
  }
  PllmLayout* layouts[3] = {&out.layout_a, &out.layout_b, &out.layout_out};
  for (int i = 0; i < 3; ++i) {
    if (parts[8 + i] == "RowMajor") *layouts[i] = PllmLayout::ROW_MAJOR;
    else if (parts[8 + i] == "ColumnMajor") *layouts[i] = PllmLayout::COL_MAJOR;
    else return false;
  }
  return true;
}

BaseGEMMWrapper* generateGEMM(const std::string& tag, WeightFormat format) {
  GemmTag t;
  if (!parseGemmTag(tag, t)) {
    NF_LOG_ERROR("generateGEMM: malformed tag \"%s\"", tag.c_str());
    return nullptr;
  }
  if (t.layout_a != PllmLayout::ROW_MAJOR || t.layout_out != PllmLayout::ROW_MAJOR) {
    NF_LOG_ERROR("generateGEMM: tag \"%s\": A and output must be RowMajor in this build", tag.c_str());
    return nullptr;
  }
  if (format == WeightFormat::E4M3) {
    if (t.layout_b != PllmLayout::ROW_MAJOR) {
      NF_LOG_ERROR("generateGEMM: tag \"%s\": e4m3 weights have one layout; the tag must say RowMajor", tag.c_str());
      return nullptr;
    }
    return new HipGEMMWrapperF8W(t);
  }
  return new HipGEMMWrapper(t);
}

void HipGEMMWrapperF8W::work() {
  const uint8_t* bq = reinterpret_cast<const uint8_t*>(pllm_tensor_b.ptr);
  const float* bs = reinterpret_cast<const float*>(bq + e4m3WeightScaleOffset(N, K));
  if (a_q && a_q_scale) {
    NF_KERNEL_CHECK(nf_gemm_f8q_f16(a_q, a_q_scale, bq, bs, pllm_tensor_c.ptr, pllm_tensor_d.ptr, (int)rows(), (int)N,
                                    (int)K, alpha, beta, workspace, workspace_bytes, stream));
    return;
  }
  NF_KERNEL_CHECK(nf_gemm_f8w_f16(pllm_tensor_a.ptr, bq, bs, pllm_tensor_c.ptr, pllm_tensor_d.ptr, (int)rows(),
                                  (int)N, (int)K, alpha, beta, workspace, workspace_bytes, stream));
}

void HipGEMMWrapper::work() {
  const int bcol = tag.layout_b == PllmLayout::COL_MAJOR ? 1 : 0;
  if (tagChoosesTile()) {
    NF_KERNEL_CHECK(nf_gemm_f16_tiled(pllm_tensor_a.ptr, pllm_tensor_b.ptr, pllm_tensor_c.ptr, pllm_tensor_d.ptr,
                                      (int)rows(), (int)N, (int)K, alpha, beta, bcol, c_is_row ? 1 : 0, tag.cta_m,
                                      tag.cta_n, taggedSplit(), splitk_workspace, splitk_workspace_bytes, stream));
    return;
  }
  if (c_is_row) {
    NF_KERNEL_CHECK(nf_gemm_bias_f16_ws(pllm_tensor_a.ptr, pllm_tensor_b.ptr, pllm_tensor_c.ptr,
                                        pllm_tensor_d.ptr, (int)rows(), (int)N, (int)K, alpha, beta, bcol,
                                        splitk_workspace, splitk_workspace_bytes, stream));
    return;
  }
  NF_KERNEL_CHECK(nf_gemm_f16_ws(pllm_tensor_a.ptr, pllm_tensor_b.ptr, pllm_tensor_c.ptr,
                                 pllm_tensor_d.ptr, (int)rows(), (int)N, (int)K, alpha, beta, bcol, splitk_workspace,
                                 splitk_workspace_bytes, stream));
}

void HipGEMMWrapper::profile() {
  hipEvent_t e0, e1;
  HIP_CHECK(hipEventCreate(&e0));
  HIP_CHECK(hipEventCreate(&e1));
  const int iters = 100;
  work();
  HIP_CHECK(hipEventRecord(e0, stream));
  for (int i = 0; i < iters; ++i) work();
  HIP_CHECK(hipEventRecord(e1, stream));
  HIP_CHECK(hipEventSynchronize(e1));
  float ms = 0;
  HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
  std::printf("%s M=%zu N=%zu K=%zu: %.3f ms, %.1f GFLOP/s\n", name.c_str(), M, N, K, ms / iters,
              gflops(ms / iters));
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
}

static float half_bits_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1f, man = h & 0x3ffu, bits;
  if (exp == 0) {
    if (man == 0) bits = sign;
    else {
      int e = -1;
      do { man <<= 1; ++e; } while (!(man & 0x400u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) bits = sign | 0x7f800000u | (man << 13);
  else bits = sign | ((exp + 112) << 23) | (man << 13);
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

// Runs the GEMM once and compares 64 sampled outputs with a host float64 dot product
// (pass rule of the reference's checkResult: (|d - ref| - 0.01) / |ref| <= 0.1).
bool HipGEMMWrapper::checkResult() {
  work();
  HIP_CHECK(hipStreamSynchronize(stream));
  const bool bcol = tag.layout_b == PllmLayout::COL_MAJOR;
  std::vector<uint16_t> arow(K), bcolv(K);
  bool ok = true;
  for (int s = 0; s < 64 && ok; ++s) {
    size_t m = (size_t)(s * 2654435761u) % std::max<size_t>(rows(), 1), n = (size_t)(s * 40503u + 7) % N;
    HIP_CHECK(hipMemcpy(arow.data(), pllm_tensor_a.ptr + m * K, K * 2, hipMemcpyDeviceToHost));
    if (bcol) HIP_CHECK(hipMemcpy(bcolv.data(), pllm_tensor_b.ptr + n * K, K * 2, hipMemcpyDeviceToHost));
    else HIP_CHECK(hipMemcpy2D(bcolv.data(), 2, pllm_tensor_b.ptr + n, N * 2, 2, K, hipMemcpyDeviceToHost));
    double ref = 0;
    for (size_t k = 0; k < K; ++k) ref += (double)half_bits_to_float(arow[k]) * half_bits_to_float(bcolv[k]);
    ref *= alpha;
    uint16_t c16 = 0, d16 = 0;
    if (beta != 0.f) {
      HIP_CHECK(hipMemcpy(&c16, pllm_tensor_c.ptr + (c_is_row ? 0 : m * N) + n, 2, hipMemcpyDeviceToHost));
      ref += beta * half_bits_to_float(c16);
    }
    HIP_CHECK(hipMemcpy(&d16, pllm_tensor_d.ptr + m * N + n, 2, hipMemcpyDeviceToHost));
    double d = half_bits_to_float(d16);
    if ((std::fabs(d - ref) - 0.01) / std::max(std::fabs(ref), 1e-6) > 0.1) ok = false;
  }
  return ok;
}

static float e4m3_bits_to_float(uint8_t v) {
  const int e = (v >> 3) & 0xf, m = v & 7;
  const float f = e == 0 ? std::ldexp((float)m, -9) : std::ldexp((float)(8 + m), e - 10);
  return (v & 0x80) ? -f : f;
}

// As HipGEMMWrapper::checkResult, the reference value taken from fp16 activations and the
// dequantised weight (so the activation quantisation counts as error, within the same pass rule).
bool HipGEMMWrapperF8W::checkResult() {
  work();
  HIP_CHECK(hipStreamSynchronize(stream));
  const uint8_t* bq = reinterpret_cast<const uint8_t*>(pllm_tensor_b.ptr);
  const float* bs = reinterpret_cast<const float*>(bq + e4m3WeightScaleOffset(N, K));
  std::vector<uint16_t> arow(K);
  std::vector<uint8_t> brow(K);
  bool ok = true;
  for (int s = 0; s < 64 && ok; ++s) {
    size_t m = (size_t)(s * 2654435761u) % std::max<size_t>(rows(), 1), n = (size_t)(s * 40503u + 7) % N;
    float scale = 0;
    HIP_CHECK(hipMemcpy(arow.data(), pllm_tensor_a.ptr + m * K, K * 2, hipMemcpyDeviceToHost));
    HIP_CHECK(hipMemcpy(brow.data(), bq + n * K, K, hipMemcpyDeviceToHost));
    HIP_CHECK(hipMemcpy(&scale, bs + n, 4, hipMemcpyDeviceToHost));
    double ref = 0;
    for (size_t k = 0; k < K; ++k) ref += (double)half_bits_to_float(arow[k]) * e4m3_bits_to_float(brow[k]);
    ref *= (double)alpha * scale;
    uint16_t c16 = 0, d16 = 0;
    if (beta != 0.f) {
      HIP_CHECK(hipMemcpy(&c16, pllm_tensor_c.ptr + m * N + n, 2, hipMemcpyDeviceToHost));
      ref += beta * half_bits_to_float(c16);
    }
    HIP_CHECK(hipMemcpy(&d16, pllm_tensor_d.ptr + m * N + n, 2, hipMemcpyDeviceToHost));
    double d = half_bits_to_float(d16);
    if ((std::fabs(d - ref) - 0.01) / std::max(std::fabs(ref), 1e-6) > 0.1) ok = false;
  }
  return ok;
}
