// test_other_wrappers: the smaller operators of the reference's vocabulary (SplitKQVOutput,
// SplitTensor, Activation, Transpose, CopyTensor, SleepWrapper; pipeline/include/otherWrapper.cuh:
// 183-301, 395-412, 542-568) driven through their wrapper classes -- init / config / setStream /
// run, as a schedule would -- on small random tensors, each result checked against plain host loops.
// Prints one line per operator and exits non-zero when one of them is wrong.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "otherWrapper.h"

// values k / 256 with |k| <= 1000: exactly representable in fp16
static uint16_t exact_half(int k) {
  if (k == 0) return 0;
  const uint16_t sign = k < 0 ? 0x8000u : 0;
  unsigned a = (unsigned)std::abs(k);  // value a * 2^-8, a < 1024
  int e = 0;
  while ((a >> e) > 1) ++e;            // a in [2^e, 2^(e+1))
  const unsigned man = ((a << (10 - e)) & 0x3ffu);
  return (uint16_t)(sign | (unsigned)((e - 8 + 15) << 10) | man);
}

static std::vector<uint16_t> random_halves(size_t n, unsigned seed) {
  std::vector<uint16_t> v(n);
  unsigned s = seed * 2654435761u + 12345u;
  for (auto& x : v) {
    s = s * 1664525u + 1013904223u;
    x = exact_half((int)((s >> 8) % 2001u) - 1000);
  }
  return v;
}

struct DeviceBuf {
  half* p = nullptr;
  size_t n = 0;
  explicit DeviceBuf(size_t n_) : n(n_) { HIP_CHECK(hipMalloc(&p, (n ? n : 1) * sizeof(half))); }
  explicit DeviceBuf(const std::vector<uint16_t>& h) : DeviceBuf(h.size()) {
    HIP_CHECK(hipMemcpy(p, h.data(), n * sizeof(half), hipMemcpyHostToDevice));
  }
  ~DeviceBuf() { (void)hipFree(p); }
  std::vector<uint16_t> host() const {
    std::vector<uint16_t> h(n);
    HIP_CHECK(hipMemcpy(h.data(), p, n * sizeof(half), hipMemcpyDeviceToHost));
    return h;
  }
};

static int failures = 0;
static void report(const char* what, bool ok, const char* detail = "") {
  std::printf("%-16s %s %s\n", what, ok ? "ok" : "WRONG", detail);
  if (!ok) ++failures;
}

int main() {
  hipStream_t stream;
  HIP_CHECK(hipStreamCreate(&stream));
  const auto ROW = PllmLayout::ROW_MAJOR, COL = PllmLayout::COL_MAJOR;

  {  // SplitKQVOutput: [rows, 16 + 32 + 24] -> k | q | v
    const int rows = 37, kd = 16, qd = 32, vd = 24, w = kd + qd + vd;
    const auto h = random_halves((size_t)rows * w, 1);
    DeviceBuf in(h), k((size_t)rows * kd), q((size_t)rows * qd), v((size_t)rows * vd);
    SplitKQVOutput op;
    op.setName("splitKQV").setStream(stream);
    op.init(pllmTensor<half>(in.p, rows, w, ROW), pllmTensor<half>(k.p, rows, kd, ROW), pllmTensor<half>(q.p, rows, qd, ROW),
            pllmTensor<half>(v.p, rows, vd, ROW), rows, kd, qd, vd);
    op.run().log();
    HIP_CHECK(hipStreamSynchronize(stream));
    const auto hk = k.host(), hq = q.host(), hv = v.host();
    bool ok = true;
    for (int r = 0; r < rows; ++r) {
      for (int c = 0; c < kd; ++c) ok &= hk[(size_t)r * kd + c] == h[(size_t)r * w + c];
      for (int c = 0; c < qd; ++c) ok &= hq[(size_t)r * qd + c] == h[(size_t)r * w + kd + c];
      for (int c = 0; c < vd; ++c) ok &= hv[(size_t)r * vd + c] == h[(size_t)r * w + kd + qd + c];
    }
    report("SplitKQVOutput", ok);
  }
  {  // SplitTensor: the rank's columns of [M, nranks * N]
    const int M = 29, N = 40, nranks = 4, rank = 2;
    const auto h = random_halves((size_t)M * nranks * N, 2);
    DeviceBuf in(h), out((size_t)M * N);
    SplitTensor op;
    op.setName("splitTensor").setStream(stream);
    op.init(pllmTensor<half>(in.p, M, nranks * N, ROW), pllmTensor<half>(out.p, M, N, ROW), nranks, rank);
    op.run().log();
    HIP_CHECK(hipStreamSynchronize(stream));
    const auto ho = out.host();
    bool ok = true;
    for (int r = 0; r < M; ++r)
      for (int c = 0; c < N; ++c) ok &= ho[(size_t)r * N + c] == h[(size_t)r * nranks * N + rank * N + c];
    report("SplitTensor", ok);
  }
  {  // Activation: [M, 2 N] -> left * silu(right)
    const int M = 33, N = 72;
    const auto h = random_halves((size_t)M * 2 * N, 3);
    DeviceBuf in(h), out((size_t)M * N);
    Activation op;
    op.setName("activation").setStream(stream);
    op.init(in.p, out.p, M * 2 * N, M * N);
    op.config(M, N);
    op.run();
    HIP_CHECK(hipStreamSynchronize(stream));
    const auto ho = out.host();
    double worst = 0;
    for (int r = 0; r < M; ++r)
      for (int c = 0; c < N; ++c) {
        const double left = tensorlog::half_to_float(h[(size_t)r * 2 * N + c]);
        const double right = tensorlog::half_to_float(h[(size_t)r * 2 * N + N + c]);
        const double want = left * (right / (1.0 + std::exp(-right)));
        const double got = tensorlog::half_to_float(ho[(size_t)r * N + c]);
        worst = std::fmax(worst, std::fabs(got - want) / (std::fabs(want) + 1e-2));
      }
    char d[64];
    std::snprintf(d, sizeof d, "(worst relative error %.2e)", worst);
    report("Activation", worst < 1e-3, d);  // one fp16 rounding: 2^-11
  }
  {  // Transpose: [rows, cols] -> [cols, rows], tails in both directions
    const int rows = 70, cols = 131;
    const auto h = random_halves((size_t)rows * cols, 4);
    DeviceBuf in(h), out((size_t)rows * cols);
    Transpose op;
    op.setName("transpose").setStream(stream);
    op.setInput(pllmTensor<half>(in.p, rows, cols, ROW)).setOutput(pllmTensor<half>(out.p, rows, cols, COL));
    op.config(rows, cols);
    op.run().log();
    HIP_CHECK(hipStreamSynchronize(stream));
    const auto ho = out.host();
    bool ok = true;
    for (int r = 0; r < rows; ++r)
      for (int c = 0; c < cols; ++c) ok &= ho[(size_t)c * rows + r] == h[(size_t)r * cols + c];
    report("Transpose", ok);
  }
  {  // CopyTensor
    const auto h = random_halves(12345, 5);
    DeviceBuf in(h), out(h.size());
    CopyTensor op;
    op.setName("copy").setStream(stream);
    op.setInput(pllmTensor<half>(in.p, h.size())).setOutput(pllmTensor<half>(out.p, h.size()));
    op.run().log();
    HIP_CHECK(hipStreamSynchronize(stream));
    report("CopyTensor", out.host() == h);
  }
  {  // SleepWrapper: the stream is busy for about the time asked for
    SleepWrapper op;
    op.setName("sleep").setStream(stream);
    hipEvent_t e0, e1;
    HIP_CHECK(hipEventCreate(&e0));
    HIP_CHECK(hipEventCreate(&e1));
    op.run();  // 10 us, as the reference's work()
    HIP_CHECK(hipEventRecord(e0, stream));
    op.sleep(stream, 3000);
    HIP_CHECK(hipEventRecord(e1, stream));
    HIP_CHECK(hipStreamSynchronize(stream));
    float ms = 0;
    HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
    char d[64];
    std::snprintf(d, sizeof d, "(3000 us asked, %.0f us taken)", ms * 1e3);
    report("SleepWrapper", ms >= 2.9f && ms < 50.f, d);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
  }
  (void)hipStreamDestroy(stream);
  return failures ? 1 : 0;
}
