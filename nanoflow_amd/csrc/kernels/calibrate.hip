// Calibration micro-benchmarks: what THIS device sustains with nothing in the way, so that the
// kernels' rates can be reported against measured ceilings as well as against the published ones.
//
//   nf_calibrate_mfma      a register-only loop of independent v_mfma_f32_32x32x16_f16 (or
//                          32x32x64 fp8) instructions, one wavefront per SIMD like the GEMM kernels,
//                          on zero operands (the least switching activity: the highest clock the
//                          part holds) or on pseudo-random ones (what a GEMM on N(0,1) data feeds
//                          the matrix pipe), or (random_operands = 2, fp16) on pseudo-random operands
//                          that every wavefront re-reads from LDS before each 16 MFMAs, as the main
//                          loop of the 256x256 GEMM tile does (8 reads of 16 bytes per lane): the
//                          matrix pipe plus the fragment traffic, still without a byte from memory;
//                          or (3) with the operand loads of that tile beside them as well (64 KB
//                          per workgroup per 64 MFMAs, straight into LDS, from a window the L2
//                          holds): the GEMM's main loop without barriers, prologue or epilogue;
//                          or (4) as 1 on v_mfma_f32_16x16x32_f16;
//                          reports TFLOP/s and the shader clock the wavefronts saw (shader-clock
//                          ticks over real-time ticks).
//   nf_calibrate_hbm_read  every CU streams its share of a buffer far larger than the last-level
//                          cache with 16-byte loads; reports GB/s.
//   nf_calibrate_paged_read  the access pattern of paged decode attention without its arithmetic:
//                          (request, kv head) workgroups walk a page table and pull 256-byte K and
//                          V rows of 64 KiB pages straight into LDS.
// No counterpart in the reference (its benchmarks quote vendor peaks).
#include <algorithm>

#include "common.h"

namespace nf {

typedef int v8i32 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x;
}

// 16 independent 32x32 accumulators per wavefront (the register tile of the 256x256 GEMM), 4 + 4
// operand fragments that never change: the matrix pipe is the only unit at work.
template <bool kF8>
__global__ __launch_bounds__(256) void calib_mfma_kernel(int iters, int random_operands, uint64_t* clocks,
                                                         float* sink) {
  const uint32_t gid = blockIdx.x * 256u + threadIdx.x;
  float16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  v8i32 a8[4], b8[4];
  half8_t a16[4], b16[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t ha = mix32(gid * 64u + i * 8u + e), hb = mix32(gid * 64u + 32u + i * 8u + e);
      if constexpr (kF8) {
        // four e4m3 codes per word, exponent field kept below 8 (|x| < 1) so sums stay finite
        a8[i][e] = random_operands ? (int)(ha & 0xb7b7b7b7u) : 0;
        b8[i][e] = random_operands ? (int)(hb & 0xb7b7b7b7u) : 0;
      } else {
        // uniform in (-1, 1)
        a16[i][e] = random_operands ? (_Float16)(((int)(ha >> 8) - (1 << 23)) * (1.0f / (1 << 23))) : (_Float16)0.f;
        b16[i][e] = random_operands ? (_Float16)(((int)(hb >> 8) - (1 << 23)) * (1.0f / (1 << 23))) : (_Float16)0.f;
      }
    }
  }
  const uint64_t c0 = __builtin_readcyclecounter(), r0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if constexpr (kF8)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b8[j], a8[i], acc[i][j], 0, 0, 0, 0, 0, 0);
        else
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b16[j], a16[i], acc[i][j], 0, 0, 0);
      }
  }
  const uint64_t c1 = __builtin_readcyclecounter(), r1 = wall_clock64();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) s += acc[i][j][r];
  sink[gid & 1023u] = s;  // keeps the loop alive; the value is never read
  if (threadIdx.x == 0 && blockIdx.x < 64) {
    clocks[blockIdx.x * 2 + 0] = c1 - c0;
    clocks[blockIdx.x * 2 + 1] = r1 - r0;
  }
}

// The same flops from v_mfma_f32_16x16x32_f16: 64 independent 16x16 accumulators (the 128x128
// register tile again), 8 + 8 operand fragments that never change, pseudo-random operands; one
// pass of its loop is two passes of calib_mfma_kernel's.
template <bool kF8>
__global__ __launch_bounds__(256) void calib_mfma16_kernel(int iters, uint64_t* clocks, float* sink) {
  const uint32_t gid = blockIdx.x * 256u + threadIdx.x;
  float4_t acc[8][8];
  half8_t a[8], b[8];
  v8i32 a8[8], b8[8];  // kF8: v_mfma_f32_16x16x128_f8f6f4 on e4m3 codes with |x| < 1
#pragma unroll
  for (int i = 0; i < 8; ++i) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t ha = mix32(gid * 128u + i * 8u + e), hb = mix32(gid * 128u + 64u + i * 8u + e);
      a[i][e] = (_Float16)(((int)(ha >> 8) - (1 << 23)) * (1.0f / (1 << 23)));
      b[i][e] = (_Float16)(((int)(hb >> 8) - (1 << 23)) * (1.0f / (1 << 23)));
      a8[i][e] = (int)(ha & 0xb7b7b7b7u);
      b8[i][e] = (int)(hb & 0xb7b7b7b7u);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
  }
  const uint64_t c0 = __builtin_readcyclecounter(), r0 = wall_clock64();
  for (int it = 0; it < iters; it += 2)
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if constexpr (kF8)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b8[j], a8[i], acc[i][j], 0, 0, 0, 0, 0, 0);
        else
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b[j], a[i], acc[i][j], 0, 0, 0);
      }
  const uint64_t c1 = __builtin_readcyclecounter(), r1 = wall_clock64();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) s += acc[i][j][r];
  sink[gid & 1023u] = s;
  if (threadIdx.x == 0 && blockIdx.x < 64) {
    clocks[blockIdx.x * 2 + 0] = c1 - c0;
    clocks[blockIdx.x * 2 + 1] = r1 - r0;
  }
}

// The same 16 accumulators, with the 4 + 4 operand fragments of every 16 MFMAs read from LDS one
// step ahead (two sets of pseudo-random fragments per wavefront, taken in turn): what the matrix
// pipe sustains when it is fed the way the GEMM's main loop feeds it.
__device__ __forceinline__ half8_t lds_read16(uint32_t addr) {
  rsrc_t v;
  asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr));
  return __builtin_bit_cast(half8_t, v);
}
// kLoads = 1: every wavefront also issues 4 direct-to-LDS loads of 1 KB per 16 MFMAs (the 64 KB a
// 256x256 tile fetches per 64-deep slab), from a 2 MB window of `src` that 64 workgroups share and
// the L2 holds, into a second 64 KB of LDS, with at most two steps of loads in flight.
template <int kLoads>
__global__ __launch_bounds__(256) void calib_mfma_lds_kernel(int iters, uint64_t* clocks, float* sink,
                                                             const uint8_t* __restrict__ src) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];  // 64 KB of fragments (+ 64 KB of landing area)
  const uint32_t gid = blockIdx.x * 256u + threadIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int c = 0; c < 16; ++c) {  // 256 bytes of fragments per thread
    half8_t v;
#pragma unroll
    for (int e = 0; e < 8; ++e)
      v[e] = (_Float16)(((int)(mix32(gid * 128u + c * 8u + e) >> 8) - (1 << 23)) * (1.0f / (1 << 23)));
    *reinterpret_cast<half8_t*>(smem + (c * 256 + threadIdx.x) * 16) = v;
  }
  __syncthreads();
  float16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  // the wavefront's 16 KB: fragment f of set s at s * 8192 + f * 1024 + lane * 16
  const uint32_t base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem + wave * 16384 + lane * 16;
  half8_t a[2][4], b[2][4];
#pragma unroll
  for (int f = 0; f < 4; ++f) {
    a[0][f] = lds_read16(base + f * 1024);
    b[0][f] = lds_read16(base + (4 + f) * 1024);
  }
  constexpr uint32_t kWindow = 2u << 20;
  const rsrc_t rsrc = make_rsrc(kLoads ? src + (size_t)(blockIdx.x / 8 % 4) * kWindow : nullptr, kLoads ? kWindow : 0);
  const uint32_t land = __builtin_amdgcn_readfirstlane(
      (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem + 65536 + wave * 1024);
  uint32_t goff = (uint32_t)(wave * 1024 + lane * 16);
  const uint64_t c0 = __builtin_readcyclecounter(), r0 = wall_clock64();
  for (int it = 0; it < iters; it += 2) {
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      if constexpr (kLoads == 1) {
        asm volatile("s_waitcnt vmcnt(4)" ::: "memory");  // the loads of the step before last have landed
#pragma unroll
        for (int q = 0; q < 4; ++q)
          load16_to_lds(rsrc, goff + (uint32_t)q * 4096u, land + (uint32_t)s * 32768u + (uint32_t)q * 4096u);
        goff = (goff + 16384u) & (kWindow - 1);
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // set s, requested one step ago
#pragma unroll
      for (int f = 0; f < 4; ++f) {
        a[s ^ 1][f] = lds_read16(base + (s ^ 1) * 8192 + f * 1024);
        b[s ^ 1][f] = lds_read16(base + (s ^ 1) * 8192 + (4 + f) * 1024);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b[s][j], a[s][i], acc[i][j], 0, 0, 0);
    }
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  const uint64_t c1 = __builtin_readcyclecounter(), r1 = wall_clock64();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) s += acc[i][j][r];
#pragma unroll
  for (int f = 0; f < 4; ++f) s += (float)a[0][f][0] + (float)b[0][f][0];  // the last reads are consumed too
  sink[gid & 1023u] = s;
  if (threadIdx.x == 0 && blockIdx.x < 64) {
    clocks[blockIdx.x * 2 + 0] = c1 - c0;
    clocks[blockIdx.x * 2 + 1] = r1 - r0;
  }
}

// Workgroup w reads bytes [w * span, (w + 1) * span) with its 256 lanes striding 4 KB per
// instruction, 8 loads in flight per lane.
__global__ __launch_bounds__(256) void calib_hbm_read_kernel(const rsrc_t* __restrict__ buf, size_t vec_per_block,
                                                             uint32_t* sink) {
  const rsrc_t* p = buf + (size_t)blockIdx.x * vec_per_block + threadIdx.x;
  uint32_t x = 0;
  size_t i = 0;
  for (; i + 8 * 256 <= vec_per_block; i += 8 * 256) {
    rsrc_t v[8];  // a 16-byte vector of four words
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(p + i + u * 256);
#pragma unroll
    for (int u = 0; u < 8; ++u) x ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  if (x == 0x9e3779b9u) sink[blockIdx.x & 1023] = x;  // practically never true; keeps the loads alive
}

// Paged decode attention's traffic without its arithmetic.  Workgroup = (request, kv head), in
// the attention kernel's order; 2 wavefronts take alternate 32-key steps; a step pulls 32 K rows
// and 32 V rows of 256 bytes (two pages each) straight into the wavefront's LDS ring of 2 K + 2 V
// tiles (non-temporal loads, as the attention kernel issues them), and waits only for the tile it
// is about to reuse.
__global__ __launch_bounds__(128) void calib_paged_read_kernel(const uint16_t* __restrict__ pool,
                                                               const int32_t* __restrict__ kv_indptr,
                                                               const int32_t* __restrict__ kv_indices,
                                                               const int32_t* __restrict__ kv_last_page_len,
                                                               int batch, int num_kv_heads, uint32_t* sink) {
  __shared__ __attribute__((aligned(1024))) uint8_t smem[2 * 4 * 8192];
  // (request, head) of a workgroup id as attn_decode_kernel orders its items: inside groups of 8
  // requests (head, request), so that one XCD starts the heads of one request together
  int req = blockIdx.x / num_kv_heads, head = blockIdx.x % num_kv_heads;
  if ((int)blockIdx.x < (batch / 8) * 8 * num_kv_heads) {
    const int j = blockIdx.x % (8 * num_kv_heads);
    req = (int)(blockIdx.x / (8 * num_kv_heads)) * 8 + j % 8;
    head = j / 8;
  }
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int p0 = kv_indptr[req], p1 = kv_indptr[req + 1];
  const int kv_len = (p1 - p0 - 1) * 16 + kv_last_page_len[req];
  const int steps = (kv_len + 31) / 32;
  const uint32_t lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem + wave * 4 * 8192;
  const size_t page_halves = (size_t)2 * 16 * num_kv_heads * 128;
  const uint32_t row_stride = (uint32_t)num_kv_heads * 256u;   // bytes between the entries of a page
  // lane -> (row = lane / 16 of 4 rows per instruction, 16-byte chunk = lane % 16)
  const uint32_t lane_off = (uint32_t)(lane >> 4) * row_stride + (uint32_t)head * 256u + (uint32_t)(lane & 15) * 16u;
  int issued = 0;
  for (int s = wave; s < steps; s += 2, ++issued) {
    const int slot = issued & 1;
    if (issued >= 2) __builtin_amdgcn_s_waitcnt(0x4070);  // vmcnt(16), lgkmcnt(0): the step before last has landed
#pragma unroll
    for (int half = 0; half < 2; ++half) {  // the two pages of a 32-key step
      const int pi = p0 + s * 2 + half;
      if (pi >= p1) break;
      const uint16_t* page = pool + (size_t)kv_indices[pi] * page_halves;
      const rsrc_t rk = make_rsrc(page, page_halves * 2);
#pragma unroll
      for (int kv = 0; kv < 2; ++kv)
#pragma unroll
        for (int t = 0; t < 4; ++t)  // 4 rows per instruction, 16 rows per page
          load16_to_lds_nt(rk, (uint32_t)kv * 16u * row_stride + (uint32_t)t * 4u * row_stride + lane_off,
                        lds + (uint32_t)(kv * 2 + slot) * 8192u + (uint32_t)(half * 4 + t) * 1024u);
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0070);
  __syncthreads();
  if (smem[threadIdx.x * 16] == 0xA5 && smem[8191] == 0x5A && kv_len == -1) sink[0] = 1;  // keeps LDS alive
}

}  // namespace nf

using namespace nf;

namespace {
struct EventPair {
  hipEvent_t a = nullptr, b = nullptr;
  bool ok() { return hipEventCreate(&a) == hipSuccess && hipEventCreate(&b) == hipSuccess; }
  ~EventPair() {
    if (a) (void)hipEventDestroy(a);
    if (b) (void)hipEventDestroy(b);
  }
};
int device_cus() {
  int dev = 0, v = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
    v = 256;
  return v;
}
}  // namespace

extern "C" {

int nf_calibrate_mfma(int fp8, int random_operands, int iters, void* scratch, size_t scratch_bytes, double* tflops,
                      double* clock_mhz, nf_stream_t stream) {
  NF_REQUIRE(iters > 0 && scratch && scratch_bytes >= 8192 && tflops && clock_mhz, "nf_calibrate_mfma: bad arguments");
  NF_REQUIRE(random_operands >= 0 && random_operands <= 4 && !(fp8 && (random_operands == 2 || random_operands == 3)),
             "nf_calibrate_mfma: random_operands = %d (0, 1, 4 = 1 with 16x16 MFMAs, or fp16 only: 2 = operands "
             "re-read from LDS, 3 = and operand loads from L2 into LDS beside them)", random_operands);
  const bool l2_loads = random_operands == 3;
  NF_REQUIRE(!l2_loads || scratch_bytes >= 8192 + ((size_t)8 << 20),
             "nf_calibrate_mfma: random_operands = 3 reads 8 MiB of scratch behind its first 8192 bytes");
  if (random_operands == 4) iters = (iters + 1) / 2 * 2;
  if (random_operands == 2 || l2_loads) {
    iters = (iters + 1) / 2 * 2;
    for (auto k : {reinterpret_cast<const void*>(calib_mfma_lds_kernel<0>), reinterpret_cast<const void*>(calib_mfma_lds_kernel<1>)})
      if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 131072) != hipSuccess) {
        set_error("nf_calibrate_mfma: cannot reserve 128 KB of LDS");
        return NF_ERR_RUNTIME;
      }
  }
  hipStream_t s = (hipStream_t)stream;
  uint64_t* clocks = static_cast<uint64_t*>(scratch);                       // 64 x 2 x 8 bytes
  float* sink = reinterpret_cast<float*>(static_cast<uint8_t*>(scratch) + 2048);  // 1024 floats
  NF_REQUIRE(scratch_bytes >= 2048 + 4096, "nf_calibrate_mfma: scratch of %zu bytes is too small", scratch_bytes);
  const int grid = device_cus() * 4;
  EventPair ev;
  if (!ev.ok()) {
    set_error("nf_calibrate_mfma: cannot create events");
    return NF_ERR_RUNTIME;
  }
  auto launch = [&](int n) {
    if (random_operands == 2) calib_mfma_lds_kernel<0><<<grid, 256, 65536, s>>>((n + 1) / 2 * 2, clocks, sink, nullptr);
    else if (random_operands == 3)
      calib_mfma_lds_kernel<1><<<grid, 256, 131072, s>>>((n + 1) / 2 * 2, clocks, sink,
                                                         static_cast<const uint8_t*>(scratch) + 8192);
    else if (random_operands == 4 && fp8) calib_mfma16_kernel<true><<<grid, 256, 0, s>>>((n + 1) / 2 * 2, clocks, sink);
    else if (random_operands == 4) calib_mfma16_kernel<false><<<grid, 256, 0, s>>>((n + 1) / 2 * 2, clocks, sink);
    else if (fp8) calib_mfma_kernel<true><<<grid, 256, 0, s>>>(n, random_operands, clocks, sink);
    else calib_mfma_kernel<false><<<grid, 256, 0, s>>>(n, random_operands, clocks, sink);
  };
  launch(std::max(iters / 8, 1));  // warm-up: clocks and power state settle
  (void)hipEventRecord(ev.a, s);
  launch(iters);
  (void)hipEventRecord(ev.b, s);
  int rc = check_launch("nf_calibrate_mfma launch");
  if (rc) return rc;
  if (hipEventSynchronize(ev.b) != hipSuccess) {
    set_error("nf_calibrate_mfma: the kernel failed");
    return NF_ERR_RUNTIME;
  }
  float ms = 0;
  (void)hipEventElapsedTime(&ms, ev.a, ev.b);
  uint64_t h[128];
  if (hipMemcpy(h, clocks, sizeof(h), hipMemcpyDeviceToHost) != hipSuccess) {
    set_error("nf_calibrate_mfma: cannot read the clock samples");
    return NF_ERR_RUNTIME;
  }
  double ratio = 0;
  for (int b = 0; b < 64; ++b) ratio += h[2 * b + 1] ? (double)h[2 * b] / (double)h[2 * b + 1] : 0.0;
  *clock_mhz = ratio / 64 * 100.0;  // the real-time counter ticks at 100 MHz
  const double flop_per_mfma = fp8 ? 2.0 * 32 * 32 * 64 : 2.0 * 32 * 32 * 16;
  *tflops = (double)grid * 4 * iters * 16 * flop_per_mfma / (ms * 1e-3) / 1e12;
  return NF_OK;
}

int nf_calibrate_hbm_read(const void* buf, size_t bytes, int reps, void* scratch, size_t scratch_bytes, double* gbps,
                          nf_stream_t stream) {
  NF_REQUIRE(buf && reps > 0 && scratch && scratch_bytes >= 4096 && gbps && (uintptr_t)buf % 16 == 0,
             "nf_calibrate_hbm_read: bad arguments");
  hipStream_t s = (hipStream_t)stream;
  const int grid = device_cus() * 8;
  const size_t vec_per_block = bytes / 16 / grid / (8 * 256) * (8 * 256);
  NF_REQUIRE(vec_per_block > 0, "nf_calibrate_hbm_read: %zu bytes are too few for %d workgroups", bytes, grid);
  EventPair ev;
  if (!ev.ok()) {
    set_error("nf_calibrate_hbm_read: cannot create events");
    return NF_ERR_RUNTIME;
  }
  auto launch = [&] {
    calib_hbm_read_kernel<<<grid, 256, 0, s>>>(static_cast<const rsrc_t*>(buf), vec_per_block, static_cast<uint32_t*>(scratch));
  };
  launch();
  (void)hipEventRecord(ev.a, s);
  for (int r = 0; r < reps; ++r) launch();
  (void)hipEventRecord(ev.b, s);
  int rc = check_launch("nf_calibrate_hbm_read launch");
  if (rc) return rc;
  if (hipEventSynchronize(ev.b) != hipSuccess) {
    set_error("nf_calibrate_hbm_read: the kernel failed");
    return NF_ERR_RUNTIME;
  }
  float ms = 0;
  (void)hipEventElapsedTime(&ms, ev.a, ev.b);
  *gbps = (double)vec_per_block * 16 * grid * reps / (ms * 1e-3) / 1e9;
  return NF_OK;
}

int nf_calibrate_paged_read(const uint16_t* kv_data, const int32_t* kv_indptr, const int32_t* kv_indices,
                            const int32_t* kv_last_page_len, int batch, int num_kv_heads, size_t kv_bytes_per_launch,
                            int reps, void* scratch, size_t scratch_bytes, double* gbps, nf_stream_t stream) {
  NF_REQUIRE(kv_data && kv_indptr && kv_indices && kv_last_page_len && batch > 0 && num_kv_heads > 0 && reps > 0 &&
                 scratch && scratch_bytes >= 4096 && gbps,
             "nf_calibrate_paged_read: bad arguments");
  hipStream_t s = (hipStream_t)stream;
  EventPair ev;
  if (!ev.ok()) {
    set_error("nf_calibrate_paged_read: cannot create events");
    return NF_ERR_RUNTIME;
  }
  auto launch = [&] {
    calib_paged_read_kernel<<<batch * num_kv_heads, 128, 0, s>>>(kv_data, kv_indptr, kv_indices, kv_last_page_len,
                                                                 batch, num_kv_heads, static_cast<uint32_t*>(scratch));
  };
  launch();
  (void)hipEventRecord(ev.a, s);
  for (int r = 0; r < reps; ++r) launch();
  (void)hipEventRecord(ev.b, s);
  int rc = check_launch("nf_calibrate_paged_read launch");
  if (rc) return rc;
  if (hipEventSynchronize(ev.b) != hipSuccess) {
    set_error("nf_calibrate_paged_read: the kernel failed");
    return NF_ERR_RUNTIME;
  }
  float ms = 0;
  (void)hipEventElapsedTime(&ms, ev.a, ev.b);
  *gbps = (double)kv_bytes_per_launch * reps / (ms * 1e-3) / 1e9;
  return NF_OK;
}

}  // extern "C"
