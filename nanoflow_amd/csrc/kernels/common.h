// Internal helpers shared by the gfx950 kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <type_traits>
#include <utility>

#include "nanoflow_kernels.h"

namespace nf {

void set_error(const char* fmt, ...);

#define NF_REQUIRE(cond, ...)              \
  do {                                     \
    if (!(cond)) {                         \
      nf::set_error(__VA_ARGS__);          \
      return NF_ERR_INVALID_ARGUMENT;      \
    }                                      \
  } while (0)

// Launch errors (bad configuration etc.) surface through hipGetLastError.
inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: %s", what, hipGetErrorString(e));
    return NF_ERR_RUNTIME;
  }
  return NF_OK;
}

constexpr int kWave = 64;

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

struct alignas(16) u32x4 {
  uint32_t x, y, z, w;
};
struct alignas(8) u32x2 {
  uint32_t x, y;
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) v += __shfl_xor(v, m, 64);
  return v;
}

// Sum over the shares of a GEMM split over K, for 4 neighbouring outputs: P[s * mn + at .. +3],
// s = 0 .. shares-1 (at most kMaxShares), added in that order.  Every load is issued before the
// first addition, so the lane waits for one memory round trip instead of one per share.
constexpr int kMaxShares = 16;
__device__ __forceinline__ float4_t sum_shares(const float* __restrict__ P, size_t mn, size_t at, int shares) {
  float4_t p[kMaxShares];
#pragma unroll
  for (int s = 0; s < kMaxShares; ++s)
    if (s < shares) p[s] = *reinterpret_cast<const float4_t*>(P + s * mn + at);
  float4_t v = p[0];
#pragma unroll
  for (int s = 1; s < kMaxShares; ++s)
    if (s < shares) v += p[s];
  return v;
}

__device__ __forceinline__ float h2f_bits(uint32_t bits16) {
  return __half2float(__ushort_as_half((unsigned short)bits16));
}
__device__ __forceinline__ uint32_t f2h_bits(float f) {
  return (uint32_t)__half_as_ushort(__float2half_rn(f));
}

// Round-to-nearest-even OCP e4m3 (bias 7, no infinities, max 448), saturating.
__device__ __forceinline__ uint32_t f32_to_e4m3(float x) {
  const uint32_t u = __float_as_uint(x);
  const uint32_t sign = (u >> 24) & 0x80u;
  const float a = fabsf(x);
  uint32_t code;
  if (!(a < 464.f)) {
    code = 0x7Eu;                                // 448; also where NaN ends up
  } else if (a < 0.015625f) {
    code = (uint32_t)(int)rintf(a * 512.f);      // subnormals: steps of 2^-9 (8 -> smallest normal)
  } else {
    uint32_t ua = __float_as_uint(a);
    ua += 0x7FFFFu + ((ua >> 20) & 1u);          // RNE at mantissa bit 20
    code = (((ua >> 23) - 120u) << 3) | ((ua >> 20) & 7u);
  }
  return sign | code;
}
// Eight halves (a 16-byte chunk) divided by s and rounded to e4m3: 8 bytes.
__device__ __forceinline__ u32x2 quantize_chunk_e4m3(const u32x4& v, float s) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  uint32_t q[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    q[2 * i] = f32_to_e4m3(h2f_bits(w[i] & 0xffffu) / s);
    q[2 * i + 1] = f32_to_e4m3(h2f_bits(w[i] >> 16) / s);
  }
  u32x2 o;
  o.x = q[0] | (q[1] << 8) | (q[2] << 16) | (q[3] << 24);
  o.y = q[4] | (q[5] << 8) | (q[6] << 16) | (q[7] << 24);
  return o;
}
// Two floats rounded to nearest-even fp16, lo in bits 15:0 (one v_cvt_pk_f16_f32 on gfx950).
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, f16x2_t));
}

// ---- global memory -> LDS without passing through registers (gfx950 buffer_load ... lds)
typedef short short4_t __attribute__((ext_vector_type(4)));

// The accumulators of G adjacent 16x16 MFMA tiles are kept as ONE vector of 4 G floats (a register
// tuple the allocator places as a unit, like a 32x32 tile's 16), and a tile's 4 floats are taken
// out of it and put back by constant shuffles, which cost no instruction: as 64 separate 4-float
// values the compiler assigned them differently on either side of the slab loop's back edge and
// permuted all 256 accumulator registers once per slab.
template <int G> struct AccVec;
template <> struct AccVec<1> { typedef float4_t type; };
template <> struct AccVec<2> { typedef float type __attribute__((ext_vector_type(8))); };
template <> struct AccVec<4> { typedef float16_t type; };
template <int Q, class V, int... I>
__device__ __forceinline__ float4_t acc_get_impl(const V& v, std::integer_sequence<int, I...>) {
  return __builtin_shufflevector(v, v, (4 * Q + I)...);
}
template <int Q, class V>
__device__ __forceinline__ float4_t acc_get(const V& v) {
  return acc_get_impl<Q>(v, std::make_integer_sequence<int, 4>{});
}
template <int Q, int N, class V, int... I>
__device__ __forceinline__ void acc_put_impl(V& v, float4_t c, std::integer_sequence<int, I...>) {
  const V w = __builtin_shufflevector(c, c, (I < 4 ? I : -1)...);                       // c widened to N floats
  v = __builtin_shufflevector(v, w, ((I >= 4 * Q && I < 4 * Q + 4) ? N + I - 4 * Q : I)...);
}
template <int Q, int N, class V>
__device__ __forceinline__ void acc_put(V& v, float4_t c) {
  acc_put_impl<Q, N>(v, c, std::make_integer_sequence<int, N>{});
}

// Out-of-range per-lane offsets read as zero (also into LDS), so tile edges need no branches:
// out-of-range chunks just get the kOob offset.  Only the per-lane offset is range-checked by
// the hardware, so the whole address stays in it.
constexpr uint32_t kOob = 0xFFFFFFF0u;
typedef uint32_t rsrc_t __attribute__((ext_vector_type(4)));  // raw buffer descriptor (4 SGPRs)
__device__ __forceinline__ rsrc_t make_rsrc(const void* p, size_t bytes) {
  const uint64_t a = (uint64_t)p;
  return rsrc_t{(uint32_t)a, (uint32_t)(a >> 32), (uint32_t)bytes, 0x00020000u};
}
// 64 lanes x 16 bytes -> LDS [lds_addr, lds_addr + 1024); lds_addr (a byte address inside LDS)
// must be the same for the whole wavefront.  Written as inline assembly on purpose: for the
// builtin form the compiler makes every later LDS read wait for ALL outstanding loads
// (vmcnt(0)), because it cannot tell the stage being filled from the stage being read, and
// that serialises the loads with the MFMAs.  The kernel waits itself (wait_loads below).
// M0 carries the LDS address and is declared clobbered (the compiler warns that M0 is a reserved
// register; the clobber still tells its M0-initialisation merging that the value changed, so the
// warning is switched off in the build flags).
__device__ __forceinline__ void load16_to_lds(rsrc_t r, uint32_t byte_off, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :: "s"(lds_addr), "v"(byte_off), "s"(r) : "memory", "m0");
}
// The same with the non-temporal hint: data that is read once (the K and V pages of decode
// attention) should not displace what the caches hold.  Measured on MI355X for 64 KiB pages read
// as 256-byte rows: 6.0 -> 6.65 TB/s; for a contiguous stream 6.3 -> 7.07 TB/s.  (Operands that ARE re-read through the caches lose
// by it: the GEMM kernels run 5-15 % slower with the hint on either operand.)
__device__ __forceinline__ void load16_to_lds_nt(rsrc_t r, uint32_t byte_off, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen nt lds"
               :: "s"(lds_addr), "v"(byte_off), "s"(r) : "memory", "m0");
}
// The same with the LDS address given as a wavefront-uniform base plus a compile-time constant.
template <int kLdsOffset>
__device__ __forceinline__ void load16_to_lds(rsrc_t r, uint32_t byte_off, uint32_t lds_base) {
  asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :: "s"(lds_base), "v"(byte_off), "s"(r), "n"(kLdsOffset) : "memory", "scc", "m0");
}
__device__ __forceinline__ short4_t lds_read_tr16(const uint8_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)p);
}

// Compile-time loop: f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N-1>{}).
template <int V>
using ic = std::integral_constant<int, V>;
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(ic<I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

}  // namespace nf
