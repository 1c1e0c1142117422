// Internal helpers shared by the gfx950 kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

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

__device__ __forceinline__ float h2f_bits(uint32_t bits16) {
  return __half2float(__ushort_as_half((unsigned short)bits16));
}
__device__ __forceinline__ uint32_t f2h_bits(float f) {
  return (uint32_t)__half_as_ushort(__float2half_rn(f));
}

}  // namespace nf
