// fp8 (OCP e4m3) x fp8 -> fp32 -> fp16 GEMM for gfx950 on v_mfma_f32_32x32x64_f8f6f4, with
// per-row activation scales and per-output-channel weight scales:
//
//   D[m][n] = half(alpha * sa[m] * sb[n] * sum_k Aq[m][k] * Bq[n][k] + beta * C[m][n])
//
// plus the row quantiser that produces (Aq, sa) from fp16 activations:
//   sa[m] = max_k |x[m][k]| / 448 (1 when the row is all zero),  Aq = e4m3_rne(x / sa[m]).
//
// Both operands are stored with k contiguous (Aq [M][K], Bq [N][K]: one row per output
// channel), so both are staged the same way: a slab is 128 k-bytes per row, written to LDS rows
// of 144 bytes (16-byte skew: conflict-free 16-byte fragment reads).  Workgroup = 256 threads
// = 4 wavefronts in a WM x WN grid; two LDS stages; while the two MFMA k-steps of slab i run,
// slab i+1 moves from registers to the other stage and slab i+2 is loaded into registers.
// The MFMA is issued as D^T = B.A^T so that a lane owns 4 consecutive output columns.
//
// A dot product does not depend on which k a lane slot holds as long as both operands use the
// same assignment; lane (l32, lg) slot s of k-step kk holds k = kk*64 + lg*32 + s for both.
#include "common.h"

namespace nf {

constexpr int F8_BK = 128;          // k-bytes per slab
constexpr int F8_LD = F8_BK + 16;   // LDS row pitch in bytes
constexpr uint32_t kOob8 = 0xFFFFFFF0u;

typedef int v8i32 __attribute__((ext_vector_type(8)));
typedef uint32_t bufvec4_8 __attribute__((ext_vector_type(4)));

template <int BM, int BN>
struct F8Smem {
  static constexpr int stage_bytes = (BM + BN) * F8_LD;
  static constexpr size_t bytes = 2 * (size_t)stage_bytes;
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc8(const void* p, size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)(uint32_t)bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 buf_load16_8(__amdgpu_buffer_rsrc_t r, uint32_t byte_off) {
  bufvec4_8 v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, 0);
  return u32x4{v.x, v.y, v.z, v.w};
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

__global__ __launch_bounds__(256) void quantize_rows_e4m3_kernel(const uint16_t* __restrict__ X,
                                                                 uint8_t* __restrict__ Xq,
                                                                 float* __restrict__ scale, int K) {
  __shared__ float red[4];
  const int row = blockIdx.x, tid = threadIdx.x;
  const u32x4* src = reinterpret_cast<const u32x4*>(X + (size_t)row * K);
  const int chunks = K / 8;
  float amax = 0.f;
  for (int c = tid; c < chunks; c += 256) {
    const u32x4 v = src[c];
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      amax = fmaxf(amax, fabsf(h2f_bits(w[i] & 0xffffu)));
      amax = fmaxf(amax, fabsf(h2f_bits(w[i] >> 16)));
    }
  }
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) amax = fmaxf(amax, __shfl_xor(amax, m, 64));
  if ((tid & 63) == 0) red[tid >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float s = amax > 0.f ? amax / 448.f : 1.f;
  if (tid == 0) scale[row] = s;
  u32x2* dst = reinterpret_cast<u32x2*>(Xq + (size_t)row * K);
  for (int c = tid; c < chunks; c += 256) {
    const u32x4 v = src[c];
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
    dst[c] = o;
  }
}

template <int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(256) void gemm_f8_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, const float* __restrict__ sa,
    const float* __restrict__ sb, const uint16_t* C, uint16_t* D, int M, int N, int K, float alpha,
    float beta, int tiles_m, int tiles_n) {
  using SM = F8Smem<BM, BN>;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  static_assert(WM * WN == 4, "four wavefronts");
  constexpr int A_CHUNKS = BM * 8 / 256;  // 16-byte chunks per thread per slab
  constexpr int B_CHUNKS = BN * 8 / 256;
  static_assert(A_CHUNKS >= 1 && B_CHUNKS >= 1, "tile too small for 256 threads");

  extern __shared__ __attribute__((aligned(16))) uint8_t smem8[];

  // XCD-aware tile order (workgroup ids round-robin over 8 XCDs): each XCD walks one
  // contiguous range of tiles, M fastest, so a weight panel stays in that XCD's L2.
  const int ntiles = tiles_m * tiles_n;
  const int per_xcd = (ntiles + 7) / 8;
  const int logical = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (logical >= ntiles) return;
  const int tile_m = logical % tiles_m, tile_n = logical / tiles_m;
  const int m_base = tile_m * BM, n_base = tile_n * BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int l32 = lane & 31, lg = lane >> 5;

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc8(A, (size_t)M * K);
  const __amdgpu_buffer_rsrc_t b_rsrc = make_rsrc8(B, (size_t)N * K);
  u32x4 a_reg[A_CHUNKS], b_reg[B_CHUNKS];
  uint32_t a_off[A_CHUNKS], b_off[B_CHUNKS];
  const int kc = tid & 7;  // this thread's 16-byte column within a slab row
#pragma unroll
  for (int i = 0; i < A_CHUNKS; ++i) {
    const int gm = m_base + ((tid + 256 * i) >> 3);
    a_off[i] = gm < M ? (uint32_t)gm * (uint32_t)K + kc * 16 : kOob8;
  }
#pragma unroll
  for (int i = 0; i < B_CHUNKS; ++i) {
    const int gn = n_base + ((tid + 256 * i) >> 3);
    b_off[i] = gn < N ? (uint32_t)gn * (uint32_t)K + kc * 16 : kOob8;
  }

  // part 0 / 1 = even / odd chunks (one half of the staging work per MFMA k-step); < 0 = all
  auto load_part = [&](int k0, int part) {
    const bool k_ok = k0 + kc * 16 < K;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      if (part >= 0 && (i & 1) != part) continue;
      a_reg[i] = buf_load16_8(a_rsrc, (k_ok && a_off[i] != kOob8) ? a_off[i] + (uint32_t)k0 : kOob8);
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i) {
      if (part >= 0 && (i & 1) != part) continue;
      b_reg[i] = buf_load16_8(b_rsrc, (k_ok && b_off[i] != kOob8) ? b_off[i] + (uint32_t)k0 : kOob8);
    }
  };
  auto store_part = [&](int stage, int part) {
    uint8_t* As = smem8 + stage * SM::stage_bytes;
    uint8_t* Bs = As + BM * F8_LD;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      if (part >= 0 && (i & 1) != part) continue;
      *reinterpret_cast<u32x4*>(As + ((tid + 256 * i) >> 3) * F8_LD + kc * 16) = a_reg[i];
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i) {
      if (part >= 0 && (i & 1) != part) continue;
      *reinterpret_cast<u32x4*>(Bs + ((tid + 256 * i) >> 3) * F8_LD + kc * 16) = b_reg[i];
    }
  };

  v8i32 af[2][TM], bf[2][TN];
  auto read32 = [&](const uint8_t* p) {
    const u32x4 lo = *reinterpret_cast<const u32x4*>(p);
    const u32x4 hi = *reinterpret_cast<const u32x4*>(p + 16);
    return v8i32{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
  };
  auto read_frags = [&](int stage, int kk, int buf) {
    const uint8_t* As = smem8 + stage * SM::stage_bytes;
    const uint8_t* Bs = As + BM * F8_LD;
#pragma unroll
    for (int i = 0; i < TM; ++i)
      af[buf][i] = read32(As + (wm * (BM / WM) + i * 32 + l32) * F8_LD + kk * 64 + lg * 32);
#pragma unroll
    for (int j = 0; j < TN; ++j)
      bf[buf][j] = read32(Bs + (wn * (BN / WN) + j * 32 + l32) * F8_LD + kk * 64 + lg * 32);
  };
  auto mfma_step = [&](int buf) {
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int i = 0; i < TM; ++i)
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf[buf][j], af[buf][i], acc[i][j],
                                                                    0, 0, 0, 0, 0, 0);
  };

  // Steady state of slab s (LDS stage s&1), two k-steps:
  //   step 0: prefetch step 1's fragments; write half of slab s+1 (held in registers) to the
  //           other stage and refill those registers from slab s+2;
  //   step 1: write the other half, barrier, prefetch slab s+1's first fragments, refill.
  auto slab = [&](int s, bool do_store, bool do_load) {
    const int cur = s & 1;
    read_frags(cur, 1, 1);
    if (do_store) store_part(cur ^ 1, 0);
    if (do_load) load_part((s + 2) * F8_BK, 0);
    mfma_step(0);
    if (do_store) store_part(cur ^ 1, 1);
    __syncthreads();
    if (do_store) read_frags(cur ^ 1, 0, 0);
    if (do_load) load_part((s + 2) * F8_BK, 1);
    mfma_step(1);
  };

  const int nslab = (K + F8_BK - 1) / F8_BK;
  load_part(0, -1);
  store_part(0, -1);
  if (nslab > 1) load_part(F8_BK, -1);
  __syncthreads();
  read_frags(0, 0, 0);
  int s = 0;
  for (; s + 2 < nslab; ++s) slab(s, true, true);
  if (s + 1 < nslab) {
    slab(s, true, false);
    ++s;
  }
  slab(s, false, false);

  // Epilogue: acc[i][j][r] is D[m][n] with m = tile row l32, n = (r/4)*8 + lg*4 + r%4.
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int gm = m_base + wm * (BM / WM) + i * 32 + l32;
    if (gm >= M) continue;
    const float row_scale = alpha * sa[gm];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const int gn = n_base + wn * (BN / WN) + j * 32 + qd * 8 + lg * 4;
        if (gn >= N) continue;  // N % 8 == 0 and gn % 4 == 0: the whole quad is in or out
        const float4_t cs = *reinterpret_cast<const float4_t*>(sb + gn);
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = row_scale * cs[e] * acc[i][j][qd * 4 + e];
        if (beta != 0.f) {
          const u32x2 c = *reinterpret_cast<const u32x2*>(C + (size_t)gm * N + gn);
          v[0] += beta * h2f_bits(c.x & 0xffffu);
          v[1] += beta * h2f_bits(c.x >> 16);
          v[2] += beta * h2f_bits(c.y & 0xffffu);
          v[3] += beta * h2f_bits(c.y >> 16);
        }
        u32x2 o;
        o.x = f2h_bits(v[0]) | (f2h_bits(v[1]) << 16);
        o.y = f2h_bits(v[2]) | (f2h_bits(v[3]) << 16);
        *reinterpret_cast<u32x2*>(D + (size_t)gm * N + gn) = o;
      }
    }
  }
}

template <int BM, int BN, int WM, int WN>
static int launch_gemm_f8(const uint8_t* A, const uint8_t* B, const float* sa, const float* sb,
                          const uint16_t* C, uint16_t* D, int M, int N, int K, float alpha, float beta,
                          hipStream_t stream) {
  using SM = F8Smem<BM, BN>;
  auto kern = gemm_f8_kernel<BM, BN, WM, WN>;
  static bool attr_set = false;  // benign race: the call is idempotent
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)SM::bytes);
    if (e != hipSuccess) {
      set_error("gemm_f8: cannot reserve %zu bytes of LDS: %s", SM::bytes, hipGetErrorString(e));
      return NF_ERR_RUNTIME;
    }
    attr_set = true;
  }
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const int grid = ((tiles_m * tiles_n + 7) / 8) * 8;
  kern<<<grid, 256, SM::bytes, stream>>>(A, B, sa, sb, C, D, M, N, K, alpha, beta, tiles_m, tiles_n);
  return check_launch("gemm_f8 launch");
}

}  // namespace nf

using namespace nf;

extern "C" {

int nf_quantize_rows_e4m3(const uint16_t* X, uint8_t* Xq, float* row_scale, int M, int K,
                          nf_stream_t stream) {
  NF_REQUIRE(M >= 0 && K > 0 && K % 16 == 0, "nf_quantize_rows_e4m3: bad shape M=%d K=%d (K %% 16)", M, K);
  NF_REQUIRE(M == 0 || (X && Xq && row_scale), "nf_quantize_rows_e4m3: null pointer");
  NF_REQUIRE(((uintptr_t)X | (uintptr_t)Xq) % 16 == 0, "nf_quantize_rows_e4m3: operands must be 16-byte aligned");
  if (M == 0) return NF_OK;
  quantize_rows_e4m3_kernel<<<M, 256, 0, (hipStream_t)stream>>>(X, Xq, row_scale, K);
  return check_launch("quantize_rows_e4m3 launch");
}

int nf_gemm_f8_f16(const uint8_t* Aq, const float* a_scale, const uint8_t* Bq, const float* b_scale,
                   const uint16_t* C, uint16_t* D, int M, int N, int K, float alpha, float beta,
                   nf_stream_t stream) {
  NF_REQUIRE(M >= 0 && N > 0 && K > 0, "nf_gemm_f8_f16: bad shape M=%d N=%d K=%d", M, N, K);
  NF_REQUIRE(K % 16 == 0 && N % 8 == 0, "nf_gemm_f8_f16: K=%d must be a multiple of 16 and N=%d of 8", K, N);
  NF_REQUIRE(M == 0 || (Aq && a_scale && Bq && b_scale && D), "nf_gemm_f8_f16: null pointer");
  NF_REQUIRE(((uintptr_t)Aq | (uintptr_t)Bq | (uintptr_t)b_scale) % 16 == 0 && ((uintptr_t)D | (uintptr_t)C) % 8 == 0,
             "nf_gemm_f8_f16: Aq, Bq, b_scale must be 16-byte and C, D 8-byte aligned");
  NF_REQUIRE(beta == 0.f || C, "nf_gemm_f8_f16: beta=%g needs C", (double)beta);
  NF_REQUIRE((size_t)M * K < 0xFFFFFF00ull && (size_t)N * K < 0xFFFFFF00ull,
             "nf_gemm_f8_f16: an operand of %d x %d x %d exceeds the 4 GiB buffer-addressing limit", M, N, K);
  if (M == 0) return NF_OK;
  hipStream_t s = (hipStream_t)stream;
  auto tiles = [&](int bm, int bn) { return (long long)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
  if (M <= 64) return launch_gemm_f8<64, 256, 1, 4>(Aq, Bq, a_scale, b_scale, C, D, M, N, K, alpha, beta, s);
  if (tiles(256, 256) >= 224) return launch_gemm_f8<256, 256, 2, 2>(Aq, Bq, a_scale, b_scale, C, D, M, N, K, alpha, beta, s);
  if (tiles(128, 256) >= 224 || M <= 128) return launch_gemm_f8<128, 256, 2, 2>(Aq, Bq, a_scale, b_scale, C, D, M, N, K, alpha, beta, s);
  return launch_gemm_f8<128, 128, 2, 2>(Aq, Bq, a_scale, b_scale, C, D, M, N, K, alpha, beta, s);
}

size_t nf_gemm_f8w_workspace_bytes(int M, int K) {
  if (M <= 0 || K <= 0) return 0;
  return ((size_t)M * K + 255) / 256 * 256 + (size_t)M * sizeof(float);
}

int nf_gemm_f8w_f16(const uint16_t* A, const uint8_t* Bq, const float* b_scale, const uint16_t* C,
                    uint16_t* D, int M, int N, int K, float alpha, float beta, void* workspace,
                    size_t workspace_bytes, nf_stream_t stream) {
  NF_REQUIRE(M >= 0 && K > 0, "nf_gemm_f8w_f16: bad shape M=%d K=%d", M, K);
  if (M == 0) return NF_OK;
  const size_t need = nf_gemm_f8w_workspace_bytes(M, K);
  if (!workspace || workspace_bytes < need) {
    set_error("nf_gemm_f8w_f16: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    return NF_ERR_WORKSPACE;
  }
  NF_REQUIRE((uintptr_t)workspace % 16 == 0, "nf_gemm_f8w_f16: workspace must be 16-byte aligned");
  uint8_t* Aq = static_cast<uint8_t*>(workspace);
  float* sa = reinterpret_cast<float*>(Aq + ((size_t)M * K + 255) / 256 * 256);
  int rc = nf_quantize_rows_e4m3(A, Aq, sa, M, K, stream);
  if (rc) return rc;
  return nf_gemm_f8_f16(Aq, sa, Bq, b_scale, C, D, M, N, K, alpha, beta, stream);
}

}  // extern "C"
