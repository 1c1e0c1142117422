// fp16 x fp16 -> fp32 -> fp16 GEMM family for gfx950 on v_mfma_f32_32x32x16_f16.
//
//   D = half(alpha * A.B + beta * C)                     (plain; QKV, O, down, LM head)
//   D = half(silu(half(A.Bg)) * half(A.Bu))              (dual; gate/up SwiGLU)
//
// Workgroup = 256 threads = 4 wavefronts in a WM x WN grid; each wavefront owns a
// (BM/WM) x (BN/WN) block of 32x32 MFMA tiles.  K is walked in slabs of 64 through two LDS
// stages: while the MFMAs of slab i run out of LDS stage i&1, the global loads of slab i+1
// are in flight into registers and are written to the other stage afterwards (one barrier per
// slab).
//
// LDS layouts (both conflict-free for the accesses used):
//   A slab  As[BM][64+8]           row = m, k contiguous; 16-byte fragment reads.
//   B slab  Bs[16][BN+2][4]        "k-quad major": quad q holds k = 4q..4q+3 for every n as one
//                                  8-byte cell.  A row-major [K,N] weight tile is loaded as
//                                  4(k) x 8(n) register blocks (four coalesced 16-byte loads),
//                                  transposed in registers with 16 byte-permutes and stored as
//                                  64 contiguous bytes; an MFMA operand is two 8-byte reads.
//
// The MFMA is issued as D^T = B^T.A^T (weights as the first operand) so that each lane ends up
// with 4 consecutive output columns of one row -> 8-byte stores/loads for D and C.
#include "common.h"

namespace nf {

constexpr int BK = 64;                 // K slab
constexpr int A_LD = BK + 8;           // halves per As row (144 B: 16-byte aligned, bank-skewed)
constexpr int NQ = BK / 4;             // k-quads per slab

template <int BM, int BN, int NB>
struct GemmSmem {
  static constexpr int B_LD = BN + 2;  // 8-byte cells per quad row (+2 cells = 16 B skew)
  static constexpr int a_halves = BM * A_LD;
  static constexpr int b_halves = NQ * B_LD * 4;
  static constexpr int stage_halves = a_halves + NB * b_halves;
  static constexpr size_t bytes = 2 * (size_t)stage_halves * sizeof(uint16_t);
};

__device__ __forceinline__ uint32_t pack_lo(uint32_t x, uint32_t y) {
  return __builtin_amdgcn_perm(y, x, 0x05040100u);  // {x.lo, y.lo}
}
__device__ __forceinline__ uint32_t pack_hi(uint32_t x, uint32_t y) {
  return __builtin_amdgcn_perm(y, x, 0x07060302u);  // {x.hi, y.hi}
}

// Raw buffer loads: an offset at or past the descriptor's byte count reads as zero, so tile
// edges need no branches -- out-of-range chunks just get the kOob offset.
constexpr uint32_t kOob = 0xFFFFFFF0u;
typedef uint32_t bufvec4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)(uint32_t)bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 buf_load16(__amdgpu_buffer_rsrc_t r, uint32_t byte_off) {
  bufvec4 v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, 0);
  return u32x4{v.x, v.y, v.z, v.w};
}

// SiLU(g)*u on values already rounded to fp16, as the reference's dual epilogue computes it.
__device__ __forceinline__ float swiglu_rounded(float g_acc, float u_acc) {
  float g = __half2float(__float2half_rn(g_acc));
  float u = __half2float(__float2half_rn(u_acc));
  return g / (1.0f + __expf(-g)) * u;
}

// kDual: two weight matrices, SwiGLU epilogue.  kBCol: weights stored [N][K].
template <int BM, int BN, int WM, int WN, bool kDual, bool kBCol>
__global__ __launch_bounds__(256) void gemm_f16_kernel(
    const uint16_t* __restrict__ A, const uint16_t* __restrict__ B0,
    const uint16_t* __restrict__ B1, const uint16_t* C, uint16_t* D,
    int M, int N, int K, float alpha, float beta, int tiles_m, int tiles_n) {
  constexpr int NB = kDual ? 2 : 1;
  using SM = GemmSmem<BM, BN, NB>;
  constexpr int B_LD = SM::B_LD;
  constexpr int TM = BM / WM / 32;  // MFMA tiles per wave along M
  constexpr int TN = BN / WN / 32;
  static_assert(WM * WN == 4, "four wavefronts");
  constexpr int A_CHUNKS = BM * (BK / 8) / 256;     // 16-byte chunks per thread per slab
  constexpr int B_BLOCKS = (BK / 4) * (BN / 8) / 256;  // 4x8 blocks per thread per slab (row-major B)
  constexpr int BC_CHUNKS = BN * (BK / 8) / 256;    // 16-byte chunks per thread (col-major B)
  static_assert(A_CHUNKS >= 1 && B_BLOCKS >= 1, "tile too small for 256 threads");

  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];

  // XCD-aware tile order: consecutive workgroup ids land on different XCDs (8 of them), so
  // give each XCD one contiguous range of tiles, M fastest, to share weight panels in its L2.
  const int ntiles = tiles_m * tiles_n;
  const int per_xcd = (ntiles + 7) / 8;
  const int logical = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (logical >= ntiles) return;
  const int tile_m = logical % tiles_m, tile_n = logical / tiles_m;
  const int m_base = tile_m * BM, n_base = tile_n * BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int l32 = lane & 31, lg = lane >> 5;

  float16_t acc[NB][TM][TN];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[b][i][j][r] = 0.f;

  // ---- staging registers: one slab's worth of this thread's global chunks
  constexpr int B_UNITS = kBCol ? BC_CHUNKS : B_BLOCKS;  // per weight matrix
  constexpr int B_LOADS = kBCol ? 1 : 4;                  // 16-byte loads per B unit
  u32x4 a_reg[A_CHUNKS];
  u32x4 b_reg[NB][B_UNITS * B_LOADS];

  // Per-thread byte offsets of the chunks it stages, at k0 = 0 (kOob when the row / column is
  // outside the matrix); the slab offset is added per iteration.
  const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(A, (size_t)M * K * 2);
  __amdgpu_buffer_rsrc_t b_rsrc[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) b_rsrc[b] = make_rsrc(b ? B1 : B0, (size_t)N * K * 2);
  uint32_t a_off[A_CHUNKS];
#pragma unroll
  for (int i = 0; i < A_CHUNKS; ++i) {
    const int id = tid + 256 * i;
    const int gm = m_base + (id >> 3);
    a_off[i] = gm < M ? ((uint32_t)gm * (uint32_t)K + (id & 7) * 8) * 2u : kOob;
  }
  uint32_t b_off[B_UNITS];
#pragma unroll
  for (int i = 0; i < B_UNITS; ++i) {
    const int id = tid + 256 * i;
    if constexpr (kBCol) {
      const int gn = n_base + (id >> 3);
      b_off[i] = gn < N ? ((uint32_t)gn * (uint32_t)K + (id & 7) * 8) * 2u : kOob;
    } else {
      const int gn = n_base + (id % (BN / 8)) * 8;
      b_off[i] = gn < N ? ((uint32_t)(id / (BN / 8)) * 4u * (uint32_t)N + gn) * 2u : kOob;
    }
  }

  // The staging work of a slab is cut into 3 parts (quarter q of the MFMA loop handles the
  // A chunks with i % 3 == q and the B units with (2 - u % 3) == q); part < 0 = everything.
  auto load_part = [&](int k0, int part) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      if (part >= 0 && i % 3 != part) continue;
      const bool ok = a_off[i] != kOob && k0 + ((tid + 256 * i) & 7) * 8 < K;
      a_reg[i] = buf_load16(a_rsrc, ok ? a_off[i] + (uint32_t)k0 * 2u : kOob);
    }
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int i = 0; i < B_UNITS; ++i) {
        if (part >= 0 && 2 - (b * B_UNITS + i) % 3 != part) continue;
        if constexpr (kBCol) {
          const bool ok = b_off[i] != kOob && k0 + ((tid + 256 * i) & 7) * 8 < K;
          b_reg[b][i] = buf_load16(b_rsrc[b], ok ? b_off[i] + (uint32_t)k0 * 2u : kOob);
        } else {
          const int kq = (tid + 256 * i) / (BN / 8);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const bool ok = b_off[i] != kOob && k0 + kq * 4 + r < K;
            b_reg[b][i * 4 + r] =
                buf_load16(b_rsrc[b], ok ? b_off[i] + ((uint32_t)(k0 + r) * (uint32_t)N) * 2u : kOob);
          }
        }
      }
  };

  auto store_part = [&](int stage, int part) {
    uint16_t* As = smem + stage * SM::stage_halves;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      if (part >= 0 && i % 3 != part) continue;
      const int id = tid + 256 * i;
      *reinterpret_cast<u32x4*>(As + (id >> 3) * A_LD + (id & 7) * 8) = a_reg[i];
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      uint16_t* Bs = As + SM::a_halves + b * SM::b_halves;
#pragma unroll
      for (int i = 0; i < B_UNITS; ++i) {
        if (part >= 0 && 2 - (b * B_UNITS + i) % 3 != part) continue;
        const int id = tid + 256 * i;
        if constexpr (kBCol) {
          const int n = id >> 3, kc = id & 7;
          const u32x4 v = b_reg[b][i];
          *reinterpret_cast<u32x2*>(Bs + ((2 * kc) * B_LD + n) * 4) = u32x2{v.x, v.y};
          *reinterpret_cast<u32x2*>(Bs + ((2 * kc + 1) * B_LD + n) * 4) = u32x2{v.z, v.w};
        } else {
          const int nb = id % (BN / 8), kq = id / (BN / 8);
          const u32x4 r0 = b_reg[b][i * 4 + 0], r1 = b_reg[b][i * 4 + 1];
          const u32x4 r2 = b_reg[b][i * 4 + 2], r3 = b_reg[b][i * 4 + 3];
          // cell(n) = {B[k0][n], B[k1][n], B[k2][n], B[k3][n]}; n = nb*8 + 0..7
          u32x4 o0, o1, o2, o3;
          o0.x = pack_lo(r0.x, r1.x); o0.y = pack_lo(r2.x, r3.x);  // n+0
          o0.z = pack_hi(r0.x, r1.x); o0.w = pack_hi(r2.x, r3.x);  // n+1
          o1.x = pack_lo(r0.y, r1.y); o1.y = pack_lo(r2.y, r3.y);  // n+2
          o1.z = pack_hi(r0.y, r1.y); o1.w = pack_hi(r2.y, r3.y);  // n+3
          o2.x = pack_lo(r0.z, r1.z); o2.y = pack_lo(r2.z, r3.z);  // n+4
          o2.z = pack_hi(r0.z, r1.z); o2.w = pack_hi(r2.z, r3.z);  // n+5
          o3.x = pack_lo(r0.w, r1.w); o3.y = pack_lo(r2.w, r3.w);  // n+6
          o3.z = pack_hi(r0.w, r1.w); o3.w = pack_hi(r2.w, r3.w);  // n+7
          u32x4* dst = reinterpret_cast<u32x4*>(Bs + (kq * B_LD + nb * 8) * 4);
          dst[0] = o0; dst[1] = o1; dst[2] = o2; dst[3] = o3;
        }
      }
    }
  };

  // ---- MFMA operand fragments, double-buffered across the 4 k-steps of a slab
  half8_t af[2][TM];
  half8_t bf[2][NB][TN];
  auto read_frags = [&](int stage, int kk, int buf) {
    const uint16_t* As = smem + stage * SM::stage_halves;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = wm * (BM / WM) + i * 32 + l32;
      af[buf][i] = *reinterpret_cast<const half8_t*>(As + row * A_LD + kk * 16 + lg * 8);
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const uint16_t* Bs = As + SM::a_halves + b * SM::b_halves;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int n = wn * (BN / WN) + j * 32 + l32;
        const int q = kk * 4 + lg * 2;
        half4_t lo = *reinterpret_cast<const half4_t*>(Bs + (q * B_LD + n) * 4);
        half4_t hi = *reinterpret_cast<const half4_t*>(Bs + ((q + 1) * B_LD + n) * 4);
        bf[buf][b][j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      }
    }
  };
  auto mfma_step = [&](int buf) {
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int i = 0; i < TM; ++i)
          acc[b][i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[buf][b][j], af[buf][i], acc[b][i][j], 0, 0, 0);
  };

  // One slab of the steady state.  While the MFMAs of slab s run out of LDS stage s&1:
  //   quarters 0-2: prefetch the next k-step's fragments; write slab s+1 (already in
  //                 registers) into the other stage; refill those registers with slab s+2;
  //   quarter 3:    barrier, then prefetch slab s+1's first fragments under the last MFMAs.
  auto slab = [&](int s, bool do_store, bool do_load) {
    const int cur = s & 1;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      if (kk == 3) __syncthreads();
      if (kk < 3) read_frags(cur, kk + 1, (kk + 1) & 1);
      else if (do_store) read_frags(cur ^ 1, 0, 0);
      if (kk < 3) {
        if (do_store) store_part(cur ^ 1, kk);
        if (do_load) load_part((s + 2) * BK, kk);
      }
      mfma_step(kk & 1);
    }
  };

  const int nslab = (K + BK - 1) / BK;
  load_part(0, -1);
  store_part(0, -1);
  if (nslab > 1) load_part(BK, -1);
  __syncthreads();
  read_frags(0, 0, 0);
  int s = 0;
  for (; s + 2 < nslab; ++s) slab(s, true, true);
  if (s + 1 < nslab) {
    slab(s, true, false);
    ++s;
  }
  slab(s, false, false);

  // Epilogue.  acc[.][i][j][r] holds D[m][n] with m = tile row l32 and
  // n = (r/4)*8 + lg*4 + r%4 of the 32x32 tile: 4 consecutive n per register quad.
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int gm = m_base + wm * (BM / WM) + i * 32 + l32;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const int gn = n_base + wn * (BN / WN) + j * 32 + qd * 8 + lg * 4;
        if (gn >= N) continue;  // N % 8 == 0 and gn % 4 == 0: the whole quad is in or out
        float v[4];
        if constexpr (kDual) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            v[e] = swiglu_rounded(acc[0][i][j][qd * 4 + e], acc[1][i][j][qd * 4 + e]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = alpha * acc[0][i][j][qd * 4 + e];
          if (beta != 0.f) {
            const u32x2 c = *reinterpret_cast<const u32x2*>(C + (size_t)gm * N + gn);
            v[0] += beta * h2f_bits(c.x & 0xffffu);
            v[1] += beta * h2f_bits(c.x >> 16);
            v[2] += beta * h2f_bits(c.y & 0xffffu);
            v[3] += beta * h2f_bits(c.y >> 16);
          }
        }
        u32x2 o;
        o.x = f2h_bits(v[0]) | (f2h_bits(v[1]) << 16);
        o.y = f2h_bits(v[2]) | (f2h_bits(v[3]) << 16);
        *reinterpret_cast<u32x2*>(D + (size_t)gm * N + gn) = o;
      }
    }
  }
}

template <int BM, int BN, int WM, int WN, bool kDual, bool kBCol>
static int launch_gemm(const uint16_t* A, const uint16_t* B0, const uint16_t* B1, const uint16_t* C,
                       uint16_t* D, int M, int N, int K, float alpha, float beta,
                       hipStream_t stream) {
  using SM = GemmSmem<BM, BN, kDual ? 2 : 1>;
  auto kern = gemm_f16_kernel<BM, BN, WM, WN, kDual, kBCol>;
  static bool attr_set = false;  // benign race: the call is idempotent
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)SM::bytes);
    if (e != hipSuccess) {
      set_error("gemm: cannot reserve %zu bytes of LDS: %s", SM::bytes, hipGetErrorString(e));
      return NF_ERR_RUNTIME;
    }
    attr_set = true;
  }
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const int ntiles = tiles_m * tiles_n;
  const int grid = ((ntiles + 7) / 8) * 8;
  kern<<<grid, 256, SM::bytes, stream>>>(A, B0, B1, C, D, M, N, K, alpha, beta, tiles_m, tiles_n);
  return check_launch("gemm launch");
}

// Tile choice: the largest tile that still yields at least ~one workgroup per CU (256 CUs);
// short M uses a 64-row tile so the padding rows do not dominate.
template <bool kBCol>
static int dispatch_plain(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D,
                          int M, int N, int K, float alpha, float beta, hipStream_t s) {
  auto tiles = [&](int bm, int bn) { return (long long)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
  if (M <= 64) return launch_gemm<64, 256, 1, 4, false, kBCol>(A, B, nullptr, C, D, M, N, K, alpha, beta, s);
  if (tiles(256, 256) >= 224) return launch_gemm<256, 256, 2, 2, false, kBCol>(A, B, nullptr, C, D, M, N, K, alpha, beta, s);
  if (tiles(128, 256) >= 224 || M <= 128) return launch_gemm<128, 256, 2, 2, false, kBCol>(A, B, nullptr, C, D, M, N, K, alpha, beta, s);
  return launch_gemm<128, 128, 2, 2, false, kBCol>(A, B, nullptr, C, D, M, N, K, alpha, beta, s);
}

}  // namespace nf

using namespace nf;

static int check_gemm_args(const char* who, const void* A, const void* B, const void* D, int M,
                           int N, int K) {
  NF_REQUIRE(M >= 0 && N > 0 && K > 0, "%s: bad shape M=%d N=%d K=%d", who, M, N, K);
  NF_REQUIRE(K % 8 == 0 && N % 8 == 0, "%s: K=%d and N=%d must be multiples of 8", who, K, N);
  NF_REQUIRE(M == 0 || (A && B && D), "%s: null pointer", who);
  NF_REQUIRE(((uintptr_t)A | (uintptr_t)B | (uintptr_t)D) % 16 == 0,
             "%s: operands must be 16-byte aligned", who);
  // operands are addressed through 32-bit buffer offsets
  NF_REQUIRE((size_t)M * K * 2 < 0xFFFFFF00ull && (size_t)N * K * 2 < 0xFFFFFF00ull,
             "%s: an operand of %d x %d x %d exceeds the 4 GiB buffer-addressing limit", who, M, N, K);
  return NF_OK;
}

extern "C" {

int nf_gemm_f16(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int M, int N,
                int K, float alpha, float beta, int b_col_major, nf_stream_t stream) {
  int rc = check_gemm_args("nf_gemm_f16", A, B, D, M, N, K);
  if (rc) return rc;
  NF_REQUIRE(beta == 0.f || C, "nf_gemm_f16: beta=%g needs C", (double)beta);
  NF_REQUIRE(((uintptr_t)C) % 8 == 0, "nf_gemm_f16: C must be 8-byte aligned");
  if (M == 0) return NF_OK;
  hipStream_t s = (hipStream_t)stream;
  return b_col_major ? dispatch_plain<true>(A, B, C, D, M, N, K, alpha, beta, s)
                     : dispatch_plain<false>(A, B, C, D, M, N, K, alpha, beta, s);
}

int nf_dual_swiglu_f16(const uint16_t* A, const uint16_t* Bgate, const uint16_t* Bup, uint16_t* out,
                       int M, int N, int K, nf_stream_t stream) {
  int rc = check_gemm_args("nf_dual_swiglu_f16", A, Bgate, out, M, N, K);
  if (rc) return rc;
  NF_REQUIRE(M == 0 || Bup, "nf_dual_swiglu_f16: null pointer");
  NF_REQUIRE(((uintptr_t)Bup) % 16 == 0, "nf_dual_swiglu_f16: operands must be 16-byte aligned");
  if (M == 0) return NF_OK;
  hipStream_t s = (hipStream_t)stream;
  if (M <= 64)
    return launch_gemm<64, 128, 1, 4, true, false>(A, Bgate, Bup, nullptr, out, M, N, K, 1.f, 0.f, s);
  const long long t256 = (long long)((M + 255) / 256) * ((N + 127) / 128);
  if (t256 >= 224)
    return launch_gemm<256, 128, 2, 2, true, false>(A, Bgate, Bup, nullptr, out, M, N, K, 1.f, 0.f, s);
  return launch_gemm<128, 128, 2, 2, true, false>(A, Bgate, Bup, nullptr, out, M, N, K, 1.f, 0.f, s);
}

}  // extern "C"
