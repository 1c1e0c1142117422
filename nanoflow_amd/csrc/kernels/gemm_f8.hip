// fp8 (OCP e4m3) x fp8 -> fp32 -> fp16 GEMM for gfx950 on v_mfma_f32_32x32x64_f8f6f4, with
// per-row activation scales and per-output-channel weight scales:
//
//   D[m][n] = half(alpha * sa[m] * sb[n] * sum_k Aq[m][k] * Bq[n][k] + beta * C[m][n])
//
// plus the row quantiser that produces (Aq, sa) from fp16 activations:
//   sa[m] = max_k |x[m][k]| / 448 (1 when the row is all zero),  Aq = e4m3_rne(x / sa[m]).
//
// Both operands are stored with k contiguous (Aq [M][K], Bq [N][K]: one row per output
// channel), so both are staged the same way: a slab is 128 k-bytes per row, moved from global
// memory straight into LDS (buffer_load ... lds, XOR-swizzled rows, multi-stage ring -- the
// scheme of gemm.hip with both operands in its row form).  Workgroup = 256 threads = 4
// wavefronts in a WM x WN grid.  The MFMA is issued as D^T = B.A^T so that a lane owns 4
// consecutive output columns.
//
// A dot product does not depend on which k a lane slot holds as long as both operands use the
// same assignment; lane (l32, lg) slot s of k-step kk holds k = kk*64 + lg*32 + s for both.
#include <algorithm>
#include <type_traits>

#include "common.h"

namespace nf {

constexpr int F8_BK = 128;  // k-bytes per slab = one 128-byte LDS row per matrix row

typedef int v8i32 __attribute__((ext_vector_type(8)));

template <int BM, int BN, int NB>
struct F8Smem {
  static constexpr int stage_bytes = (BM + NB * BN) * 128;
  static constexpr int stages = (144 * 1024) / stage_bytes > 4 ? 4 : (144 * 1024) / stage_bytes;
  static_assert(stages >= 2, "tile too large for two LDS stages");
  static constexpr size_t bytes = (size_t)stages * stage_bytes;
};

// One workgroup per row.  kChunks > 0: the row (at most kChunks x 256 chunks of 8 halves) stays in
// registers between the maximum and the rounding, so it is read once; kChunks == 0: any length, the
// second pass reads the row again.
template <int kChunks>
__global__ __launch_bounds__(256) void quantize_rows_e4m3_kernel(const uint16_t* __restrict__ X,
                                                                 uint8_t* __restrict__ Xq,
                                                                 float* __restrict__ scale, int K) {
  __shared__ float red[4];
  const int row = blockIdx.x, tid = threadIdx.x;
  const u32x4* src = reinterpret_cast<const u32x4*>(X + (size_t)row * K);
  const int chunks = K / 8;
  constexpr int kHeld = kChunks > 0 ? kChunks : 1;
  u32x4 held[kHeld];
  float amax = 0.f;
  auto chunk_max = [&](const u32x4& v) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      amax = fmaxf(amax, fabsf(h2f_bits(w[i] & 0xffffu)));
      amax = fmaxf(amax, fabsf(h2f_bits(w[i] >> 16)));
    }
  };
  if constexpr (kChunks > 0) {
#pragma unroll
    for (int u = 0; u < kChunks; ++u)
      if (tid + u * 256 < chunks) held[u] = src[tid + u * 256];
#pragma unroll
    for (int u = 0; u < kChunks; ++u)
      if (tid + u * 256 < chunks) chunk_max(held[u]);
  } else {
    for (int c = tid; c < chunks; c += 256) chunk_max(src[c]);
  }
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) amax = fmaxf(amax, __shfl_xor(amax, m, 64));
  if ((tid & 63) == 0) red[tid >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float s = amax > 0.f ? amax / 448.f : 1.f;
  if (tid == 0) scale[row] = s;
  u32x2* dst = reinterpret_cast<u32x2*>(Xq + (size_t)row * K);
  if constexpr (kChunks > 0) {
#pragma unroll
    for (int u = 0; u < kChunks; ++u)
      if (tid + u * 256 < chunks) dst[tid + u * 256] = quantize_chunk_e4m3(held[u], s);
  } else {
    for (int c = tid; c < chunks; c += 256) dst[c] = quantize_chunk_e4m3(src[c], s);
  }
}

// Weight quantiser: W fp16 [K][N] (the pipeline's weight orientation) -> Wq e4m3 [N][K] (one row
// per output channel, k contiguous) with scale[n] = max_k |W[k][n]| / 448 (1 for an all-zero
// column), Wq[n][k] = e4m3_rne(W[k][n] / scale[n]): the row quantiser applied to the transpose.
// First the column maxima (64 columns per workgroup, rows read in 128-byte runs) ...
__global__ __launch_bounds__(256) void weight_col_scale_kernel(const uint16_t* __restrict__ W,
                                                               float* __restrict__ scale, int K, int N) {
  __shared__ float red[8][64];
  const int tid = threadIdx.x, c2 = tid & 31, r = tid >> 5;
  const int n = blockIdx.x * 64 + 2 * c2;
  float a0 = 0.f, a1 = 0.f;
  if (n < N)
    for (int k = r; k < K; k += 8) {
      const uint32_t w = *reinterpret_cast<const uint32_t*>(W + (size_t)k * N + n);
      a0 = fmaxf(a0, fabsf(h2f_bits(w & 0xffffu)));
      a1 = fmaxf(a1, fabsf(h2f_bits(w >> 16)));
    }
  red[r][2 * c2] = a0;
  red[r][2 * c2 + 1] = a1;
  __syncthreads();
  if (tid < 64 && blockIdx.x * 64 + tid < N) {
    float a = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) a = fmaxf(a, red[i][tid]);
    scale[blockIdx.x * 64 + tid] = a > 0.f ? a / 448.f : 1.f;
  }
}

// ... then 64 x 64 tiles are quantised on the way into LDS and written out transposed, 16 bytes
// of one output channel per thread.
__global__ __launch_bounds__(256) void weight_quantize_transpose_kernel(const uint16_t* __restrict__ W,
                                                                        const float* __restrict__ scale,
                                                                        uint8_t* __restrict__ Wq, int K, int N) {
  __shared__ __attribute__((aligned(16))) uint8_t tile[64][64 + 16];  // [n][k]
  const int tid = threadIdx.x, c2 = tid & 31, r = tid >> 5;
  const int k0 = blockIdx.x * 64, n0 = blockIdx.y * 64;
  const int n = n0 + 2 * c2;
  float s0 = 1.f, s1 = 1.f;
  if (n < N) {
    s0 = scale[n];
    s1 = scale[n + 1];
  }
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    const int kl = p * 8 + r, k = k0 + kl;
    uint32_t w = 0;
    if (n < N && k < K) w = *reinterpret_cast<const uint32_t*>(W + (size_t)k * N + n);
    tile[2 * c2][kl] = (uint8_t)f32_to_e4m3(h2f_bits(w & 0xffffu) / s0);
    tile[2 * c2 + 1][kl] = (uint8_t)f32_to_e4m3(h2f_bits(w >> 16) / s1);
  }
  __syncthreads();
  const int nl = tid >> 2, kc = (tid & 3) * 16;
  if (n0 + nl < N && k0 + kc < K)  // K % 16 == 0: a chunk is inside or outside as a whole
    *reinterpret_cast<u32x4*>(Wq + (size_t)(n0 + nl) * K + k0 + kc) = *reinterpret_cast<const u32x4*>(&tile[nl][kc]);
}

// SiLU(g) * u on products already rounded to fp16, as the fp16 dual kernel's epilogue does it.
__device__ __forceinline__ float swiglu_rounded_f16(float g_acc, float u_acc) {
  const float g = __half2float(__float2half_rn(g_acc));
  const float u = __half2float(__float2half_rn(u_acc));
  return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * u;
}

// kDual: two weight matrices B (gate) and B1 (up) with scales sb and sb1,
//   D[m][n] = half(silu(g) * u),  g = half(sa[m] * sb[n] * sum_k Aq.Bq),  u = half(sa[m] * sb1[n] * sum_k Aq.B1q);
// alpha, beta and C are not used.
// kPartial: one share of a GEMM split over K (see gemm.hip).  Workgroup (tile, share) sums over
// k in [share * k_per, ...) and stores the fp32 sums, unscaled, to D taken as float
// [shares][M][N] (kDual: the sums of the second product to C taken the same way); Kt is then the
// whole contraction (the row stride of both operands), shares and k_per describe the split.
template <int BM, int BN, int WM, int WN, bool kDual, bool kPartial = false>
__global__ __launch_bounds__(256) void gemm_f8_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, const uint8_t* __restrict__ B1,
    const float* __restrict__ sa, const float* __restrict__ sb, const float* __restrict__ sb1,
    const uint16_t* C, uint16_t* D, int M, int N, int Kt, float alpha, float beta, int tiles_m, int tiles_n,
    int shares, int k_per) {
  constexpr int NB = kDual ? 2 : 1;
  using SM = F8Smem<BM, BN, NB>;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  static_assert(WM * WN == 4, "four wavefronts");
  constexpr int A_LOADS = BM / 32;  // 1 KB (8 rows) load instructions per wave per slab
  constexpr int B_LOADS = BN / 32;  // ... per weight matrix
  constexpr int NS = SM::stages;
  constexpr int LOADS = A_LOADS + NB * B_LOADS;
  // k-steps the loads of one slab are spread over; with two stages they must land within one step
  constexpr int PARTS = NS == 2 ? 1 : 2;

  extern __shared__ __attribute__((aligned(1024))) uint8_t smem8[];
  const uint32_t smem_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem8;

  // XCD-aware tile order (workgroup ids round-robin over 8 XCDs): each XCD walks one
  // contiguous range of tiles, M fastest, so a weight panel stays in that XCD's L2.
  const int ntiles = tiles_m * tiles_n * (kPartial ? shares : 1);
  const int per_xcd = (ntiles + 7) / 8;
  int logical = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (logical >= ntiles) return;
  int K = Kt;                       // extent of this workgroup's contraction
  const int lda = Kt;               // row stride of both operands (k contiguous)
  size_t p_off = 0;                 // this share's slice of the partial sums
  if constexpr (kPartial) {
    const int share = logical % shares;
    logical /= shares;
    const int k0 = share * k_per;
    K = Kt - k0 < k_per ? Kt - k0 : k_per;
    A += k0;
    B += k0;
    if constexpr (kDual) B1 += k0;
    p_off = (size_t)share * M * N;
  }
  const int tile_m = logical % tiles_m, tile_n = logical / tiles_m;
  const int m_base = tile_m * BM, n_base = tile_n * BN;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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

  // Both operands are rows of 128 k-bytes; they go from global memory straight into LDS
  // (see gemm.hip): 8 rows per load instruction, row r keeping its logical 16-byte chunk c at
  // position c ^ ((r >> 1) & 7) (bit 3 of the row number is the wave's parity).  One running
  // offset per load instruction, advanced by a slab after each use; rows past the operand's last
  // one lie at or past the end of the buffer and read as zero, which leaves only k >= K inside a
  // row to be masked.
  const rsrc_t a_rsrc = make_rsrc(A, (size_t)(M - 1) * lda + K);
  const rsrc_t b_rsrc[2] = {make_rsrc(B, (size_t)(N - 1) * lda + K), make_rsrc(kDual ? B1 : B, (size_t)(N - 1) * lda + K)};
  const int kc = ((lane & 7) ^ (((lane >> 4) & 3) | ((wave & 1) << 2))) * 16;  // k-byte of this lane's chunk inside the slab
  uint32_t a_off[A_LOADS], b_off[NB][B_LOADS];
#pragma unroll
  for (int t = 0; t < A_LOADS; ++t)
    a_off[t] = (uint32_t)(m_base + (t * 4 + wave) * 8 + (lane >> 3)) * (uint32_t)lda + kc;
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int t = 0; t < B_LOADS; ++t)
      b_off[b][t] = (uint32_t)(n_base + (t * 4 + wave) * 8 + (lane >> 3)) * (uint32_t)lda + kc;
  auto load_one = [&](auto t_c, uint32_t st, bool k_ok) {
    constexpr int t = decltype(t_c)::value;
    if constexpr (t < A_LOADS) {
      load16_to_lds<t * 4096>(a_rsrc, k_ok ? a_off[t] : kOob, st);
      a_off[t] += F8_BK;
    } else {
      constexpr int b = (t - A_LOADS) / B_LOADS, tt = (t - A_LOADS) % B_LOADS;
      load16_to_lds<(BM + b * BN) * 128 + tt * 4096>(b_rsrc[b], k_ok ? b_off[b][tt] : kOob, st);
      b_off[b][tt] += F8_BK;
    }
  };
  auto load_slab = [&](int stage, int k0) {
    const uint32_t st = __builtin_amdgcn_readfirstlane(smem_lds + stage * SM::stage_bytes + wave * 1024);
    const bool k_ok = k0 + kc < K;
    static_for<LOADS>([&](auto t_c) { load_one(t_c, st, k_ok); });
  };

  // MFMA operand of k-step kk: 32 bytes of row r = the logical chunks 4kk + 2lg and + 1, which
  // sit at positions p and p ^ 1 with p = (4kk + 2lg) ^ ((r >> 1) & 7).
  const uint32_t a_rd = (uint32_t)(wm * (BM / WM) + l32) * 128u;
  const uint32_t b_rd = (uint32_t)(BM * 128 + (wn * (BN / WN) + l32) * 128);
  uint32_t swz[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) swz[kk] = (uint32_t)(((kk * 4 + lg * 2) ^ ((l32 >> 1) & 7)) << 4);
  v8i32 af[2][TM], bf[2][NB][TN];
  auto read32 = [&](const uint8_t* p, uint32_t pos) {
    const u32x4 lo = *reinterpret_cast<const u32x4*>(p + pos);
    const u32x4 hi = *reinterpret_cast<const u32x4*>(p + (pos ^ 16u));
    return v8i32{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
  };
  constexpr int READS = TM + NB * TN;
  auto read_one = [&](auto q_c, auto kk_c, auto buf_c, const uint8_t* st) {
    constexpr int q = decltype(q_c)::value, kk = decltype(kk_c)::value, buf = decltype(buf_c)::value;
    if constexpr (q < TM) {
      af[buf][q] = read32(st + a_rd + q * 32 * 128, swz[kk]);
    } else {
      constexpr int b = (q - TM) / TN, j = (q - TM) % TN;
      bf[buf][b][j] = read32(st + b_rd + (b * BN + j * 32) * 128, swz[kk]);
    }
  };

  // One k-step: its MFMAs (64 cycles of the matrix pipe each) with the loads LP, LP + PARTS, ...
  // of the slab being fetched (LP < 0: none) and the fragment reads of k-step RK (RK < 0: none)
  // dealt out between them, order pinned -- the scheme of gemm.hip.
  constexpr int NM = NB * TN * TM;
  auto step = [&](auto kk_c, auto lp_c, auto rk_c, uint32_t ld_st, bool ld_ok, const uint8_t* rd_st) {
    constexpr int kk = decltype(kk_c)::value, LP = decltype(lp_c)::value, RK = decltype(rk_c)::value;
    constexpr int NL = LP < 0 ? 0 : (LOADS - LP + PARTS - 1) / PARTS;
    constexpr int NR = RK < 0 ? 0 : READS;
    constexpr int S = NL + NR;
    static_for<NM>([&](auto n_c) {
      constexpr int n = decltype(n_c)::value;
      constexpr int b = n / (TN * TM), j = n / TM % TN, i = n % TM;
      acc[b][i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf[kk][b][j], af[kk][i], acc[b][i][j], 0, 0, 0, 0, 0, 0);
      constexpr int lo = n * S / NM, hi = (n + 1) * S / NM;
      static_for<hi - lo>([&](auto d_c) {
        constexpr int q = lo + decltype(d_c)::value;
        if constexpr (q < NL) load_one(ic<(LP < 0 ? 0 : LP) + PARTS * q>{}, ld_st, ld_ok);
        else read_one(ic<q - NL>{}, ic<(RK < 0 ? 0 : RK)>{}, ic<1 - kk>{}, rd_st);
      });
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  // vmcnt(n) with lgkmcnt(0): n in bits [3:0] and [15:14]
  auto wait_loads = [&](int younger) {
    if (younger == 0) __builtin_amdgcn_s_waitcnt(0x0070);
    else __builtin_amdgcn_s_waitcnt(0x0070 | (LOADS * (NS - 2) & 15) | (((LOADS * (NS - 2)) >> 4) << 14));
  };
  static_assert(LOADS * (NS - 2) < 64, "vmcnt range");
  auto next = [](int st) { return st + 1 == NS ? 0 : st + 1; };

  // Slab s lives in LDS stage s % NS and is two k-steps.  Step 0 prefetches the fragments of step
  // 1; then the wavefront waits for its own loads of slab s+1 and its reads of this stage, and
  // meets the others at the slab's one barrier; step 1 prefetches the first fragments of slab
  // s+1 and starts refilling this stage with slab s+NS (the rest of those loads, if spread over
  // two steps, go out during step 0 of slab s+1).
  //   IA: slab s+NS-1 exists (loads in step 0), IB: slab s+NS exists (loads in step 1), LAST: no slab s+1.
  auto slab = [&](auto ia_c, auto ib_c, auto last_c, int s, int cs, int ls) {
    constexpr bool IA = decltype(ia_c)::value, IB = decltype(ib_c)::value, LAST = decltype(last_c)::value;
    const uint8_t* st = smem8 + cs * SM::stage_bytes;
    const uint32_t ld_a = __builtin_amdgcn_readfirstlane(smem_lds + ls * SM::stage_bytes + wave * 1024);
    step(ic<0>{}, ic<(IA && PARTS > 1) ? 1 : -1>{}, ic<1>{}, ld_a, (s + NS - 1) * F8_BK + kc < K, st);
    if constexpr (!LAST) {
      wait_loads(IA ? 1 : 0);
      __syncthreads();
    }
    const uint32_t ld_b = __builtin_amdgcn_readfirstlane(smem_lds + cs * SM::stage_bytes + wave * 1024);
    step(ic<1>{}, ic<IB ? 0 : -1>{}, ic<LAST ? -1 : 0>{}, ld_b, (s + NS) * F8_BK + kc < K,
         smem8 + next(cs) * SM::stage_bytes);
  };

  const int nslab = (K + F8_BK - 1) / F8_BK;
#pragma unroll
  for (int p = 0; p < NS - 1; ++p)
    if (p < nslab) load_slab(p, p * F8_BK);
  wait_loads(nslab >= NS - 1 ? 1 : 0);
  __syncthreads();
  static_for<READS>([&](auto q_c) { read_one(q_c, ic<0>{}, ic<0>{}, smem8); });
  if (NS - 1 < nslab) {  // the share of slab NS-1 that a slab's step 1 would have issued
    const uint32_t st = __builtin_amdgcn_readfirstlane(smem_lds + (NS - 1) * SM::stage_bytes + wave * 1024);
    const bool k_ok = (NS - 1) * F8_BK + kc < K;
    static_for<(LOADS + PARTS - 1) / PARTS>([&](auto q_c) { load_one(ic<PARTS * decltype(q_c)::value>{}, st, k_ok); });
  }
  int cs = 0, ls = NS - 1, s = 0;
  using T_ = std::true_type;
  using F_ = std::false_type;
  for (; s + NS < nslab; ++s) {  // steady state
    slab(T_{}, T_{}, F_{}, s, cs, ls);
    cs = next(cs);
    ls = next(ls);
  }
  for (; s + 1 < nslab; ++s) {   // drain: the last loads, then none
    if (s + NS - 1 < nslab) slab(T_{}, F_{}, F_{}, s, cs, ls);
    else slab(F_{}, F_{}, F_{}, s, cs, ls);
    cs = next(cs);
    ls = next(ls);
  }
  slab(F_{}, F_{}, T_{}, s, cs, ls);

  // Epilogue, as in gemm.hip: acc[i][j][r] is D[m][n] with m = tile row l32 and
  // n = (r/4)*8 + lg*4 + r%4; each wavefront turns its block around through LDS, 32 rows at a
  // time in fp32, and stores (and reads C and the row scales) in whole runs through buffer
  // descriptors that end with the matrix, so a pass has no branches.
  constexpr int CW = BN / WN, ROWP = CW * 4 + 16, CPR = CW / 4, ITER = 32 * CPR / 64;
  static_assert(NB * 4 * 32 * ROWP <= (int)SM::bytes && (32 * CPR) % 64 == 0 && 64 % CPR == 0, "epilogue staging");
  typedef unsigned int u32v2_t __attribute__((ext_vector_type(2)));
  __syncthreads();  // every wavefront has read its last fragments
  uint8_t* ep = smem8 + wave * (32 * ROWP);
  uint8_t* ep1 = smem8 + (4 + wave) * (32 * ROWP);  // kDual: the second product
  const int gn0 = n_base + wn * CW;
  const int gn = gn0 + (lane % CPR) * 4;  // the same 4 columns in every pass: 64 % CPR == 0
  float4_t cs4 = float4_t{0.f, 0.f, 0.f, 0.f}, cu4 = float4_t{0.f, 0.f, 0.f, 0.f};
  if constexpr (!kPartial) {
    if (gn < N) cs4 = *reinterpret_cast<const float4_t*>(sb + gn);
    if constexpr (kDual) {
      if (gn < N) cu4 = *reinterpret_cast<const float4_t*>(sb1 + gn);
    } else {
      cs4 *= alpha;
    }
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int gm0 = m_base + wm * (BM / WM) + i * 32;
    const int rows = M - gm0 < 32 ? M - gm0 : 32;
    const int recs = rows > 0 ? rows * N * 2 : 0;
    const size_t row0 = (size_t)(rows > 0 ? gm0 : 0);
    if constexpr (kPartial) {
      // the fp32 sums as they are (scales, alpha, beta and C belong to the reduction), one product
      // after the other through the first staging area
      typedef unsigned int u32v4_t __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int b = 0; b < NB; ++b) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int qd = 0; qd < 4; ++qd) {
            float4_t v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = acc[b][i][j][qd * 4 + e];
            *reinterpret_cast<float4_t*>(ep + l32 * ROWP + (j * 32 + qd * 8 + lg * 4) * 4) = v;
          }
        float* dst = (b == 0 ? reinterpret_cast<float*>(D) : reinterpret_cast<float*>(const_cast<uint16_t*>(C))) + p_off;
        const __amdgpu_buffer_rsrc_t p_rsrc =
            __builtin_amdgcn_make_buffer_rsrc(dst + row0 * N, 0, rows > 0 ? rows * N * 4 : 0, 0x00020000);
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
          const int c = it * 64 + lane;
          const float4_t p4 = *reinterpret_cast<const float4_t*>(ep + (c / CPR) * ROWP + (c % CPR) * 16);
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32v4_t, p4), p_rsrc,
                                                 gn < N ? (uint32_t)((c / CPR) * N + gn) * 4u : kOob, 0, 0);
        }
      }
      continue;
    }
    const __amdgpu_buffer_rsrc_t d_rsrc = __builtin_amdgcn_make_buffer_rsrc(D + row0 * N, 0, recs, 0x00020000);
    const __amdgpu_buffer_rsrc_t s_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(sa) + row0, 0, rows > 0 ? rows * 4 : 0, 0x00020000);
    uint32_t off[ITER];
    float rs[ITER];
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int r = (it * 64 + lane) / CPR;
      off[it] = gn < N ? (uint32_t)(r * N + gn) * 2u : kOob;
      rs[it] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(s_rsrc, r * 4, 0, 0));
    }
    u32v2_t cv[ITER];
    if constexpr (!kDual) {
      if (beta != 0.f) {
        const __amdgpu_buffer_rsrc_t c_rsrc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(C) + row0 * N, 0, recs, 0x00020000);
#pragma unroll
        for (int it = 0; it < ITER; ++it) cv[it] = __builtin_amdgcn_raw_buffer_load_b64(c_rsrc, off[it], 0, 0);
      }
    }
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
          float4_t v;
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = acc[b][i][j][qd * 4 + e];
          *reinterpret_cast<float4_t*>((b ? ep1 : ep) + l32 * ROWP + (j * 32 + qd * 8 + lg * 4) * 4) = v;
        }
    float4_t a4[ITER];
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int c = it * 64 + lane;
      a4[it] = *reinterpret_cast<const float4_t*>(ep + (c / CPR) * ROWP + (c % CPR) * 16);
    }
    auto store_group = [&](int it, float4_t v) {
      __builtin_amdgcn_raw_buffer_store_b64(u32v2_t{pack_f16x2(v[0], v[1]), pack_f16x2(v[2], v[3])}, d_rsrc, off[it], 0, 0);
    };
    if constexpr (kDual) {
#pragma unroll
      for (int it = 0; it < ITER; ++it) {
        const int c = it * 64 + lane;
        const float4_t u4 = *reinterpret_cast<const float4_t*>(ep1 + (c / CPR) * ROWP + (c % CPR) * 16);
        const float4_t g = a4[it] * cs4 * rs[it], u = u4 * cu4 * rs[it];
        float4_t v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = swiglu_rounded_f16(g[e], u[e]);
        store_group(it, v);
      }
    } else if (beta == 0.f) {
#pragma unroll
      for (int it = 0; it < ITER; ++it) store_group(it, a4[it] * cs4 * rs[it]);
    } else {
#pragma unroll
      for (int it = 0; it < ITER; ++it) {
        float4_t v = a4[it] * cs4 * rs[it];
        v[0] += beta * h2f_bits(cv[it].x & 0xffffu);
        v[1] += beta * h2f_bits(cv[it].x >> 16);
        v[2] += beta * h2f_bits(cv[it].y & 0xffffu);
        v[3] += beta * h2f_bits(cv[it].y >> 16);
        store_group(it, v);
      }
    }
  }
}

template <int BM, int BN, int WM, int WN, bool kDual = false>
static int launch_gemm_f8(const uint8_t* A, const uint8_t* B, const float* sa, const float* sb,
                          const uint16_t* C, uint16_t* D, int M, int N, int K, float alpha, float beta,
                          hipStream_t stream, const uint8_t* B1 = nullptr, const float* sb1 = nullptr) {
  using SM = F8Smem<BM, BN, kDual ? 2 : 1>;
  auto kern = gemm_f8_kernel<BM, BN, WM, WN, kDual>;
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
  kern<<<grid, 256, SM::bytes, stream>>>(A, B, B1, sa, sb, sb1, C, D, M, N, K, alpha, beta, tiles_m, tiles_n, 1, K);
  return check_launch("gemm_f8 launch");
}

// D[m][n..n+3] = half(alpha * sa[m] * sb[n..] * sum_s P[s][m][n..] + beta * C[m][n..])
__global__ __launch_bounds__(256) void splitk_reduce_f8_kernel(const float* __restrict__ P, int shares,
                                                               const float* __restrict__ sa,
                                                               const float* __restrict__ sb, const uint16_t* C,
                                                               uint16_t* D, int M, int N, float alpha, float beta) {
  const size_t groups = (size_t)M * N / 4, mn = (size_t)M * N;
  for (size_t g = (size_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += (size_t)gridDim.x * 256) {
    float4_t v = sum_shares(P, mn, g * 4, shares);
    const size_t m = g * 4 / N, n = g * 4 % N;
    v = v * (*reinterpret_cast<const float4_t*>(sb + n) * alpha) * sa[m];
    if (beta != 0.f) {
      const u32x2 c = *reinterpret_cast<const u32x2*>(C + g * 4);
      v[0] += beta * h2f_bits(c.x & 0xffffu);
      v[1] += beta * h2f_bits(c.x >> 16);
      v[2] += beta * h2f_bits(c.y & 0xffffu);
      v[3] += beta * h2f_bits(c.y >> 16);
    }
    *reinterpret_cast<u32x2*>(D + g * 4) = u32x2{pack_f16x2(v[0], v[1]), pack_f16x2(v[2], v[3])};
  }
}

// the gate/up pair: both sums scaled, rounded to fp16, then SiLU-mul
__global__ __launch_bounds__(256) void splitk_reduce_dual_f8_kernel(const float* __restrict__ P0,
                                                                    const float* __restrict__ P1, int shares,
                                                                    const float* __restrict__ sa,
                                                                    const float* __restrict__ sg,
                                                                    const float* __restrict__ su, uint16_t* out,
                                                                    int M, int N) {
  const size_t groups = (size_t)M * N / 4, mn = (size_t)M * N;
  for (size_t g = (size_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += (size_t)gridDim.x * 256) {
    float4_t a = sum_shares(P0, mn, g * 4, shares), b = sum_shares(P1, mn, g * 4, shares);
    const size_t m = g * 4 / N, n = g * 4 % N;
    a = a * *reinterpret_cast<const float4_t*>(sg + n) * sa[m];
    b = b * *reinterpret_cast<const float4_t*>(su + n) * sa[m];
    float4_t v;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = swiglu_rounded_f16(a[e], b[e]);
    *reinterpret_cast<u32x2*>(out + g * 4) = u32x2{pack_f16x2(v[0], v[1]), pack_f16x2(v[2], v[3])};
  }
}

// Shares of a split over K (see gemm.hip): at most 256 rows, tiles of 64 x 256 (the pair: 64 x 128)
// up to 64 rows, else 128 x 128, as many shares as fill the CUs, each at least 1024 k deep (8 slabs).
static int splitk_plan_f8(int M, int N, int K, bool dual, int* k_per) {
  if (M > 256 || K < 2048) return 1;
  const int bm = M <= 64 ? 64 : 128, bn = M <= 64 && !dual ? 256 : 128;
  const int tiles = ((M + bm - 1) / bm) * ((N + bn - 1) / bn);
  int cus = 256, dev = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  const int shares = std::min(std::min(cus / tiles, K / 1024), kMaxShares);
  if (shares < 2) return 1;
  *k_per = ((K + shares - 1) / shares + F8_BK - 1) / F8_BK * F8_BK;
  return (K + *k_per - 1) / *k_per;
}

template <int BM, int BN, int WM, int WN, bool kDual>
static int launch_splitk_f8(const uint8_t* A, const uint8_t* B, const uint8_t* B1, const float* sa,
                            const float* sb, const float* sb1, const uint16_t* C, uint16_t* D, int M, int N,
                            int K, float alpha, float beta, int shares, int k_per, float* P, hipStream_t stream) {
  using SM = F8Smem<BM, BN, kDual ? 2 : 1>;
  auto kern = gemm_f8_kernel<BM, BN, WM, WN, kDual, true>;
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
  float* P1 = kDual ? P + (size_t)shares * M * N : nullptr;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const int grid = ((tiles_m * tiles_n * shares + 7) / 8) * 8;
  kern<<<grid, 256, SM::bytes, stream>>>(A, B, B1, nullptr, nullptr, nullptr, reinterpret_cast<const uint16_t*>(P1),
                                         reinterpret_cast<uint16_t*>(P), M, N, K, 1.f, 0.f, tiles_m, tiles_n,
                                         shares, k_per);
  int rc = check_launch("gemm_f8 split-K launch");
  if (rc) return rc;
  const int rgrid = (int)std::min<size_t>(((size_t)M * N / 4 + 255) / 256, 2048);
  if constexpr (kDual) splitk_reduce_dual_f8_kernel<<<rgrid, 256, 0, stream>>>(P, P1, shares, sa, sb, sb1, D, M, N);
  else splitk_reduce_f8_kernel<<<rgrid, 256, 0, stream>>>(P, shares, sa, sb, C, D, M, N, alpha, beta);
  return check_launch("gemm_f8 split-K reduction launch");
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
  hipStream_t s = (hipStream_t)stream;
  if (K <= 4 * 2048) quantize_rows_e4m3_kernel<4><<<M, 256, 0, s>>>(X, Xq, row_scale, K);
  else if (K <= 16 * 2048) quantize_rows_e4m3_kernel<16><<<M, 256, 0, s>>>(X, Xq, row_scale, K);
  else quantize_rows_e4m3_kernel<0><<<M, 256, 0, s>>>(X, Xq, row_scale, K);
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
  // 32-bit buffer offsets run up to a tile past the last row and a few slabs past K
  NF_REQUIRE(((size_t)M + 256) * ((size_t)K + 1024) < 0xFFFFFF00ull && ((size_t)N + 256) * ((size_t)K + 1024) < 0xFFFFFF00ull,
             "nf_gemm_f8_f16: an operand of %d x %d x %d exceeds the 4 GiB buffer-addressing limit", M, N, K);
  if (M == 0) return NF_OK;
  hipStream_t s = (hipStream_t)stream;
  if (M <= 64) return launch_gemm_f8<64, 256, 1, 4>(Aq, Bq, a_scale, b_scale, C, D, M, N, K, alpha, beta, s);
  // Tile choice by cost, as for the fp16 kernels: rounds of one tile per CU, a partly filled last
  // round charged 0.47 + 0.53 x its fill, a round costing the tile's area over its efficiency
  // (1 / 0.80 / 0.60 for 256x256 / 128x256 / 128x128, from full rounds with the weights streamed
  // from HBM).  Picks the fastest tile on the Llama-3-8B and -70B layer shapes at 1024 and 2048
  // rows (2048 x 6144 x 4096: 49 us on 192 tiles of 256x256, 64 us on 384 of 128x256).
  static int cus = 0;  // benign race: every thread computes the same value
  if (cus == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
      v = 256;
    cus = v;
  }
  auto cost = [&](int bm, int bn, double eff) {
    const long long tiles = (long long)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
    const long long full = tiles / cus, rest = tiles % cus;
    return ((double)full + (rest ? 0.47 + 0.53 * (double)rest / cus : 0.0)) * bm * bn / eff;
  };
  const double c256 = cost(256, 256, 1.0), c128x256 = cost(128, 256, 0.80), c128 = cost(128, 128, 0.60);
  const double best = std::min(c256, std::min(c128x256, c128));
  if (best == c256) return launch_gemm_f8<256, 256, 2, 2>(Aq, Bq, a_scale, b_scale, C, D, M, N, K, alpha, beta, s);
  if (best == c128x256) return launch_gemm_f8<128, 256, 2, 2>(Aq, Bq, a_scale, b_scale, C, D, M, N, K, alpha, beta, s);
  return launch_gemm_f8<128, 128, 2, 2>(Aq, Bq, a_scale, b_scale, C, D, M, N, K, alpha, beta, s);
}

int nf_quantize_weight_e4m3(const uint16_t* W, uint8_t* Wq, float* col_scale, int K, int N,
                            nf_stream_t stream) {
  NF_REQUIRE(K > 0 && N > 0 && K % 16 == 0 && N % 8 == 0,
             "nf_quantize_weight_e4m3: bad shape K=%d N=%d (K %% 16, N %% 8)", K, N);
  NF_REQUIRE(W && Wq && col_scale, "nf_quantize_weight_e4m3: null pointer");
  NF_REQUIRE(((uintptr_t)W | (uintptr_t)Wq) % 16 == 0, "nf_quantize_weight_e4m3: operands must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  weight_col_scale_kernel<<<(N + 63) / 64, 256, 0, s>>>(W, col_scale, K, N);
  int rc = check_launch("weight_col_scale launch");
  if (rc) return rc;
  weight_quantize_transpose_kernel<<<dim3((K + 63) / 64, (N + 63) / 64), 256, 0, s>>>(W, col_scale, Wq, K, N);
  return check_launch("weight_quantize_transpose launch");
}

int nf_dual_swiglu_f8_f16(const uint8_t* Aq, const float* a_scale, const uint8_t* Gq, const float* g_scale,
                          const uint8_t* Uq, const float* u_scale, uint16_t* out, int M, int N, int K,
                          nf_stream_t stream) {
  NF_REQUIRE(M >= 0 && N > 0 && K > 0, "nf_dual_swiglu_f8_f16: bad shape M=%d N=%d K=%d", M, N, K);
  NF_REQUIRE(K % 16 == 0 && N % 8 == 0, "nf_dual_swiglu_f8_f16: K=%d must be a multiple of 16 and N=%d of 8", K, N);
  NF_REQUIRE(M == 0 || (Aq && a_scale && Gq && g_scale && Uq && u_scale && out), "nf_dual_swiglu_f8_f16: null pointer");
  NF_REQUIRE(((uintptr_t)Aq | (uintptr_t)Gq | (uintptr_t)Uq | (uintptr_t)g_scale | (uintptr_t)u_scale) % 16 == 0 &&
                 (uintptr_t)out % 8 == 0,
             "nf_dual_swiglu_f8_f16: Aq, Gq, Uq and the weight scales must be 16-byte, out 8-byte aligned");
  NF_REQUIRE(((size_t)M + 256) * ((size_t)K + 1024) < 0xFFFFFF00ull && ((size_t)N + 256) * ((size_t)K + 1024) < 0xFFFFFF00ull,
             "nf_dual_swiglu_f8_f16: an operand of %d x %d x %d exceeds the 4 GiB buffer-addressing limit", M, N, K);
  if (M == 0) return NF_OK;
  hipStream_t s = (hipStream_t)stream;
  if (M <= 64)
    return launch_gemm_f8<64, 128, 2, 2, true>(Aq, Gq, a_scale, g_scale, nullptr, out, M, N, K, 1.f, 0.f, s, Uq, u_scale);
  const long long t256 = (long long)((M + 255) / 256) * ((N + 127) / 128);
  const int tail = M % 256;  // rows in the last 256-row tile: half-empty tiles go to the 128-row kernel
  if (t256 >= 192 && (tail == 0 || tail > 128))
    return launch_gemm_f8<256, 128, 2, 2, true>(Aq, Gq, a_scale, g_scale, nullptr, out, M, N, K, 1.f, 0.f, s, Uq, u_scale);
  return launch_gemm_f8<128, 128, 2, 2, true>(Aq, Gq, a_scale, g_scale, nullptr, out, M, N, K, 1.f, 0.f, s, Uq, u_scale);
}

size_t nf_gemm_f8w_workspace_bytes(int M, int K) {
  if (M <= 0 || K <= 0) return 0;
  return ((size_t)M * K + 255) / 256 * 256 + (size_t)M * sizeof(float);
}

// The GEMM on rows that are quantised already: split over K when the launch has few rows against a
// narrow N and the workspace holds the partial sums behind the place of the quantised rows.
static int gemm_f8q(const uint8_t* Aq, const float* sa, const uint8_t* Bq, const float* b_scale, const uint16_t* C,
                    uint16_t* D, int M, int N, int K, float alpha, float beta, void* workspace, size_t workspace_bytes,
                    nf_stream_t stream) {
  int k_per = 0;
  const int shares = N > 0 && N % 8 == 0 && K % 16 == 0 ? splitk_plan_f8(M, N, K, false, &k_per) : 1;
  const size_t p_at = (nf_gemm_f8w_workspace_bytes(M, K) + 255) / 256 * 256;
  if (shares >= 2 && workspace && (uintptr_t)workspace % 16 == 0 &&
      workspace_bytes >= p_at + (size_t)shares * M * N * sizeof(float) && Bq && b_scale && D &&
      ((size_t)N + 256) * ((size_t)K + 1024) < 0xFFFFFF00ull &&
      (beta == 0.f || C) && ((uintptr_t)Bq | (uintptr_t)b_scale) % 16 == 0 && ((uintptr_t)D | (uintptr_t)C) % 8 == 0) {
    float* P = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + p_at);
    hipStream_t s = (hipStream_t)stream;
    if (M <= 64)
      return launch_splitk_f8<64, 256, 1, 4, false>(Aq, Bq, nullptr, sa, b_scale, nullptr, C, D, M, N, K, alpha, beta, shares, k_per, P, s);
    return launch_splitk_f8<128, 128, 2, 2, false>(Aq, Bq, nullptr, sa, b_scale, nullptr, C, D, M, N, K, alpha, beta, shares, k_per, P, s);
  }
  return nf_gemm_f8_f16(Aq, sa, Bq, b_scale, C, D, M, N, K, alpha, beta, stream);
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
  return gemm_f8q(Aq, sa, Bq, b_scale, C, D, M, N, K, alpha, beta, workspace, workspace_bytes, stream);
}

int nf_gemm_f8q_f16(const uint8_t* Aq, const float* a_scale, const uint8_t* Bq, const float* b_scale,
                    const uint16_t* C, uint16_t* D, int M, int N, int K, float alpha, float beta, void* workspace,
                    size_t workspace_bytes, nf_stream_t stream) {
  NF_REQUIRE(M >= 0 && K > 0, "nf_gemm_f8q_f16: bad shape M=%d K=%d", M, K);
  if (M == 0) return NF_OK;
  return gemm_f8q(Aq, a_scale, Bq, b_scale, C, D, M, N, K, alpha, beta, workspace, workspace_bytes, stream);
}

size_t nf_gemm_f8w_split_workspace_bytes(int M, int N, int K) {
  const size_t need = nf_gemm_f8w_workspace_bytes(M, K);
  if (M <= 0 || N <= 0 || K <= 0) return need;
  int k_per = 0;
  const int shares = splitk_plan_f8(M, N, K, false, &k_per);
  return shares < 2 ? need : (need + 255) / 256 * 256 + (size_t)shares * M * N * sizeof(float);
}

size_t nf_gemm_f8w_split_workspace_bytes_upto(int max_M, int N, int K) {
  size_t need = nf_gemm_f8w_workspace_bytes(max_M, K);
  for (int m = 1; m <= max_M && m <= 256; ++m) need = std::max(need, nf_gemm_f8w_split_workspace_bytes(m, N, K));
  return need;
}

size_t nf_dual_swiglu_f8w_split_workspace_bytes(int M, int N, int K) {
  const size_t need = nf_gemm_f8w_workspace_bytes(M, K);
  if (M <= 0 || N <= 0 || K <= 0) return need;
  int k_per = 0;
  const int shares = splitk_plan_f8(M, N, K, true, &k_per);
  return shares < 2 ? need : (need + 255) / 256 * 256 + (size_t)2 * shares * M * N * sizeof(float);
}

size_t nf_dual_swiglu_f8w_split_workspace_bytes_upto(int max_M, int N, int K) {
  size_t need = nf_gemm_f8w_workspace_bytes(max_M, K);
  for (int m = 1; m <= max_M && m <= 256; ++m) need = std::max(need, nf_dual_swiglu_f8w_split_workspace_bytes(m, N, K));
  return need;
}

static int dual_swiglu_f8q(const uint8_t* Aq, const float* sa, const uint8_t* Gq, const float* g_scale,
                           const uint8_t* Uq, const float* u_scale, uint16_t* out, int M, int N, int K, void* workspace,
                           size_t workspace_bytes, nf_stream_t stream) {
  int k_per = 0;
  const int shares = N > 0 && N % 8 == 0 && K % 16 == 0 ? splitk_plan_f8(M, N, K, true, &k_per) : 1;
  const size_t p_at = (nf_gemm_f8w_workspace_bytes(M, K) + 255) / 256 * 256;
  if (shares >= 2 && workspace && (uintptr_t)workspace % 16 == 0 &&
      workspace_bytes >= p_at + (size_t)2 * shares * M * N * sizeof(float) && Gq && g_scale && Uq &&
      ((size_t)N + 256) * ((size_t)K + 1024) < 0xFFFFFF00ull &&
      u_scale && out &&
      ((uintptr_t)Gq | (uintptr_t)Uq | (uintptr_t)g_scale | (uintptr_t)u_scale) % 16 == 0 && (uintptr_t)out % 8 == 0) {
    float* P = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + p_at);
    hipStream_t s = (hipStream_t)stream;
    if (M <= 64)
      return launch_splitk_f8<64, 128, 2, 2, true>(Aq, Gq, Uq, sa, g_scale, u_scale, nullptr, out, M, N, K, 1.f, 0.f, shares, k_per, P, s);
    return launch_splitk_f8<128, 128, 2, 2, true>(Aq, Gq, Uq, sa, g_scale, u_scale, nullptr, out, M, N, K, 1.f, 0.f, shares, k_per, P, s);
  }
  return nf_dual_swiglu_f8_f16(Aq, sa, Gq, g_scale, Uq, u_scale, out, M, N, K, stream);
}

int nf_dual_swiglu_f8w_f16(const uint16_t* A, const uint8_t* Gq, const float* g_scale, const uint8_t* Uq,
                           const float* u_scale, uint16_t* out, int M, int N, int K, void* workspace,
                           size_t workspace_bytes, nf_stream_t stream) {
  NF_REQUIRE(M >= 0 && K > 0, "nf_dual_swiglu_f8w_f16: bad shape M=%d K=%d", M, K);
  if (M == 0) return NF_OK;
  const size_t need = nf_gemm_f8w_workspace_bytes(M, K);
  if (!workspace || workspace_bytes < need) {
    set_error("nf_dual_swiglu_f8w_f16: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    return NF_ERR_WORKSPACE;
  }
  NF_REQUIRE((uintptr_t)workspace % 16 == 0, "nf_dual_swiglu_f8w_f16: workspace must be 16-byte aligned");
  uint8_t* Aq = static_cast<uint8_t*>(workspace);
  float* sa = reinterpret_cast<float*>(Aq + ((size_t)M * K + 255) / 256 * 256);
  int rc = nf_quantize_rows_e4m3(A, Aq, sa, M, K, stream);
  if (rc) return rc;
  return dual_swiglu_f8q(Aq, sa, Gq, g_scale, Uq, u_scale, out, M, N, K, workspace, workspace_bytes, stream);
}

int nf_dual_swiglu_f8q_f16(const uint8_t* Aq, const float* a_scale, const uint8_t* Gq, const float* g_scale,
                           const uint8_t* Uq, const float* u_scale, uint16_t* out, int M, int N, int K, void* workspace,
                           size_t workspace_bytes, nf_stream_t stream) {
  NF_REQUIRE(M >= 0 && K > 0, "nf_dual_swiglu_f8q_f16: bad shape M=%d K=%d", M, K);
  if (M == 0) return NF_OK;
  return dual_swiglu_f8q(Aq, a_scale, Gq, g_scale, Uq, u_scale, out, M, N, K, workspace, workspace_bytes, stream);
}

}  // extern "C"
