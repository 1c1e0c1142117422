// 16-bit x 16-bit -> fp32 -> 16-bit GEMM family for gfx950 on v_mfma_f32_16x16x32_f16 (fp16, the
// pipeline's type; 32x32x16 for the tiles on eight wavefronts) and the bf16 forms of the same
// instructions (bf16: same kernels, other element type).
//
//   D = half(alpha * A.B + beta * C)                     (plain; QKV, O, down, LM head)
//   D = half(silu(half(A.Bg)) * half(A.Bu))              (dual; gate/up SwiGLU)
//
// Workgroup = 256 threads = 4 wavefronts in a WM x WN grid; each wavefront owns a
// (BM/WM) x (BN/WN) block of 16x16 (or 32x32) MFMA tiles.  K is walked in slabs of 64 through a
// ring of two to four LDS stages (as many as fit 144 KB).
//
// Operands go from global memory STRAIGHT INTO LDS (buffer_load_dwordx4 ... lds): a CU moves
// about 38 GB/s through the load-to-register path but well over 100 GB/s through this one, and
// a 256x256 tile needs ~60 GB/s per CU to keep the matrix pipe busy.  One such instruction
// writes 64 lanes x 16 bytes to 1 KB of consecutive LDS, so the LDS image cannot be padded;
// bank conflicts are avoided by choosing WHICH 16-byte chunk each lane fetches (an XOR swizzle
// applied on the global side):
// (LDS has 64 banks of 4 bytes: a 16-byte read is served 16 lanes per cycle, an 8-byte read 32
// lanes per cycle, each cycle covering 256 bytes of distinct banks when conflict-free.)
//   A slab (and [N][K] weights)  rows of 128 bytes (64 k), 8 rows per instruction; row r keeps
//       logical chunk c at position c ^ ((r >> 1) & 7).  An MFMA fragment is one 16-byte read;
//       the 16 rows of a read cycle (two per 256 bytes) land on 16 different 16-byte slots.
//   [K][N] weights               kept row-major, 64 rows of BN*2 bytes; row r keeps chunk c at
//       position c ^ ((r & 3) << 2) ^ (((r >> 3) & 1) << 1).  The k-contiguous MFMA operand is
//       produced by the transposing LDS read (ds_read_b64_tr_b16: 16 lanes read a 4(k) x 16(n)
//       block row-wise and receive it column-wise), two per operand; the 2 x 4 rows x 32 bytes a
//       read cycle touches (two k-groups of 8 rows, 8 rows apart) sit in 8 different 32-byte
//       bank groups.
// With these two permutations SQ_LDS_BANK_CONFLICT reads zero for the kernel.
// No staging registers, no permutes, no LDS stores in the main loop.  A wavefront is alone on
// its SIMD, so nothing hides a stall of its instruction stream: the loads of later slabs and
// the fragment reads of the next k-step are dealt out one at a time between the MFMAs of the
// current k-step, in a pinned order; one barrier per slab.
//
// The MFMA is issued as D^T = B^T.A^T (weights as the first operand): a lane ends up with 4
// consecutive output columns of a row (of 32 rows with the 32x32 instruction).  The epilogue turns each wavefront's block around
// through LDS so that D is stored, and C read, in whole 512-byte runs.
#include <algorithm>
#include <cmath>
#include <type_traits>
#include <utility>

#include "common.h"

namespace nf {

constexpr int BK = 64;  // K slab (halves); an A-style LDS row is 128 bytes

template <int BM, int BN, int NB>
struct GemmSmem {
  static constexpr int a_bytes = BM * 128;
  static constexpr int b_bytes = BN * 128;  // 64 rows x BN*2 bytes, or BN rows x 128 bytes
  static constexpr int stage_bytes = a_bytes + NB * b_bytes;
  // as many stages as fit 144 KB (of the CU's 160 KB), at most 4: the loads of a slab are issued
  // stages-1 slabs before they are needed
  static constexpr int stages = (144 * 1024) / stage_bytes > 4 ? 4 : (144 * 1024) / stage_bytes;
  static_assert(stages >= 2, "tile too large for two LDS stages");
  // Tiles with room for two stages only (256 x 256, the 256 x 128 pair: 64 KB per slab) would have to
  // land every load of a slab within the slab before it -- less than a microsecond, which a load
  // that misses the L2 does not make.  They keep the activations in a ring of two stages and give
  // the weights (the operand that streams from HBM) a ring of three: 2 x 32 + 3 x 32 KB = all 160 KB.
  static constexpr bool split = stages == 2 && 2 * a_bytes + 3 * NB * b_bytes <= 160 * 1024;
  static constexpr int b_ring = 2 * a_bytes;  // split rings: activation stages first, then the weight stages
  static constexpr size_t bytes = split ? (size_t)2 * a_bytes + (size_t)3 * NB * b_bytes : (size_t)stages * stage_bytes;
};

// Element types of the family: how 16-bit storage is multiplied, widened and rounded.
struct F16 {
  static __device__ __forceinline__ float16_t mfma(half8_t b, half8_t a, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(b, a, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float4_t mfma16(half8_t b, half8_t a, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(b, a, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float widen(uint32_t bits) { return h2f_bits(bits); }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_f16x2(lo, hi); }
  static __device__ __forceinline__ float rounded(float x) { return __half2float(__float2half_rn(x)); }
};
struct BF16 {
  typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ float16_t mfma(half8_t b, half8_t a, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, b), __builtin_bit_cast(bf16x8_t, a), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float4_t mfma16(half8_t b, half8_t a, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, b), __builtin_bit_cast(bf16x8_t, a), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float widen(uint32_t bits) { return __builtin_bit_cast(float, bits << 16); }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {  // round to nearest even
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
  }
  static __device__ __forceinline__ float rounded(float x) { return widen(pack2(x, 0.f) & 0xffffu); }
};

// SiLU(g)*u on values already rounded to the storage type, as the reference's dual epilogue
// computes it (in fp16 there).
template <class E>
__device__ __forceinline__ float swiglu_rounded(float g_acc, float u_acc) {
  float g = E::rounded(g_acc);
  float u = E::rounded(u_acc);
  // hardware reciprocal (1 ulp of fp32): the result is rounded to fp16 afterwards
  return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * u;
}

// WM x WN wavefronts: four (one per SIMD, up to 512 registers each) or eight (two per SIMD, up to
// 256 each: for tiles whose accumulators do not fit four wavefronts, the 320 x 128 gate/up pair).
// kDual: two weight matrices, SwiGLU epilogue.  kBCol: weights stored [N][K].
// One BM x BN output tile at (m_base, n_base), computed by the whole workgroup.
// K is the extent of the contraction and lda the row stride (elements) of the k-contiguous
// operands (A, and [N][K] weights): equal for a whole GEMM, K < lda for one share of a GEMM split
// over K, whose operand pointers already point at the share's first k.
// kPartial: the fp32 sums are stored as they are to D taken as float [M][N] (no alpha, beta, C).
template <class E, int BM, int BN, int WM, int WN, bool kDual, bool kBCol, bool kPartial = false>
__device__ __forceinline__ void gemm_tile(
    const uint16_t* __restrict__ A, const uint16_t* __restrict__ B0,
    const uint16_t* __restrict__ B1, const uint16_t* C, uint16_t* D,
    int M, int N, int K, float alpha, float beta, const int ldc, const int m_base, const int n_base,
    const int lda) {
  constexpr int NB = kDual ? 2 : 1;
  using SM = GemmSmem<BM, BN, NB>;
  // four wavefronts (one per SIMD) or eight (two per SIMD, at most 256 registers each)
  constexpr int NW = WM * WN;
  // The MFMA the tile is computed with.  kM16: v_mfma_f32_16x16x32 -- at this part's power cap the
  // register-only loop delivers 19 % more flops on it than on 32x32x16 (half the accumulator
  // traffic per flop), for the same LDS bytes per flop; its fragments are 32 deep, so a 64-deep
  // slab is two k-steps, each issued as two sub-steps: one half of the wavefront's tile columns
  // each, column by column.  The activation fragments of a k-step stay in registers for the step
  // (double-buffered by k-step); the weight fragments are double-buffered by sub-step -- a
  // sub-step reads the columns of the next one -- so that everything but the accumulators fits
  // the 256 architectural registers and the compiler has no reason to shuffle accumulators
  // between the two register files.
  // Eight-wavefront tiles keep 32x32x16 (256 registers per wavefront in all).
  constexpr bool kM16 = NW == 4;
  constexpr int MT = kM16 ? 16 : 32;  // rows and columns of an MFMA tile
  constexpr int TM = BM / WM / MT;    // MFMA tiles per wave along M
  constexpr int TN = BN / WN / MT;
  constexpr int CH = NB * TN / 2;  // kM16: columns of MFMA tiles per sub-step, over both weight matrices
  static_assert(!kM16 || (NB * TN) % 2 == 0, "a sub-step takes half of the tile columns");
  static_assert(NW == 4 || NW == 8, "four or eight wavefronts");
  static_assert((BN / WN) % 32 == 0 && (BM / WM) % 32 == 0 && BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "tile shape");
  constexpr int A_LOADS = BM / (8 * NW);   // 1 KB load instructions per wave per slab
  constexpr int B_LOADS = BN / (8 * NW);   // ... per weight matrix
  constexpr int ROWB = BN * 2;       // bytes per k row of a [K][N] weight slab
  constexpr int B_CPR = BN / 8;      // 16-byte chunks per such row

  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const uint32_t smem_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int l32 = lane & 31, lg = lane >> 5;
  const int l16 = lane & 15, lq = lane >> 4;

  // kM16: G adjacent column tiles share one accumulator vector (see AccVec)
  constexpr int G = !kM16 ? 1 : TN % 4 == 0 ? 4 : TN % 2 == 0 ? 2 : 1;
  constexpr int TNG = TN / G;
  using acc_t = std::conditional_t<kM16, typename AccVec<G>::type, float16_t>;
  acc_t acc[NB][TM][TNG];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TNG; ++j)
#pragma unroll
        for (int r = 0; r < (kM16 ? 4 * G : 16); ++r) acc[b][i][j][r] = 0.f;

  // ---- global -> LDS: per-lane byte offsets of the chunks this lane fetches
  const rsrc_t a_rsrc = make_rsrc(A, ((size_t)(M - 1) * lda + K) * 2);
  rsrc_t b_rsrc[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b)
    b_rsrc[b] = make_rsrc(b ? B1 : B0, kBCol ? ((size_t)(N - 1) * lda + K) * 2 : (size_t)N * K * 2);
  // A-style rows: lane -> (row lane/8 of the instruction's 8 rows, position lane%8), fetching
  // logical chunk position ^ ((row >> 1) & 7); bit 3 of the row number is the wave's parity.
  const int a_kc = ((lane & 7) ^ (((lane >> 4) & 3) | ((wave & 1) << 2))) * 8;
  // One running offset per load instruction, advanced by a slab after each use.  Rows past the
  // operand's last one lie at or past the end of the buffer and read as zero; so do k >= K rows of
  // [K][N] weights.  Weight columns n >= N of such a slab alias the next row: they only reach
  // output columns that are never stored.  Left to test: k >= K inside a 128-byte activation (or
  // [N][K] weight) row, which would read the next row's start.
  uint32_t a_off[A_LOADS];
#pragma unroll
  for (int t = 0; t < A_LOADS; ++t) {
    const int gm = m_base + (t * NW + wave) * 8 + (lane >> 3);
    a_off[t] = ((uint32_t)gm * (uint32_t)lda + a_kc) * 2u;
  }
  uint32_t b_off[NB][B_LOADS];
  const uint32_t b_slab = (uint32_t)BK * (uint32_t)N * 2u;
#pragma unroll
  for (int t = 0; t < B_LOADS; ++t) {
    uint32_t off;
    if constexpr (kBCol) {
      const int gn = n_base + (t * NW + wave) * 8 + (lane >> 3);
      off = ((uint32_t)gn * (uint32_t)lda + a_kc) * 2u;
    } else {
      const int g = (t * NW + wave) * 64 + lane;  // 16-byte slot of the slab's LDS image
      const int row = g / B_CPR;
      const int c = (g % B_CPR) ^ ((row & 3) << 2) ^ (((row >> 3) & 1) << 1);
      off = ((uint32_t)row * (uint32_t)N + n_base + c * 8) * 2u;
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) b_off[b][t] = off;
  }

  // ---- global -> LDS, one 1 KB load instruction at a time.  Load t of a slab: t < A_LOADS
  // fetches activation rows, the rest weight rows.  st = LDS address of the stage + wave * 1024.
  constexpr int NS = SM::stages;
  constexpr int LOADS = A_LOADS + NB * B_LOADS;  // per wave per slab
  constexpr int PARTS = NS == 2 ? 3 : 4;         // k-steps the loads of one slab are spread over
  // k_ok: this lane's 16 bytes of the slab's 128-byte rows lie below K.  la / lb: LDS address of
  // the stage the activations / the weights of the slab go to, + wave * 1024.
  auto load_one = [&](auto t_c, uint32_t la, uint32_t lb, bool k_ok) {
    constexpr int t = decltype(t_c)::value;
    if constexpr (t < A_LOADS) {
      load16_to_lds<t * NW * 1024>(a_rsrc, k_ok ? a_off[t] : kOob, la);
      a_off[t] += BK * 2;
    } else {
      constexpr int b = (t - A_LOADS) / B_LOADS, tt = (t - A_LOADS) % B_LOADS;
      constexpr int dst = b * SM::b_bytes + tt * NW * 1024;
      if constexpr (kBCol) {
        load16_to_lds<dst>(b_rsrc[b], k_ok ? b_off[b][tt] : kOob, lb);
        b_off[b][tt] += BK * 2;
      } else {
        load16_to_lds<dst>(b_rsrc[b], b_off[b][tt], lb);
        b_off[b][tt] += b_slab;
      }
    }
  };
  // The same load in two pieces, for steps whose MFMAs leave room for two or three other
  // instructions each: the offset (masked, and advanced for the next slab) first, the M0 write and
  // the load instruction one MFMA later.
  uint32_t pend = 0;
  auto load_prepare = [&](auto t_c, bool k_ok) {
    constexpr int t = decltype(t_c)::value;
    if constexpr (t < A_LOADS) {
      pend = k_ok ? a_off[t] : kOob;
      a_off[t] += BK * 2;
    } else {
      constexpr int b = (t - A_LOADS) / B_LOADS, tt = (t - A_LOADS) % B_LOADS;
      if constexpr (kBCol) {
        pend = k_ok ? b_off[b][tt] : kOob;
        b_off[b][tt] += BK * 2;
      } else {
        pend = b_off[b][tt];
        b_off[b][tt] += b_slab;
      }
    }
  };
  auto load_issue = [&](auto t_c, uint32_t la, uint32_t lb) {
    constexpr int t = decltype(t_c)::value;
    if constexpr (t < A_LOADS) {
      load16_to_lds<t * NW * 1024>(a_rsrc, pend, la);
    } else {
      constexpr int b = (t - A_LOADS) / B_LOADS, tt = (t - A_LOADS) % B_LOADS;
      load16_to_lds<b * SM::b_bytes + tt * NW * 1024>(b_rsrc[b], pend, lb);
    }
  };
  auto load_slab = [&](int stage, int k0) {  // every load of one slab, back to back (one ring for both operands)
    const uint32_t st = __builtin_amdgcn_readfirstlane(smem_lds + stage * SM::stage_bytes + wave * 1024);
    const bool k_ok = k0 + a_kc < K;
    static_for<LOADS>([&](auto t_c) { load_one(t_c, st, st + SM::a_bytes, k_ok); });
  };

  // ---- LDS -> MFMA operand fragments, double-buffered across k-steps
  // A-style: row r = l32 (+ multiples of 32), logical chunk kk*2+lg sits at chunk ^ ((r>>1)&7).
  // kM16: row r = l16 (+ multiples of 16), logical chunk kk*4 + lq of k-step kk (32 deep), same
  // permutation: the 16 rows of a read cycle land on 16 different 16-byte slots as well.
  const int lrow = kM16 ? l16 : l32;
  const uint32_t a_rd = (uint32_t)(wm * (BM / WM) + lrow) * 128u;
  const uint32_t bc_rd = (uint32_t)(wn * (BN / WN) + lrow) * 128u;  // [N][K] weights
  uint32_t swz[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk)
    swz[kk] = kM16 ? (uint32_t)((((kk & 1) * 4 + lq) ^ ((l16 >> 1) & 7)) << 4) : (uint32_t)(((kk * 2 + lg) ^ ((l32 >> 1) & 7)) << 4);
  // [K][N] weights: 16-lane group g reads the 4(k) x 16(n) block at rows lg*8 + 4h.., columns
  // (g&1)*16.. of the MFMA tile, lane i of the group addressing row i/4, columns (i&3)*4..+3.
  // 32-byte unit u of a row sits at u ^ ((row & 3) << 1) ^ ((row >> 3) & 1), row & 3 = (i/4) & 3 and
  // (row >> 3) & 1 = the parity of the lane group's k rows.
  // kM16: the 16-lane group lq holds k rows lq*8.. of the 32-deep k-step, all four groups the
  // same 16 columns (one 32-byte unit per MFMA tile).
  const int i16 = lane & 15, bx = (i16 >> 2) & 3, g1 = (lane >> 4) & 1;
  const uint32_t br_row = (uint32_t)((kM16 ? lq : lg) * 8 + (i16 >> 2)) * ROWB + (uint32_t)(i16 & 3) * 8u;
  uint32_t br_tbl[TN];  // byte offset inside the row of this lane's 8 bytes, per MFMA tile j
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int unit = kM16 ? (wn * (BN / WN)) / 16 + j : (wn * (BN / WN)) / 16 + 2 * j + g1;  // logical 32-byte unit
    br_tbl[j] = (uint32_t)((unit ^ (bx << 1) ^ (kM16 ? (lq & 1) : lg)) * 32);
  }

  half8_t af[2][TM];
  half8_t bf[2][NB][TN];
  half8_t bh[2][CH > 0 ? CH : 1];  // kM16: the weight fragments of a sub-step's columns
  constexpr int READS = TM + NB * TN;  // fragment reads per k-step: q < TM activations, then weights
  constexpr int KSTEP = kM16 ? 32 : 16;
  // sa / sb: the stage holding the slab's activations / weights
  auto read_one = [&](auto q_c, auto kk_c, auto buf_c, const uint8_t* sa, const uint8_t* sb) {
    constexpr int q = decltype(q_c)::value, kk = decltype(kk_c)::value, buf = decltype(buf_c)::value;
    if constexpr (q < TM) {
      af[buf][q] = *reinterpret_cast<const half8_t*>(sa + a_rd + swz[kk] + q * MT * 128);
    } else {
      constexpr int b = (q - TM) / TN, j = (q - TM) % TN;
      const uint8_t* bs = sb + b * SM::b_bytes;
      // kM16: `buf` is the sub-step's slot, the fragment goes to its place among the sub-step's columns
      half8_t& dst = kM16 ? bh[buf][(q - TM) % (CH > 0 ? CH : 1)] : bf[buf][b][j];
      if constexpr (kBCol) {
        dst = *reinterpret_cast<const half8_t*>(bs + bc_rd + swz[kk] + j * MT * 128);
      } else {
        const uint8_t* p = bs + br_row + br_tbl[j] + kk * KSTEP * ROWB;
        const short4_t lo = lds_read_tr16(p);
        const short4_t hi = lds_read_tr16(p + 4 * ROWB);
        typedef short short8_t __attribute__((ext_vector_type(8)));
        const short8_t v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        dst = __builtin_bit_cast(half8_t, v);
      }
    }
  };

  // One k-step: the MFMAs on fragment buffer kk & 1, with the step's side work dealt out
  // between them and the order pinned -- a wavefront is alone on its SIMD, so whatever it issues
  // between two MFMAs must fit into the 32 cycles the first one occupies the matrix pipe:
  //   loads L0, L0 + LSTR, ... (NL of them) of a slab being fetched, into the stages at la / lb;
  //   then the fragment reads of k-step RK from the stages sa / sb into the other buffer (RK < 0: none).
  constexpr int NM = NB * TN * TM;
  auto step = [&](auto kk_c, auto l0_c, auto lstr_c, auto nl_c, auto rk_c, uint32_t la, uint32_t lb, bool ld_ok,
                  const uint8_t* sa, const uint8_t* sb) {
    constexpr int kk = decltype(kk_c)::value, L0 = decltype(l0_c)::value, LSTR = decltype(lstr_c)::value;
    constexpr int NL = decltype(nl_c)::value, RK = decltype(rk_c)::value;
    if constexpr (kM16) {
      // Sub-step kk of the slab: the MFMAs of k-step kk / 2 (32 deep) on half kk % 2 of the tile
      // columns, column by column.  Fragment reads dealt out between them: the weight fragments of
      // the next sub-step's columns (from the stage at sb: the next slab's for sub-step 3, which
      // runs past the slab's barrier), and activation fragments -- sub-steps 0 and 1 one half each
      // of k-step 1's, sub-step 2 none, sub-step 3 all of the next slab's k-step 0.  The callers
      // name the 16-deep k-step the step would prefetch: RK = kk + 1, 0 past the barrier, -1 for none.
      constexpr int K2 = kk >> 1, H = kk & 1, NMH = CH * TM;
      constexpr int NXT = (kk + 1) & 3, K2N = NXT >> 1, HN = NXT & 1;  // the sub-step the weight reads are for
      constexpr int NRB = RK < 0 ? 0 : CH;
      constexpr int A0 = RK == 2 ? TM / 2 : 0, A1 = RK == 1 ? TM / 2 : (RK == 0 || RK == 2) ? TM : 0;
      constexpr int NRA = A1 - A0, AK = RK == 0 ? 0 : 1;  // the k-step (and buffer) those activation fragments are of
      constexpr int S16 = 2 * NL + NRB + NRA;  // a load counts twice: prepared, then issued
      static_for<NMH>([&](auto n_c) {
        constexpr int n = decltype(n_c)::value;
        constexpr int c = n / TM, i = n % TM, col = H * CH + c, b = col / TN, j = col % TN;
        acc_put<j % G, 4 * G>(acc[b][i][j / G], E::mfma16(bh[H][c], af[K2][i], acc_get<j % G>(acc[b][i][j / G])));
        constexpr int lo = n * S16 / NMH, hi = (n + 1) * S16 / NMH;
        static_for<hi - lo>([&](auto d_c) {
          constexpr int q = lo + decltype(d_c)::value;
          // reads first (activation fragments, then weight fragments), then the load pieces: the
          // fragments are what the next sub-step waits for
          constexpr int NRD = NRB + NRA;
          constexpr int qq = q < NRA ? 2 * NL + NRB + q : q < NRD ? 2 * NL + (q - NRA) : q - NRD;
          if constexpr (qq < 2 * NL) {
            if constexpr (qq % 2 == 0) load_prepare(ic<L0 + LSTR * (qq / 2)>{}, ld_ok);
            else load_issue(ic<L0 + LSTR * (qq / 2)>{}, la, lb);
          } else if constexpr (qq < 2 * NL + NRB) {
            read_one(ic<TM + HN * CH + (qq - 2 * NL)>{}, ic<K2N>{}, ic<HN>{}, sa, sb);
          } else {
            read_one(ic<A0 + (qq - 2 * NL - NRB)>{}, ic<AK>{}, ic<AK>{}, sa, sb);
          }
        });
        __builtin_amdgcn_sched_barrier(0);
      });
    } else {
    constexpr int NR = RK < 0 ? 0 : READS;
    constexpr int S = NL + NR;
    static_for<NM>([&](auto n_c) {
      constexpr int n = decltype(n_c)::value;
      constexpr int b = n / (TN * TM), j = (n / TM) % TN, i = n % TM;
      if constexpr (!kM16) acc[b][i][j] = E::mfma(bf[kk & 1][b][j], af[kk & 1][i], acc[b][i][j]);
      // Side work is dealt out evenly, the loads ahead of the fragment reads.  Measured the other
      // way round (reads first, in the order the next step consumes them): 3-5 % slower on the
      // 256-row tiles -- the loads then queue behind each other at the end of the step.
      constexpr int lo = n * S / NM, hi = (n + 1) * S / NM;
      static_for<hi - lo>([&](auto d_c) {
        constexpr int q = lo + decltype(d_c)::value;
        if constexpr (q < NL) load_one(ic<L0 + LSTR * q>{}, la, lb, ld_ok);
        else read_one(ic<q - NL>{}, ic<(RK < 0 ? 0 : RK)>{}, ic<(kk + 1) & 1>{}, sa, sb);
      });
      __builtin_amdgcn_sched_barrier(0);
    });
    }
  };
  using T_ = std::true_type;
  using F_ = std::false_type;
  const int nslab = (K + BK - 1) / BK;

  if constexpr (SM::split) {
    // ---- two activation stages, three weight stages.  Slab s has its activations in stage s % 2
    // and its weights in stage s % 3.  During slab s a wavefront issues, in this order: the second
    // half of the activation loads of slab s+1 (k-step 0; the first half went out in k-step 3 of
    // slab s-1), all weight loads of slab s+2 (k-steps 1 and 2), then waits until everything but
    // those weight loads has landed -- its loads of slab s+1 -- and meets the others at the barrier;
    // k-step 3 prefetches the first fragments of slab s+1 and issues the first half of the
    // activation loads of slab s+2 into the stage the barrier has just freed.  A weight load has
    // five to six k-steps to land, an activation load three.
    constexpr int HA = (A_LOADS + 1) / 2;               // activation loads issued in k-step 3
    constexpr int BL = NB * B_LOADS, HB = (BL + 1) / 2;  // weight loads, and those issued in k-step 1
    static_assert(BL < 64, "vmcnt range");
    constexpr int wait_but_b = 0x0070 | (BL & 15) | ((BL >> 4) << 14);  // vmcnt(BL), lgkmcnt(0)
    auto a_lds = [&](int stage) { return __builtin_amdgcn_readfirstlane(smem_lds + stage * SM::a_bytes + wave * 1024); };
    auto b_lds = [&](int stage) {
      return __builtin_amdgcn_readfirstlane(smem_lds + SM::b_ring + stage * NB * SM::b_bytes + wave * 1024);
    };
    auto a_ptr = [&](int stage) { return smem + stage * SM::a_bytes; };
    auto b_ptr = [&](int stage) { return smem + SM::b_ring + stage * NB * SM::b_bytes; };
    auto k_ok_of = [&](int slab_idx) { return slab_idx * BK + a_kc < K; };
    // prologue: activations and weights of slab 0, weights of slab 1
    {
      const uint32_t la = a_lds(0), lb0 = b_lds(0), lb1 = b_lds(1);
      static_for<A_LOADS>([&](auto t_c) { load_one(t_c, la, lb0, k_ok_of(0)); });
      static_for<BL>([&](auto t_c) { load_one(ic<A_LOADS + decltype(t_c)::value>{}, la, lb0, k_ok_of(0)); });
      if (nslab > 1) {
        static_for<BL>([&](auto t_c) { load_one(ic<A_LOADS + decltype(t_c)::value>{}, la, lb1, k_ok_of(1)); });
        __builtin_amdgcn_s_waitcnt(wait_but_b);
      } else {
        __builtin_amdgcn_s_waitcnt(0x0070);
      }
    }
    __syncthreads();
    static_for<(kM16 ? TM + CH : READS)>([&](auto q_c) { read_one(q_c, ic<0>{}, ic<0>{}, a_ptr(0), b_ptr(0)); });
    if (nslab > 1) {  // what k-step 3 of a slab before slab 0 would have issued
      const uint32_t la = a_lds(1);
      static_for<HA>([&](auto t_c) { load_one(t_c, la, la, k_ok_of(1)); });
    }
    // H1: slab s+1 exists, H2: slab s+2 exists
    auto slab2 = [&](auto h1_c, auto h2_c, int s, int bs) {
      constexpr bool H1 = decltype(h1_c)::value, H2 = decltype(h2_c)::value;
      const uint8_t *sa = a_ptr(s & 1), *sb = b_ptr(bs);
      const int bs1 = bs == 2 ? 0 : bs + 1, bs2 = bs1 == 2 ? 0 : bs1 + 1;
      const uint32_t la1 = a_lds((s + 1) & 1), lb2 = b_lds(bs2);
      step(ic<0>{}, ic<HA>{}, ic<1>{}, ic<H1 ? A_LOADS - HA : 0>{}, ic<1>{}, la1, la1, k_ok_of(s + 1), sa, sb);
      step(ic<1>{}, ic<A_LOADS>{}, ic<1>{}, ic<H2 ? HB : 0>{}, ic<2>{}, lb2, lb2, k_ok_of(s + 2), sa, sb);
      step(ic<2>{}, ic<A_LOADS + HB>{}, ic<1>{}, ic<H2 ? BL - HB : 0>{}, ic<3>{}, lb2, lb2, k_ok_of(s + 2), sa, sb);
      if constexpr (H1) {
        __builtin_amdgcn_s_waitcnt(H2 ? wait_but_b : 0x0070);
        __syncthreads();
      }
      const uint32_t la2 = a_lds(s & 1);  // slab s+2's activations reuse this slab's stage
      step(ic<3>{}, ic<0>{}, ic<1>{}, ic<H2 ? HA : 0>{}, ic<H1 ? 0 : -1>{}, la2, la2, k_ok_of(s + 2), a_ptr((s + 1) & 1),
           b_ptr(bs1));
    };
    int s = 0, bs = 0;
    for (; s + 2 < nslab; ++s) {
      slab2(T_{}, T_{}, s, bs);
      bs = bs == 2 ? 0 : bs + 1;
    }
    if (s + 1 < nslab) {
      slab2(T_{}, F_{}, s, bs);
      bs = bs == 2 ? 0 : bs + 1;
      ++s;
    }
    slab2(F_{}, F_{}, s, bs);
  } else {

  // vmcnt(n) with lgkmcnt(0): n in bits [3:0] and [15:14]
  auto wait_loads = [&](int younger) {
    if (younger == 0) __builtin_amdgcn_s_waitcnt(0x0070);
    else __builtin_amdgcn_s_waitcnt(0x0070 | (LOADS * (NS - 2) & 15) | (((LOADS * (NS - 2)) >> 4) << 14));
  };
  static_assert(LOADS * (NS - 2) < 64, "vmcnt range");
  auto next = [](int st) { return st + 1 == NS ? 0 : st + 1; };
  constexpr auto nl = [](int lp) { return (LOADS - lp + PARTS - 1) / PARTS; };  // loads lp, lp + PARTS, ...

  // Slab s lives in LDS stage s % NS.  Its k-steps 0..2 prefetch the fragments of the step after
  // them; then the wavefront waits until its own loads of slab s+1 have landed and its fragment
  // reads of this stage have returned, and meets the others at the slab's one barrier.  Past the
  // barrier slab s+1 is visible to everybody and nobody reads this stage any more, so k-step 3
  // prefetches the first fragments of slab s+1 and starts refilling this stage with slab s+NS;
  // the rest of that slab's loads go out during k-steps 0.. of slab s+1.  (With two stages the
  // loads must land within the same slab and are issued in the first two of those steps only.)
  //   IA: slab s+NS-1 exists (loads in steps 0..2), IB: slab s+NS exists (loads in step 3),
  //   LAST: no slab s+1.
  auto slab = [&](auto ia_c, auto ib_c, auto last_c, int s, int cs, int ls) {
    constexpr bool IA = decltype(ia_c)::value, IB = decltype(ib_c)::value, LAST = decltype(last_c)::value;
    const uint8_t* st = smem + cs * SM::stage_bytes;
    const uint8_t* sb = st + SM::a_bytes;
    const uint32_t ld_a = __builtin_amdgcn_readfirstlane(smem_lds + ls * SM::stage_bytes + wave * 1024);
    const bool ok_a = (s + NS - 1) * BK + a_kc < K;
    step(ic<0>{}, ic<1>{}, ic<PARTS>{}, ic<(IA && PARTS > 1) ? nl(1) : 0>{}, ic<1>{}, ld_a, ld_a + SM::a_bytes, ok_a, st, sb);
    step(ic<1>{}, ic<2>{}, ic<PARTS>{}, ic<(IA && PARTS > 2) ? nl(2) : 0>{}, ic<2>{}, ld_a, ld_a + SM::a_bytes, ok_a, st, sb);
    step(ic<2>{}, ic<3>{}, ic<PARTS>{}, ic<(IA && PARTS > 3) ? nl(3) : 0>{}, ic<3>{}, ld_a, ld_a + SM::a_bytes, ok_a, st, sb);
    if constexpr (!LAST) {
      wait_loads(IA ? 1 : 0);
      __syncthreads();
    }
    const uint32_t ld_b = __builtin_amdgcn_readfirstlane(smem_lds + cs * SM::stage_bytes + wave * 1024);
    const uint8_t* nst = smem + next(cs) * SM::stage_bytes;
    step(ic<3>{}, ic<0>{}, ic<PARTS>{}, ic<IB ? nl(0) : 0>{}, ic<LAST ? -1 : 0>{}, ld_b, ld_b + SM::a_bytes,
         (s + NS) * BK + a_kc < K, nst, nst + SM::a_bytes);
  };

#pragma unroll
  for (int p = 0; p < NS - 1; ++p)
    if (p < nslab) load_slab(p, p * BK);
  // slab 0 must have landed; later prologue loads may still be in flight (exact count only
  // matters for speed: waiting for everything is always correct)
  wait_loads(nslab >= NS - 1 ? 1 : 0);
  __syncthreads();
  static_for<(kM16 ? TM + CH : READS)>([&](auto q_c) { read_one(q_c, ic<0>{}, ic<0>{}, smem, smem + SM::a_bytes); });
  if (NS - 1 < nslab) {  // the share of slab NS-1 that a slab's k-step 3 would have issued
    const uint32_t st = __builtin_amdgcn_readfirstlane(smem_lds + (NS - 1) * SM::stage_bytes + wave * 1024);
    const bool k_ok = (NS - 1) * BK + a_kc < K;
    static_for<(LOADS + PARTS - 1) / PARTS>([&](auto q_c) { load_one(ic<PARTS * decltype(q_c)::value>{}, st, st + SM::a_bytes, k_ok); });
  }
  int cs = 0, ls = NS - 1, s = 0;
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
  slab(F_{}, F_{}, T_{}, s, cs, ls);  // the last slab: nothing left to fetch or prefetch
  }  // one ring for both operands

  // Epilogue.  acc[.][i][j][r] holds D[m][n] with m = tile row l32 and
  // n = (r/4)*8 + lg*4 + r%4 of the 32x32 tile: a lane owns 4 consecutive columns of 32 different
  // rows, which as direct stores would touch 32 cache lines per instruction.  So each wavefront
  // turns its block around through LDS (free now), 32 rows at a time in fp32: written as the
  // MFMA left it, read back row by row, so that 64 lanes store (and read C from) whole 512-byte
  // runs.  Rows are padded by 16 bytes: both directions are free of bank conflicts.
  constexpr int CW = BN / WN;        // columns of the wavefront's block
  constexpr int ROWP = CW * 4 + 16;  // bytes per padded fp32 row
  constexpr int CPR = CW / 4;        // 4-column groups per row
  static_assert(NW * 32 * ROWP <= (int)SM::bytes && (32 * CPR) % 64 == 0, "epilogue staging");
  constexpr int PASSES = BM / WM / 32;  // 32 rows of the wavefront's block per pass
  auto ep_of = [&](int row) { return smem + wave * (32 * ROWP) + row * ROWP; };
  // the pass's rows as the MFMA left them: a lane's 4 consecutive columns of a row, 16 bytes
  auto stage_pass = [&](int i, auto value) {
    if constexpr (kM16) {
#pragma unroll
      for (int ii = 0; ii < 2; ++ii)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          float4_t v;
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = value(2 * i + ii, j, e);
          *reinterpret_cast<float4_t*>(ep_of(ii * 16 + l16) + (j * 16 + lq * 4) * 4) = v;
        }
    } else {
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
          float4_t v;
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = value(i, j, qd * 4 + e);
          *reinterpret_cast<float4_t*>(ep_of(l32) + (j * 32 + qd * 8 + lg * 4) * 4) = v;
        }
    }
  };
  __syncthreads();  // every wavefront has read its last fragments
  uint8_t* ep = smem + wave * (32 * ROWP);
  constexpr int ITER = 32 * CPR / 64;  // 4-column groups per lane and pass
  typedef unsigned int u32v2_t __attribute__((ext_vector_type(2)));
#pragma unroll
  for (int i = 0; i < PASSES; ++i) {
    // C and D go through buffer descriptors based at the pass's first row and ending with the
    // matrix (rows >= M fall outside and are dropped by the hardware; columns >= N get an
    // out-of-range offset), so the pass has no branches and all its loads are in flight together.
    const int gm0 = m_base + wm * (BM / WM) + i * 32, gn0 = n_base + wn * CW;
    const int rows = M - gm0 < 32 ? M - gm0 : 32;
    const int recs = rows > 0 ? rows * N * 2 : 0;
    const size_t row0 = (size_t)(rows > 0 ? gm0 : 0) * N;
    const __amdgpu_buffer_rsrc_t d_rsrc = __builtin_amdgcn_make_buffer_rsrc(D + row0, 0, recs, 0x00020000);
    uint32_t off[ITER];
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int c = it * 64 + lane, gn = gn0 + (c % CPR) * 4;
      off[it] = gn < N ? (uint32_t)((c / CPR) * N + gn) * 2u : kOob;
    }
    u32v2_t cv[ITER];
    if constexpr (!kDual && !kPartial) {
      if (beta != 0.f) {  // issued first: the longest latency of the pass
        // C has row stride ldc (N, or 0 when one row is added to every row of the product):
        // the D offset less the row's share of the difference
        const int c_recs = rows > 0 ? ((rows - 1) * ldc + N) * 2 : 0;
        const uint32_t c_skip = (uint32_t)(N - ldc) * 2u;
        const __amdgpu_buffer_rsrc_t c_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint16_t*>(C) + (size_t)(rows > 0 ? gm0 : 0) * ldc, 0, c_recs, 0x00020000);
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
          const uint32_t r = (uint32_t)((it * 64 + lane) / CPR);
          cv[it] = __builtin_amdgcn_raw_buffer_load_b64(c_rsrc, off[it] == kOob ? kOob : off[it] - r * c_skip, 0, 0);
        }
      }
    }
    if constexpr (kPartial) {
      // the fp32 sums as they are, one product after the other through the staging area; the
      // gate sums go to D, the up sums of the dual form to C (both float [M][N] here)
      typedef unsigned int u32v4_t __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        stage_pass(i, [&](int ti, int tj, int r) { return kM16 ? acc[b][ti][tj / G][(tj % G) * 4 + r] : acc[b][ti][tj][r]; });
        float* dst = b == 0 ? reinterpret_cast<float*>(D) : reinterpret_cast<float*>(const_cast<uint16_t*>(C));
        const __amdgpu_buffer_rsrc_t p_rsrc =
            __builtin_amdgcn_make_buffer_rsrc(dst + row0, 0, rows > 0 ? rows * N * 4 : 0, 0x00020000);
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
          const int c = it * 64 + lane;
          const float4_t p4 = *reinterpret_cast<const float4_t*>(ep + (c / CPR) * ROWP + (c % CPR) * 16);
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32v4_t, p4), p_rsrc,
                                                 off[it] == kOob ? kOob : off[it] * 2u, 0, 0);
        }
      }
      continue;
    }
    stage_pass(i, [&](int ti, int tj, int r) {
      const int gj = kM16 ? tj / G : tj, gr = kM16 ? (tj % G) * 4 + r : r;
      if constexpr (kDual) return swiglu_rounded<E>(acc[0][ti][gj][gr], acc[1][ti][gj][gr]);
      else return acc[0][ti][gj][gr];
    });
    float4_t a4[ITER];
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int c = it * 64 + lane;
      a4[it] = *reinterpret_cast<const float4_t*>(ep + (c / CPR) * ROWP + (c % CPR) * 16);
    }
    auto store_group = [&](int it, float4_t v) {
      __builtin_amdgcn_raw_buffer_store_b64(u32v2_t{E::pack2(v[0], v[1]), E::pack2(v[2], v[3])}, d_rsrc, off[it], 0, 0);
    };
    if (kDual) {
#pragma unroll
      for (int it = 0; it < ITER; ++it) store_group(it, a4[it]);
    } else if (beta == 0.f) {
#pragma unroll
      for (int it = 0; it < ITER; ++it) store_group(it, a4[it] * alpha);
    } else {
#pragma unroll
      for (int it = 0; it < ITER; ++it) {
        float4_t v = a4[it] * alpha;
        v[0] += beta * E::widen(cv[it].x & 0xffffu);
        v[1] += beta * E::widen(cv[it].x >> 16);
        v[2] += beta * E::widen(cv[it].y & 0xffffu);
        v[3] += beta * E::widen(cv[it].y >> 16);
        store_group(it, v);
      }
    }
  }
}

// XCD-aware tile order: consecutive workgroup ids land on different XCDs (8 of them), so give
// each XCD one contiguous range of the n tiles (M fastest) to share weight panels in its L2.
__device__ __forceinline__ int xcd_order(int bid, int n) {
  return (bid % 8) * ((n + 7) / 8) + bid / 8;
}

// The tile of workgroup `bid` in a launch of tiles_m x tiles_n tiles.  An XCD's L2 fetches every
// activation row panel and every weight column panel its tiles touch, so the memory side carries
// (row panels + column panels per XCD) x 8: with 16 or more tile rows, each XCD takes half of the
// rows and a quarter of the columns instead of all rows and an eighth of the columns (32 tiles in
// flight as 8 x 4 instead of 16 x 2: a fifth less traffic on the layer's 2048-row launches, which
// buys 0.3-1.4 % of their time).
__device__ __forceinline__ bool xcd_tile(int bid, int tiles_m, int tiles_n, int* tm, int* tn) {
  if (tiles_m >= 16 && tiles_m % 2 == 0 && tiles_n % 4 == 0) {
    const int x = bid % 8, i = bid / 8, hm = tiles_m / 2, qn = tiles_n / 4;
    if (i >= hm * qn) return false;
    *tm = (x & 1) * hm + i % hm;
    *tn = (x >> 1) * qn + i / hm;
    return true;
  }
  const int logical = xcd_order(bid, tiles_m * tiles_n);
  if (logical >= tiles_m * tiles_n) return false;
  *tm = logical % tiles_m;
  *tn = logical / tiles_m;
  return true;
}

template <class E, int BM, int BN, int WM, int WN, bool kDual, bool kBCol>
__global__ __launch_bounds__(WM * WN * 64) void gemm_f16_kernel(
    const uint16_t* __restrict__ A, const uint16_t* __restrict__ B0,
    const uint16_t* __restrict__ B1, const uint16_t* C, uint16_t* D,
    int M, int N, int K, float alpha, float beta, int ldc, int tiles_m, int tiles_n) {
  int tm, tn;
  if (!xcd_tile(blockIdx.x, tiles_m, tiles_n, &tm, &tn)) return;
  gemm_tile<E, BM, BN, WM, WN, kDual, kBCol>(A, B0, B1, C, D, M, N, K, alpha, beta, ldc, tm * BM, tn * BN, K);
}

// Two tile heights in one launch, for shapes whose 256-row tiles fill the 256 CUs a whole number
// of times plus at most half a round: the first n_big tiles (in M-fastest order) are computed
// 256 rows high, each of the rest as two 128-row halves by two workgroups, so the last round
// takes half the time instead of leaving half the CUs idle.
template <class E, int BN, bool kDual, bool kBCol>
__global__ __launch_bounds__(256) void gemm_f16_hybrid_kernel(
    const uint16_t* __restrict__ A, const uint16_t* __restrict__ B0,
    const uint16_t* __restrict__ B1, const uint16_t* C, uint16_t* D,
    int M, int N, int K, float alpha, float beta, int ldc, int tiles_m, int tiles_n, int n_big) {
  const int big_grid = (n_big + 7) / 8 * 8;
  if ((int)blockIdx.x < big_grid) {
    const int t = xcd_order(blockIdx.x, n_big);
    if (t >= n_big) return;
    gemm_tile<E, 256, BN, 2, 2, kDual, kBCol>(A, B0, B1, C, D, M, N, K, alpha, beta, ldc,
                                            (t % tiles_m) * 256, (t / tiles_m) * BN, K);
  } else {
    const int n_small = 2 * (tiles_m * tiles_n - n_big);
    const int u = xcd_order(blockIdx.x - big_grid, n_small);
    if (u >= n_small) return;
    const int t = n_big + u / 2;
    const int m_base = (t % tiles_m) * 256 + (u & 1) * 128;
    if (m_base >= M) return;
    gemm_tile<E, 128, BN, 2, 2, kDual, kBCol>(A, B0, B1, C, D, M, N, K, alpha, beta, ldc, m_base,
                                            (t / tiles_m) * BN, K);
  }
}

// A GEMM with too few output tiles to fill the chip (few rows against a narrow N), split over K:
// workgroup (tile, share) computes the tile's sums over k in [share * k_per, ...) and stores them
// as fp32 to P[share][M][N]; splitk_reduce_kernel adds the shares and applies alpha, beta and C.
// kDual: two weight matrices; the sums of the second go to P1[share][M][N].
template <class E, int BM, int BN, int WM, int WN, bool kDual, bool kBCol>
__global__ __launch_bounds__(WM * WN * 64) void gemm_f16_splitk_kernel(
    const uint16_t* __restrict__ A, const uint16_t* __restrict__ B, const uint16_t* __restrict__ B1,
    float* __restrict__ P, float* __restrict__ P1, int M, int N, int K, int shares, int k_per, int tiles_m,
    int tiles_n) {
  const int total = tiles_m * tiles_n * shares;
  const int logical = xcd_order(blockIdx.x, total);
  if (logical >= total) return;
  const int share = logical % shares, tile = logical / shares;
  const int k0 = share * k_per;
  const int k_len = K - k0 < k_per ? K - k0 : k_per;
  const size_t b_off = kBCol ? (size_t)k0 : (size_t)k0 * N, p_off = (size_t)share * M * N;
  gemm_tile<E, BM, BN, WM, WN, kDual, kBCol, true>(
      A + k0, B + b_off, kDual ? B1 + b_off : nullptr,
      kDual ? reinterpret_cast<const uint16_t*>(P1 + p_off) : nullptr, reinterpret_cast<uint16_t*>(P + p_off), M, N,
      k_len, 1.f, 0.f, N, (tile % tiles_m) * BM, (tile / tiles_m) * BN, K);
}

// out[m][n..n+3] = round(silu(g) * u) with g = round(sum_s P0[s][m][n..]), u likewise from P1: the
// epilogue of the fused gate/up pair on the summed shares.
template <class E>
__global__ __launch_bounds__(256) void splitk_reduce_dual_kernel(const float* __restrict__ P0,
                                                                 const float* __restrict__ P1, int shares,
                                                                 uint16_t* out, int M, int N) {
  const size_t groups = (size_t)M * N / 4, mn = (size_t)M * N;
  for (size_t g = (size_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += (size_t)gridDim.x * 256) {
    const float4_t a = sum_shares(P0, mn, g * 4, shares), b = sum_shares(P1, mn, g * 4, shares);
    float4_t v;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = swiglu_rounded<E>(a[e], b[e]);
    *reinterpret_cast<u32x2*>(out + g * 4) = u32x2{E::pack2(v[0], v[1]), E::pack2(v[2], v[3])};
  }
}

// D[m][n..n+3] = round(alpha * sum_s P[s][m][n..] + beta * C[m][n..]); C has row stride ldc.
template <class E>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ P, int shares,
                                                            const uint16_t* C, int ldc, uint16_t* D,
                                                            int M, int N, float alpha, float beta) {
  const size_t groups = (size_t)M * N / 4, mn = (size_t)M * N;
  for (size_t g = (size_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += (size_t)gridDim.x * 256) {
    float4_t v = sum_shares(P, mn, g * 4, shares) * alpha;
    if (beta != 0.f) {
      const size_t m = g * 4 / N, n = g * 4 % N;
      const u32x2 c = *reinterpret_cast<const u32x2*>(C + m * ldc + n);
      v[0] += beta * E::widen(c.x & 0xffffu);
      v[1] += beta * E::widen(c.x >> 16);
      v[2] += beta * E::widen(c.y & 0xffffu);
      v[3] += beta * E::widen(c.y >> 16);
    }
    *reinterpret_cast<u32x2*>(D + g * 4) = u32x2{E::pack2(v[0], v[1]), E::pack2(v[2], v[3])};
  }
}

// kDual: B1 is the second weight matrix, C is not used, D = the SwiGLU output.
template <class E, int BM, int BN, int WM, int WN, bool kBCol, bool kDual = false>
static int launch_splitk(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int M, int N,
                         int K, float alpha, float beta, int ldc, int shares, int k_per, float* P,
                         hipStream_t stream, const uint16_t* B1 = nullptr) {
  using SM = GemmSmem<BM, BN, kDual ? 2 : 1>;
  auto kern = gemm_f16_splitk_kernel<E, BM, BN, WM, WN, kDual, kBCol>;
  float* P1 = kDual ? P + (size_t)shares * M * N : nullptr;
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
  const int grid = ((tiles_m * tiles_n * shares + 7) / 8) * 8;
  kern<<<grid, WM * WN * 64, SM::bytes, stream>>>(A, B, B1, P, P1, M, N, K, shares, k_per, tiles_m, tiles_n);
  int rc = check_launch("gemm split-K launch");
  if (rc) return rc;
  const size_t groups = (size_t)M * N / 4;
  const int rgrid = (int)std::min<size_t>((groups + 255) / 256, 2048);
  if constexpr (kDual) splitk_reduce_dual_kernel<E><<<rgrid, 256, 0, stream>>>(P, P1, shares, D, M, N);
  else splitk_reduce_kernel<E><<<rgrid, 256, 0, stream>>>(P, shares, C, ldc, D, M, N, alpha, beta);
  return check_launch("gemm split-K reduction launch");
}

template <class E, int BM, int BN, int WM, int WN, bool kDual, bool kBCol>
static int launch_gemm(const uint16_t* A, const uint16_t* B0, const uint16_t* B1, const uint16_t* C,
                       uint16_t* D, int M, int N, int K, float alpha, float beta, int ldc,
                       hipStream_t stream) {
  using SM = GemmSmem<BM, BN, kDual ? 2 : 1>;
  auto kern = gemm_f16_kernel<E, BM, BN, WM, WN, kDual, kBCol>;
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
  kern<<<grid, WM * WN * 64, SM::bytes, stream>>>(A, B0, B1, C, D, M, N, K, alpha, beta, ldc, tiles_m, tiles_n);
  return check_launch("gemm launch");
}

template <class E, int BN, bool kDual, bool kBCol>
static int launch_hybrid(const uint16_t* A, const uint16_t* B0, const uint16_t* B1, const uint16_t* C,
                         uint16_t* D, int M, int N, int K, float alpha, float beta, int ldc, int n_big,
                         hipStream_t stream) {
  constexpr size_t big = GemmSmem<256, BN, kDual ? 2 : 1>::bytes, small = GemmSmem<128, BN, kDual ? 2 : 1>::bytes;
  constexpr size_t lds = big > small ? big : small;
  auto kern = gemm_f16_hybrid_kernel<E, BN, kDual, kBCol>;
  static bool attr_set = false;  // benign race: the call is idempotent
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) {
      set_error("gemm: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
      return NF_ERR_RUNTIME;
    }
    attr_set = true;
  }
  const int tiles_m = (M + 255) / 256, tiles_n = (N + BN - 1) / BN;
  const int n_small = 2 * (tiles_m * tiles_n - n_big);
  const int grid = (n_big + 7) / 8 * 8 + (n_small + 7) / 8 * 8;
  kern<<<grid, 256, lds, stream>>>(A, B0, B1, C, D, M, N, K, alpha, beta, ldc, tiles_m, tiles_n, n_big);
  return check_launch("gemm launch");
}

// Compute units of the current device (256 on MI355X); one workgroup of these kernels fills one.
static int cu_count() {
  static int n = 0;  // benign race: every caller computes the same value
  if (n == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
      v = 256;
    n = v;
  }
  return n;
}

// Split over K: for at most 512 rows whose tiles (64 x 256 up to 64 rows, 128 x 128 up to 256,
// 320 x 128 up to 320, else 256 x 256) would leave more than half of the CUs idle, as many shares
// as fill them, each at least 512 deep.  Above 256 rows the unsplit launch already fills the chip
// with 128 x 128 tiles, but those pass the weight bytes through LDS once per 128 rows.  From 257
// to 320 rows one 320-row tile per column panel passes them once (267 x 10240 x 8192: 72 -> 63 us,
// 267 x 8192 x 28672: 209 -> 188 us, 267 x 4096 x 4096: 32 -> 28 us).  From 321 to 512 rows two
// 256-row tiles per panel pass them twice instead of four times, but half of the second tile's
// MFMAs are padding: measured, that pays for a long contraction only (the down projection), so
// there the split needs K >= 12288.
// Returns the number of shares (1 = no split) and their depth.
constexpr int kSplitMaxRows = 512;
constexpr int kTallRows = 320;  // 257 .. 320 rows: one 320 x 128 tile per column panel
static int splitk_plan(int M, int N, int K, int* k_per) {
  if (M > kSplitMaxRows || K < 1024 || (M > kTallRows && K < 12288)) return 1;
  const int bm = M <= 64 ? 64 : M <= 256 ? 128 : M <= kTallRows ? 320 : 256;
  const int bn = M <= 64 || M > kTallRows ? 256 : 128;
  const int tiles = ((M + bm - 1) / bm) * ((N + bn - 1) / bn);
  const int cus = cu_count();
  int shares = std::min(std::min(cus / tiles, K / 512), kMaxShares);
  if (shares < 2) return 1;
  *k_per = ((K + shares - 1) / shares + BK - 1) / BK * BK;
  return (K + *k_per - 1) / *k_per;  // shares that are not empty
}

// More than 512 rows whose 256 x 256 tiles number half the CUs or fewer against a long contraction
// (the 8B down projection: 2048 x 4096 x 14336, 128 tiles): two shares of K on 256 x 256 tiles fill
// the chip, and with K that long the 67 MB of fp32 sums written, read back and added by a second
// launch cost less than the smaller 128 x 256 tile does (measured with streamed [N][K] weights:
// 199 us against 211; at K = 4096, the O projection, the split loses: 78 us against 64).
constexpr int kDenseSplitMinK = 8192;
static int dense_split_plan(int M, int N, int K, int* k_per) {
  if (M <= kSplitMaxRows || K < kDenseSplitMinK) return 1;
  const long long t256 = (long long)((M + 255) / 256) * ((N + 255) / 256);
  if (t256 * 2 > cu_count() || t256 * 2 <= cu_count() / 2) return 1;
  *k_per = ((K + 1) / 2 + BK - 1) / BK * BK;
  return 2;
}

// The same for the fused gate/up pair (tiles of 64 x 128 up to 64 rows, 128 x 128 up to 256,
// 320 x 128 on eight wavefronts up to 320).
static int splitk_plan_dual(int M, int N, int K, int* k_per) {
  if (M > kTallRows || K < 1024) return 1;
  const int bm = M <= 64 ? 64 : M <= 256 ? 128 : 320;
  const int tiles = ((M + bm - 1) / bm) * ((N + 127) / 128);
  const int shares = std::min(std::min(cu_count() / tiles, K / 512), kMaxShares);
  if (shares < 2) return 1;
  *k_per = ((K + shares - 1) / shares + BK - 1) / BK * BK;
  return (K + *k_per - 1) / *k_per;
}

// Tile choice.  A launch takes tiles / CUs rounds of one tile per CU, a round costing the tile's
// area over its relative efficiency (bigger tiles re-read less through LDS); the cheapest candidate
// wins.  A last, partly filled round is not charged in full: the part is power-bound, so the
// fewer CUs clock higher, and measured it costs 0.47 + 0.53 x its fill (a quarter-full round 0.61,
// three quarters 0.86 of a full one).  Efficiencies and that rule are fitted to launches of 1024
// and 2048 rows on the Llama-3-8B and -70B layer shapes WITH THE WEIGHTS STREAMED FROM HBM, as a
// layer's weights are (multiplying by the same weights again finds the smaller matrices in the
// 256 MB last-level cache and flatters tiles with two LDS stages): the model picks the fastest of
// the three tiles in all ten cases.  2048 x 6144 x 4096 runs on 192 tiles of 256x256 (93-98 us)
// rather than 384 of 128x256 (116-122) or 768 of 128x128 (118-120).  A 128x384 tile, which fills
// the chip exactly once on that shape, has room for two LDS stages only, and a load that misses
// the cache does not land within a slab: 102-105 us, and last or second to last in every case;
// it is not a candidate.  Short M uses a 64-row tile so that padding rows do not dominate.
template <class E, bool kBCol>
static int dispatch_plain(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D,
                          int M, int N, int K, float alpha, float beta, int ldc, hipStream_t s) {
  if (M <= 64) return launch_gemm<E, 64, 256, 1, 4, false, kBCol>(A, B, nullptr, C, D, M, N, K, alpha, beta, ldc, s);
  const int cus = cu_count();
  auto cost = [&](int bm, int bn, double eff) {
    const long long tiles = (long long)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
    const long long full = tiles / cus, rest = tiles % cus;
    const double rounds = (double)full + (rest ? 0.47 + 0.53 * (double)rest / cus : 0.0);
    return rounds * bm * bn / eff;
  };
  double c256 = cost(256, 256, 1.0);
  const double c128x256 = cost(128, 256, 0.95), c128 = cost(128, 128, 0.80);
  // 256x256 tiles that fill the chip a whole number of times plus at most half a round: the tiles of
  // that last round are computed as two 128-row halves by two workgroups each, in the same launch
  // (2048 x 10240 x 8192, 320 tiles: 256 + 2 x 64)
  const long long t256 = (long long)((M + 255) / 256) * ((N + 255) / 256);
  const int rest256 = (int)(t256 % cus);
  const bool two_heights = t256 > cus && rest256 > 0 && rest256 <= cus / 2;
  if (two_heights)
    c256 = ((double)(t256 / cus) + 0.5 * (0.47 + 0.53 * 2.0 * rest256 / cus) / 0.95) * 256 * 256;
  // k-contiguous weights only: 256 x 192, which fills the chip exactly once on 2048 x 6144 (QKV: 84 us
  // against 89 on 192 tiles of 256 x 256) at 0.965 of the larger tile's efficiency (LM head: 1772 us
  // against 1715 for the same area)
  const double c256x192 = kBCol ? cost(256, 192, 0.965) : 1e300;
  const double best = std::min(std::min(c256, c256x192), std::min(c128x256, c128));
  if constexpr (kBCol)
    if (best == c256x192 && best < c256)
      return launch_gemm<E, 256, 192, 2, 2, false, true>(A, B, nullptr, C, D, M, N, K, alpha, beta, ldc, s);
  if (best == c256 && two_heights)
    return launch_hybrid<E, 256, false, kBCol>(A, B, nullptr, C, D, M, N, K, alpha, beta, ldc, (int)(t256 - rest256), s);
  if (best == c256) return launch_gemm<E, 256, 256, 2, 2, false, kBCol>(A, B, nullptr, C, D, M, N, K, alpha, beta, ldc, s);
  if (best == c128x256) return launch_gemm<E, 128, 256, 2, 2, false, kBCol>(A, B, nullptr, C, D, M, N, K, alpha, beta, ldc, s);
  return launch_gemm<E, 128, 128, 2, 2, false, kBCol>(A, B, nullptr, C, D, M, N, K, alpha, beta, ldc, s);
}

// ---- a caller-chosen tile and split over K (the cta_m / cta_n / split_k fields of a GEMM tag).
// The menu: 64 x 256, 128 x 128, 128 x 256, 256 x 256 for both weight layouts, 256 x 192 for
// k-contiguous weights (a row of a [K][N] slab must hold a multiple of 16 chunks for its swizzle).
struct MenuTile {
  int bm, bn;
  bool col_only;
};
constexpr MenuTile kTileMenu[] = {{64, 256, false}, {128, 128, false}, {128, 256, false}, {256, 256, false}, {256, 192, true}};
constexpr int kTileMenuSize = (int)(sizeof(kTileMenu) / sizeof(kTileMenu[0]));

// The menu entry closest to (tile_m, tile_n) in log scale, among those the layout allows.
static int menu_pick(int tile_m, int tile_n, bool b_col) {
  int best = -1;
  double best_d = 1e30;
  for (int i = 0; i < kTileMenuSize; ++i) {
    if (kTileMenu[i].col_only && !b_col) continue;
    const double dm = std::log((double)kTileMenu[i].bm / tile_m), dn = std::log((double)kTileMenu[i].bn / tile_n);
    const double d = std::fabs(dm) + std::fabs(dn);
    if (d < best_d) {
      best_d = d;
      best = i;
    }
  }
  return best;
}

// shares of a forced split: at most kMaxShares, each at least one slab deep
static int forced_shares(int K, int split_k, int* k_per) {
  int shares = std::min(std::min(split_k, kMaxShares), (K + BK - 1) / BK);
  if (shares < 2) return 1;
  *k_per = ((K + shares - 1) / shares + BK - 1) / BK * BK;
  return (K + *k_per - 1) / *k_per;
}

template <class E, int BM, int BN, int WM, int WN, bool kBCol>
static int launch_menu(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int M, int N, int K,
                       float alpha, float beta, int ldc, int shares, int k_per, float* P, hipStream_t s) {
  if (shares > 1) return launch_splitk<E, BM, BN, WM, WN, kBCol>(A, B, C, D, M, N, K, alpha, beta, ldc, shares, k_per, P, s);
  return launch_gemm<E, BM, BN, WM, WN, false, kBCol>(A, B, nullptr, C, D, M, N, K, alpha, beta, ldc, s);
}

template <class E, bool kBCol>
static int dispatch_menu(int index, const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int M, int N,
                         int K, float alpha, float beta, int ldc, int shares, int k_per, float* P, hipStream_t s) {
  switch (index) {
    case 0: return launch_menu<E, 64, 256, 1, 4, kBCol>(A, B, C, D, M, N, K, alpha, beta, ldc, shares, k_per, P, s);
    case 1: return launch_menu<E, 128, 128, 2, 2, kBCol>(A, B, C, D, M, N, K, alpha, beta, ldc, shares, k_per, P, s);
    case 2: return launch_menu<E, 128, 256, 2, 2, kBCol>(A, B, C, D, M, N, K, alpha, beta, ldc, shares, k_per, P, s);
    case 3: return launch_menu<E, 256, 256, 2, 2, kBCol>(A, B, C, D, M, N, K, alpha, beta, ldc, shares, k_per, P, s);
    case 4:
      if constexpr (kBCol) return launch_menu<E, 256, 192, 2, 2, true>(A, B, C, D, M, N, K, alpha, beta, ldc, shares, k_per, P, s);
      break;
  }
  set_error("gemm: no tile %d in the menu for this weight layout", index);
  return NF_ERR_INVALID_ARGUMENT;
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
  // operands are addressed through 32-bit buffer offsets, which run up to a tile past the last
  // row or column and a few slabs past K before they are discarded
  NF_REQUIRE(((size_t)M + 256) * ((size_t)K + 512) * 2 < 0xFFFFFF00ull &&
                 ((size_t)N + 256) * ((size_t)K + 512) * 2 < 0xFFFFFF00ull,
             "%s: an operand of %d x %d x %d exceeds the 4 GiB buffer-addressing limit", who, M, N, K);
  return NF_OK;
}

template <class E>
static int gemm_entry(const char* who, const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D,
                      int M, int N, int K, float alpha, float beta, int b_col_major, nf_stream_t stream,
                      bool c_is_row = false) {
  int rc = check_gemm_args(who, A, B, D, M, N, K);
  if (rc) return rc;
  NF_REQUIRE(beta == 0.f || C, "%s: beta=%g needs C", who, (double)beta);
  NF_REQUIRE(((uintptr_t)C) % 8 == 0, "%s: C must be 8-byte aligned", who);
  if (M == 0) return NF_OK;
  hipStream_t s = (hipStream_t)stream;
  const int ldc = c_is_row ? 0 : N;  // row stride of C: 0 reads the same row for every m
  return b_col_major ? dispatch_plain<E, true>(A, B, C, D, M, N, K, alpha, beta, ldc, s)
                     : dispatch_plain<E, false>(A, B, C, D, M, N, K, alpha, beta, ldc, s);
}

// gemm_entry with a workspace: shapes that profit are split over K through it.
template <class E>
static int gemm_ws_entry(const char* who, const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D,
                         int M, int N, int K, float alpha, float beta, int b_col_major, void* workspace,
                         size_t workspace_bytes, nf_stream_t stream, bool c_is_row = false) {
  int k_per = 0;
  const bool shape_ok = M > 0 && N > 0 && K > 0 && N % 8 == 0 && K % 8 == 0;
  int shares = shape_ok ? splitk_plan(M, N, K, &k_per) : 1;
  const bool dense = shares < 2 && shape_ok && (shares = dense_split_plan(M, N, K, &k_per)) > 1;
  if (shares < 2 || !workspace || workspace_bytes < (size_t)shares * M * N * sizeof(float))
    return gemm_entry<E>(who, A, B, C, D, M, N, K, alpha, beta, b_col_major, stream, c_is_row);
  int rc = check_gemm_args(who, A, B, D, M, N, K);
  if (rc) return rc;
  NF_REQUIRE(beta == 0.f || C, "%s: beta=%g needs C", who, (double)beta);
  NF_REQUIRE(((uintptr_t)C) % 8 == 0 && (uintptr_t)workspace % 16 == 0, "%s: C must be 8-byte and the workspace 16-byte aligned", who);
  hipStream_t s = (hipStream_t)stream;
  float* P = static_cast<float*>(workspace);
  if (dense)
    return b_col_major ? launch_splitk<E, 256, 256, 2, 2, true>(A, B, C, D, M, N, K, alpha, beta, c_is_row ? 0 : N, shares, k_per, P, s)
                       : launch_splitk<E, 256, 256, 2, 2, false>(A, B, C, D, M, N, K, alpha, beta, c_is_row ? 0 : N, shares, k_per, P, s);
  if (M <= 64)
    return b_col_major ? launch_splitk<E, 64, 256, 1, 4, true>(A, B, C, D, M, N, K, alpha, beta, c_is_row ? 0 : N, shares, k_per, P, s)
                       : launch_splitk<E, 64, 256, 1, 4, false>(A, B, C, D, M, N, K, alpha, beta, c_is_row ? 0 : N, shares, k_per, P, s);
  if (M > 256 && M <= kTallRows)
    return b_col_major ? launch_splitk<E, 320, 128, 2, 2, true>(A, B, C, D, M, N, K, alpha, beta, c_is_row ? 0 : N, shares, k_per, P, s)
                       : launch_splitk<E, 320, 128, 2, 2, false>(A, B, C, D, M, N, K, alpha, beta, c_is_row ? 0 : N, shares, k_per, P, s);
  if (M > 256)
    return b_col_major ? launch_splitk<E, 256, 256, 2, 2, true>(A, B, C, D, M, N, K, alpha, beta, c_is_row ? 0 : N, shares, k_per, P, s)
                       : launch_splitk<E, 256, 256, 2, 2, false>(A, B, C, D, M, N, K, alpha, beta, c_is_row ? 0 : N, shares, k_per, P, s);
  return b_col_major ? launch_splitk<E, 128, 128, 2, 2, true>(A, B, C, D, M, N, K, alpha, beta, c_is_row ? 0 : N, shares, k_per, P, s)
                     : launch_splitk<E, 128, 128, 2, 2, false>(A, B, C, D, M, N, K, alpha, beta, c_is_row ? 0 : N, shares, k_per, P, s);
}

template <class E, bool kBCol>
static int dual_entry(const char* who, const uint16_t* A, const uint16_t* Bgate, const uint16_t* Bup,
                      uint16_t* out, int M, int N, int K, nf_stream_t stream) {
  int rc = check_gemm_args(who, A, Bgate, out, M, N, K);
  if (rc) return rc;
  NF_REQUIRE(M == 0 || Bup, "%s: null pointer", who);
  NF_REQUIRE(((uintptr_t)Bup) % 16 == 0, "%s: operands must be 16-byte aligned", who);
  if (M == 0) return NF_OK;
  hipStream_t s = (hipStream_t)stream;
  if (M <= 64)
    return launch_gemm<E, 64, 128, 2, 2, true, kBCol>(A, Bgate, Bup, nullptr, out, M, N, K, 1.f, 0.f, N, s);
  // 257 .. 320 rows against enough column panels to fill the chip: one 320-row tile per panel, so
  // the weights pass through LDS once instead of three times; its two 320 x 128 accumulators are
  // spread over eight wavefronts (160 registers each)
  if (M > 256 && M <= kTallRows && (N + 127) / 128 >= 192)
    return launch_gemm<E, 320, 128, 2, 4, true, kBCol>(A, Bgate, Bup, nullptr, out, M, N, K, 1.f, 0.f, N, s);
  const long long t256 = (long long)((M + 255) / 256) * ((N + 127) / 128);
  const int tail = M % 256;  // rows in the last 256-row tile: half-empty tiles go to the 128-row kernel
  if (t256 >= 192 && (tail == 0 || tail > 128)) {
    const int cus = cu_count();
    const int rest = (int)(t256 % cus);  // tiles of the last, partial round
    if (t256 > cus && rest > 0 && rest <= cus / 2)
      return launch_hybrid<E, 128, true, kBCol>(A, Bgate, Bup, nullptr, out, M, N, K, 1.f, 0.f, N, (int)(t256 - rest), s);
    return launch_gemm<E, 256, 128, 2, 2, true, kBCol>(A, Bgate, Bup, nullptr, out, M, N, K, 1.f, 0.f, N, s);
  }
  return launch_gemm<E, 128, 128, 2, 2, true, kBCol>(A, Bgate, Bup, nullptr, out, M, N, K, 1.f, 0.f, N, s);
}

template <class E, bool kBCol>
static int dual_ws_entry(const char* who, const uint16_t* A, const uint16_t* Bgate, const uint16_t* Bup,
                         uint16_t* out, int M, int N, int K, void* workspace, size_t workspace_bytes,
                         nf_stream_t stream) {
  int k_per = 0;
  const int shares = M > 0 && N > 0 && K > 0 && N % 8 == 0 && K % 8 == 0 ? splitk_plan_dual(M, N, K, &k_per) : 1;
  if (shares < 2 || !workspace || workspace_bytes < (size_t)2 * shares * M * N * sizeof(float))
    return dual_entry<E, kBCol>(who, A, Bgate, Bup, out, M, N, K, stream);
  int rc = check_gemm_args(who, A, Bgate, out, M, N, K);
  if (rc) return rc;
  NF_REQUIRE(Bup && ((uintptr_t)Bup | (uintptr_t)workspace) % 16 == 0, "%s: Bup and the workspace must be 16-byte aligned", who);
  hipStream_t s = (hipStream_t)stream;
  float* P = static_cast<float*>(workspace);
  if (M <= 64)
    return launch_splitk<E, 64, 128, 2, 2, kBCol, true>(A, Bgate, nullptr, out, M, N, K, 1.f, 0.f, N, shares, k_per, P, s, Bup);
  if (M > 256)
    return launch_splitk<E, 320, 128, 2, 4, kBCol, true>(A, Bgate, nullptr, out, M, N, K, 1.f, 0.f, N, shares, k_per, P, s, Bup);
  return launch_splitk<E, 128, 128, 2, 2, kBCol, true>(A, Bgate, nullptr, out, M, N, K, 1.f, 0.f, N, shares, k_per, P, s, Bup);
}

// ---- the entry point that allocates nothing: split-K partial sums in a static device array.
// In host code the array's name is only a stand-in for the symbol; its device address is looked
// up once per device (each device holds its own copy) and only that address is handed to kernels.
constexpr size_t kStaticScratchBytes = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices] = {};  // benign race: every caller stores the same address

static int static_scratch(const char* who, void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("%s: cannot tell the current device", who);
    return NF_ERR_RUNTIME;
  }
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      set_error("%s: hipGetSymbolAddress(scratch) on device %d: %s", who, dev, hipGetErrorString(e));
      return NF_ERR_RUNTIME;
    }
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return NF_OK;
}

extern "C" {

int nf_gemm_f16(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int M, int N,
                int K, float alpha, float beta, int b_col_major, nf_stream_t stream) {
  return gemm_entry<F16>("nf_gemm_f16", A, B, C, D, M, N, K, alpha, beta, b_col_major, stream);
}

size_t nf_gemm_workspace_bytes(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  int k_per = 0;
  int shares = splitk_plan(M, N, K, &k_per);
  if (shares < 2) shares = dense_split_plan(M, N, K, &k_per);
  return shares < 2 ? 0 : (size_t)shares * M * N * sizeof(float);
}

size_t nf_gemm_workspace_bytes_upto(int max_M, int N, int K) {
  size_t need = 0;
  for (int m = 1; m <= max_M && m <= kSplitMaxRows; ++m) need = std::max(need, nf_gemm_workspace_bytes(m, N, K));
  // above that only the two-share split of launches with few 256 x 256 tiles: every count of tile rows
  for (int m = kSplitMaxRows + 1; m <= max_M; m = (m + 255) / 256 * 256 + 1)
    need = std::max(need, nf_gemm_workspace_bytes(std::min((m + 255) / 256 * 256, max_M), N, K));
  return need;
}

size_t nf_dual_swiglu_workspace_bytes(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  int k_per = 0;
  const int shares = splitk_plan_dual(M, N, K, &k_per);
  return shares < 2 ? 0 : (size_t)2 * shares * M * N * sizeof(float);
}

size_t nf_dual_swiglu_workspace_bytes_upto(int max_M, int N, int K) {
  size_t need = 0;
  for (int m = 1; m <= max_M && m <= kTallRows; ++m) need = std::max(need, nf_dual_swiglu_workspace_bytes(m, N, K));
  return need;
}

int nf_dual_swiglu_f16_ws(const uint16_t* A, const uint16_t* Bgate, const uint16_t* Bup, uint16_t* out, int M,
                          int N, int K, int b_col_major, void* workspace, size_t workspace_bytes, nf_stream_t stream) {
  return b_col_major ? dual_ws_entry<F16, true>("nf_dual_swiglu_f16_ws", A, Bgate, Bup, out, M, N, K, workspace,
                                                workspace_bytes, stream)
                     : dual_ws_entry<F16, false>("nf_dual_swiglu_f16_ws", A, Bgate, Bup, out, M, N, K, workspace,
                                                 workspace_bytes, stream);
}

int nf_gemm_f16_ws(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int M, int N, int K,
                   float alpha, float beta, int b_col_major, void* workspace, size_t workspace_bytes,
                   nf_stream_t stream) {
  return gemm_ws_entry<F16>("nf_gemm_f16_ws", A, B, C, D, M, N, K, alpha, beta, b_col_major, workspace,
                            workspace_bytes, stream);
}

int nf_gemm_f16_noalloc(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int M, int N, int K,
                        float alpha, float beta, int b_col_major, nf_stream_t stream) {
  // the few-row split only: the two-share split of dense launches is an optimisation that needs more
  // than the array holds at any shape it applies to, and such a launch runs unsplit here
  int k_per = 0;
  const int few = M > 0 && N > 0 && K > 0 ? splitk_plan(M, N, K, &k_per) : 1;
  const size_t need = few < 2 ? 0 : (size_t)few * M * N * sizeof(float);
  NF_REQUIRE(need <= kStaticScratchBytes,
             "nf_gemm_f16_noalloc: %d x %d x %d is split over K through %zu bytes of partial sums; the static "
             "scratch array holds %zu (use nf_gemm_f16_ws with a workspace of your own, or nf_gemm_f16)",
             M, N, K, need, kStaticScratchBytes);
  void* ws = nullptr;
  if (need) {  // shapes that are not split never touch the array
    const int rc = static_scratch("nf_gemm_f16_noalloc", &ws);
    if (rc) return rc;
  }
  return gemm_ws_entry<F16>("nf_gemm_f16_noalloc", A, B, C, D, M, N, K, alpha, beta, b_col_major, ws,
                            need ? kStaticScratchBytes : 0, stream);
}

size_t nf_gemm_noalloc_scratch_bytes(void) { return kStaticScratchBytes; }

int nf_gemm_tile_menu(int index, int* tile_m, int* tile_n, int* k_contiguous_weights_only) {
  if (index >= 0 && index < kTileMenuSize) {
    if (tile_m) *tile_m = kTileMenu[index].bm;
    if (tile_n) *tile_n = kTileMenu[index].bn;
    if (k_contiguous_weights_only) *k_contiguous_weights_only = kTileMenu[index].col_only ? 1 : 0;
  }
  return kTileMenuSize;
}

size_t nf_gemm_tiled_workspace_bytes(int M, int N, int K, int split_k) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  int k_per = 0;
  const int shares = forced_shares(K, split_k, &k_per);
  return shares < 2 ? 0 : (size_t)shares * M * N * sizeof(float);
}

int nf_gemm_f16_tiled(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int M, int N, int K,
                      float alpha, float beta, int b_col_major, int c_is_row, int tile_m, int tile_n, int split_k,
                      void* workspace, size_t workspace_bytes, nf_stream_t stream) {
  const char* who = "nf_gemm_f16_tiled";
  NF_REQUIRE(tile_m > 0 && tile_n > 0, "%s: tile %d x %d", who, tile_m, tile_n);
  int rc = check_gemm_args(who, A, B, D, M, N, K);
  if (rc) return rc;
  NF_REQUIRE(beta == 0.f || C, "%s: beta=%g needs C", who, (double)beta);
  NF_REQUIRE(((uintptr_t)C) % 8 == 0, "%s: C must be 8-byte aligned", who);
  if (M == 0) return NF_OK;
  int k_per = 0;
  const int shares = forced_shares(K, split_k, &k_per);
  NF_REQUIRE(shares < 2 || (workspace && (uintptr_t)workspace % 16 == 0 &&
                            workspace_bytes >= (size_t)shares * M * N * sizeof(float)),
             "%s: a split over K into %d shares needs a 16-byte aligned workspace of %zu bytes (nf_gemm_tiled_workspace_bytes)",
             who, shares, (size_t)shares * M * N * sizeof(float));
  const int index = menu_pick(tile_m, tile_n, b_col_major != 0);
  const int ldc = c_is_row ? 0 : N;
  float* P = static_cast<float*>(workspace);
  hipStream_t s = (hipStream_t)stream;
  return b_col_major ? dispatch_menu<F16, true>(index, A, B, C, D, M, N, K, alpha, beta, ldc, shares, k_per, P, s)
                     : dispatch_menu<F16, false>(index, A, B, C, D, M, N, K, alpha, beta, ldc, shares, k_per, P, s);
}

int nf_gemm_bias_f16_ws(const uint16_t* A, const uint16_t* B, const uint16_t* bias, uint16_t* D, int M, int N,
                        int K, float alpha, float beta, int b_col_major, void* workspace, size_t workspace_bytes,
                        nf_stream_t stream) {
  NF_REQUIRE(bias, "nf_gemm_bias_f16_ws: null bias");
  return gemm_ws_entry<F16>("nf_gemm_bias_f16_ws", A, B, bias, D, M, N, K, alpha, beta, b_col_major, workspace,
                            workspace_bytes, stream, true);
}

int nf_gemm_bias_f16(const uint16_t* A, const uint16_t* B, const uint16_t* bias, uint16_t* D, int M,
                     int N, int K, float alpha, float beta, int b_col_major, nf_stream_t stream) {
  NF_REQUIRE(bias, "nf_gemm_bias_f16: null bias");
  return gemm_entry<F16>("nf_gemm_bias_f16", A, B, bias, D, M, N, K, alpha, beta, b_col_major, stream, true);
}

int nf_dual_swiglu_f16(const uint16_t* A, const uint16_t* Bgate, const uint16_t* Bup, uint16_t* out,
                       int M, int N, int K, int b_col_major, nf_stream_t stream) {
  return b_col_major ? dual_entry<F16, true>("nf_dual_swiglu_f16", A, Bgate, Bup, out, M, N, K, stream)
                     : dual_entry<F16, false>("nf_dual_swiglu_f16", A, Bgate, Bup, out, M, N, K, stream);
}

int nf_gemm_bf16(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, int M, int N,
                 int K, float alpha, float beta, int b_col_major, nf_stream_t stream) {
  return gemm_entry<BF16>("nf_gemm_bf16", A, B, C, D, M, N, K, alpha, beta, b_col_major, stream);
}

int nf_dual_swiglu_bf16(const uint16_t* A, const uint16_t* Bgate, const uint16_t* Bup, uint16_t* out,
                        int M, int N, int K, nf_stream_t stream) {
  return dual_entry<BF16, false>("nf_dual_swiglu_bf16", A, Bgate, Bup, out, M, N, K, stream);
}

}  // extern "C"
