// Paged-KV attention for gfx950: decode (one query row per request, HBM-bound) and chunked
// prefill (causal, many rows) on v_mfma_f32_16x16x32_f16.
//
// Formulation per (request, kv head):   S^T = K . Q^T   then   O^T = V^T . P^T
//   * the MFMA "column" dimension (16 wide) carries query rows: column c of a block is
//     (token c / GROUP, q head c % GROUP) of the kv head's GQA group, so decode with GROUP 4
//     uses 4 live columns and a prefill block packs 16 / GROUP tokens;
//   * S^T comes out of the first MFMA with a lane holding 4 consecutive kv positions of one
//     column -- exactly the B-operand layout of the second MFMA, so P never leaves registers;
//   * K and V pages go from global memory straight into LDS (buffer_load ... lds); K rows are
//     read back as 16-byte A operands, V^T operands come from the transposing LDS read.
// Online softmax runs in the exp2 domain with fp32 state per column; masked keys contribute
// exactly zero (the reference's -5e4 mask underflows to zero in fp32 as well).
//
// Decode: a workgroup's wavefronts split the request's pages (32 keys per step each) and
// merge (m, l, O) through LDS; work item = (request, kv head), ordered so that the workgroups
// one XCD starts together are the heads of one request and stream the same 64 KiB pages.  Prefill: a workgroup is a
// 16-token tile (for GQA 4) whose wavefronts share the streamed K/V tiles; tiles are planned
// on the device from qo_indptr (prefix of tiles per request) -- no host round trip in either mode.
#include <type_traits>

#include "common.h"

namespace nf {

constexpr int D = 128;      // head_dim
constexpr int PAGE = 16;    // kv entries per page

union H8 {
  u32x4 u;
  half8_t h;
  uint32_t w[4];
};

// Tile plan of a chunked-prefill launch, made on the device (no host round trip):
//   tile_start[i] = number of query tiles (wg_tok tokens each) of requests < i; tile_start[batch] = total;
//   tile_order[k] = the tile that workgroup slot k computes: tiles in descending order of the keys
//   they see.  A causal chunk's last tile sees the whole context and its first tile only what came
//   before the chunk, and a launch is over when its longest tile is, so the long tiles start first
//   and the short ones fill in behind them.  (Ranked by counting, at most kPlanSortMax tiles;
//   beyond that tiles keep their order.)
//   first_wave > 0: the number of slots k whose workgroups are the first on their CU.  When all
//   tiles fit into two such waves every workgroup is resident from the start, nothing fills in
//   behind anything, and what counts is which two tiles share a CU: the second wave then runs from
//   the shortest tile up, so that the longest tile shares its CU with the shortest.
constexpr int kPlanSortMax = 1024;
__global__ __launch_bounds__(256) void attn_plan_kernel(const int32_t* __restrict__ qo_indptr,
                                                        const int32_t* __restrict__ kv_indptr,
                                                        const int32_t* __restrict__ kv_last_page_len,
                                                        int32_t* __restrict__ tile_start, int32_t* __restrict__ tile_order,
                                                        int batch, int wg_tok, int causal, int first_wave) {
  __shared__ int s_sum[256];
  __shared__ int s_key[kPlanSortMax];
  const int per = (batch + 255) / 256;
  const int lo = threadIdx.x * per, hi = min(lo + per, batch);
  int sum = 0;
  for (int i = lo; i < hi; ++i) {
    int len = qo_indptr[i + 1] - qo_indptr[i];
    sum += len > 0 ? (len + wg_tok - 1) / wg_tok : 0;
  }
  s_sum[threadIdx.x] = sum;
  __syncthreads();
  // inclusive scan over the 256 partial sums (Hillis-Steele)
  for (int off = 1; off < 256; off <<= 1) {
    int v = threadIdx.x >= off ? s_sum[threadIdx.x - off] : 0;
    __syncthreads();
    s_sum[threadIdx.x] += v;
    __syncthreads();
  }
  int run = s_sum[threadIdx.x] - sum;  // exclusive prefix of this thread's range
  const int total = s_sum[255];
  if (threadIdx.x == 255) tile_start[batch] = total;
  for (int i = lo; i < hi; ++i) {
    tile_start[i] = run;
    const int len = qo_indptr[i + 1] - qo_indptr[i];
    const int n = len > 0 ? (len + wg_tok - 1) / wg_tok : 0;
    if (total <= kPlanSortMax) {  // keys the request's tiles see
      const int npages = kv_indptr[i + 1] - kv_indptr[i];
      const int kv_len = npages > 0 ? (npages - 1) * PAGE + kv_last_page_len[i] : 0;
      for (int t = 0; t < n; ++t) {
        const int last = min((t + 1) * wg_tok, len) - 1;
        s_key[run + t] = causal ? min(kv_len, kv_len - len + last + 1) : kv_len;
      }
    }
    run += n;
  }
  __syncthreads();
  if (total > kPlanSortMax) {
    for (int t = threadIdx.x; t < total; t += 256) tile_order[t] = t;
    return;
  }
  for (int t = threadIdx.x; t < total; t += 256) {
    const int key = s_key[t];
    int rank = 0;
    for (int u = 0; u < total; ++u) rank += (s_key[u] > key) || (s_key[u] == key && u < t);
    const bool pair_up = first_wave > 0 && total <= 2 * first_wave && rank >= first_wave;
    tile_order[pair_up ? first_wave + (total - 1 - rank) : rank] = t;
  }
}

// Decode attention (one query row per request, or few): the HBM-bound kernel.  Same
// formulation and column packing as attn_paged_kernel; what differs is how K and V travel:
//
//   * K and V pages go from global memory STRAIGHT INTO LDS (buffer_load ... lds), not through
//     registers: the load-to-register path of a CU saturates near 38 GB/s, the direct path
//     carries half again as much from HBM, and the data in flight no longer costs registers.
//   * A workgroup is (request, kv head); its NW wavefronts take every NW-th 32-key step and merge
//     (m, l, O) at the end.  Every wavefront owns a private LDS ring (2 K tiles + 2 V tiles of
//     32 keys x 256 bytes), so no barrier is needed while streaming: a wavefront only waits
//     for its own loads (s_waitcnt vmcnt), and refills a tile as soon as its MFMAs have read it
//     -- the K tile of step i+2 is requested right after the score MFMAs of step i.
//   * Layout in LDS = the page layout (one 256-byte row per key), with the 16-byte chunks of a
//     row permuted on the way in so that operand reads are bank-conflict free: K row r keeps
//     chunk c at c ^ (r & 15) (16-byte A-operand reads), V row r keeps chunk c at
//     c ^ ((r & 7) << 1) and is read with the transposing LDS read (ds_read_b64_tr_b16), which
//     hands each lane 4 consecutive keys of one feature: the V^T operand with no permutes.
//   * The loads carry the non-temporal hint: every K and V byte is read once per launch, and
//     without the hint the same pattern streams 10 % slower.
//   * A page is addressed through its own buffer descriptor (base = page, 64 KiB range), so
//     pools larger than 4 GiB need no 64-bit per-lane arithmetic and out-of-page offsets
//     (used to zero-fill V rows past the end of the sequence) read as zero.
template <int GROUP, int NW>
__global__ __launch_bounds__(NW * 64, 1) void attn_decode_kernel(
    const uint16_t* __restrict__ q, uint16_t* __restrict__ o, const int32_t* __restrict__ qo_indptr,
    const uint16_t* __restrict__ kv_data, const int32_t* __restrict__ kv_indptr,
    const int32_t* __restrict__ kv_indices, const int32_t* __restrict__ kv_last_page_len, int batch,
    int Hq, int Hkv, int causal, float scale_log2) {
  constexpr int TPB = 16 / GROUP;  // tokens per 16-column block = tokens per work item pass
  constexpr int WAVE_LDS = 32768;  // per wavefront: K0 K1 V0 V1, 8 KB each
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c16 = lane & 15, g = lane >> 4;
  const uint32_t wlds = __builtin_amdgcn_readfirstlane(lds0 + wave * WAVE_LDS);  // DMA destination base
  uint8_t* const wptr = lds + wave * WAVE_LDS;                                   // same, for reads
  const uint32_t page_bytes = (uint32_t)(2 * PAGE * Hkv * D * 2);
  const uint32_t v_half = (uint32_t)(PAGE * Hkv * D * 2);  // byte offset of the V half of a page

  // operand read offsets inside a tile (constant per lane)
  uint32_t kx[4];  // K: row blk*16 + c16, logical chunk 4j + g
#pragma unroll
  for (int j = 0; j < 4; ++j) kx[j] = (uint32_t)(c16 * 256 + (((j * 4 + g) ^ c16) << 4));
  // V: lanes 16g..16g+15 read the 4(key) x 16(feature) block of keys 4g.. and features 16i..;
  // lane i16 addresses key 4g + i16/4, features 16i + 4(i16&3)..+3; 32-byte unit i of a row
  // sits at i ^ (key & 7) (the 8 keys x 32 bytes of a read cycle then cover all 64 banks).
  const int i16 = lane & 15, vx_x = ((g & 1) << 2) | ((i16 >> 2) & 3);
  uint32_t vx[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
    vx[i] = (uint32_t)((g * 4 + (i16 >> 2)) * 256 + ((i ^ vx_x) * 32) + (i16 & 3) * 8);

  // Work item w -> (request, kv head).  Workgroup ids go round the 8 XCDs, so in groups of 8
  // requests the item order is (head, request): the workgroups an XCD starts one after the other
  // are then the heads of ONE request, which walk the same pages at about the same time and pull
  // each key's 256-byte rows of all heads -- one contiguous Hkv x 256 bytes in the pool -- together
  // (the bare load pattern: 6.55 -> 6.76 TB/s).  The requests past the last whole group of 8 keep
  // (request, head) order.
  const long long grouped = (long long)(batch / 8) * 8 * Hkv;
  for (long long w = blockIdx.x; w < (long long)batch * Hkv; w += gridDim.x) {
    int req = (int)(w / Hkv), kvh = (int)(w % Hkv);
    if (w < grouped) {
      const int j = (int)(w % (8 * Hkv));
      req = (int)(w / (8 * Hkv)) * 8 + j % 8;
      kvh = j / 8;
    }
    const int qo0 = qo_indptr[req];
    const int qo_len = qo_indptr[req + 1] - qo0;
    const int pg0 = kv_indptr[req];
    const int npages = kv_indptr[req + 1] - pg0;
    const int kv_len = npages > 0 ? (npages - 1) * PAGE + kv_last_page_len[req] : 0;
    // DMA source offsets inside a page: instruction t4 moves keys 4*t4 .. 4*t4+3 of a page
    // (64 lanes x 16 bytes = 4 rows), lane -> key 4*t4 + lane/16, position lane%16.
    uint32_t k_src[4], v_src[4];
#pragma unroll
    for (int t4 = 0; t4 < 4; ++t4) {
      const int key = 4 * t4 + (lane >> 4), pos = lane & 15;
      const uint32_t row = (uint32_t)((key * Hkv + kvh) * D * 2);
      k_src[t4] = row + (uint32_t)(((pos ^ key) & 15) << 4);
      v_src[t4] = v_half + row + (uint32_t)((pos ^ ((key & 7) << 1)) << 4);
    }
    const int n_sub = (qo_len + TPB - 1) / TPB;
    for (int sub = 0; sub < n_sub; ++sub) {
      const int tok0 = sub * TPB;
      float4_t oacc[8];
      float m_run = -1e30f, l_run = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) oacc[i] = float4_t{0.f, 0.f, 0.f, 0.f};

      // Q operand: column c16 = (token tok0 + c16/GROUP, head c16%GROUP)
      H8 qf[4];
      const int tq = tok0 + c16 / GROUP;
      const bool live = tq < qo_len;
      {
        const uint16_t* qp = q + ((size_t)(qo0 + (live ? tq : 0)) * Hq + kvh * GROUP + c16 % GROUP) * D + g * 8;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          qf[j].u = live ? *reinterpret_cast<const u32x4*>(qp + j * 32) : u32x4{0, 0, 0, 0};
      }
      int key_limit = causal ? kv_len - qo_len + tq : kv_len - 1;
      if (!live) key_limit = -1;
      const int tok_last = min(tok0 + TPB, qo_len) - 1;
      const int kv_end = causal ? min(kv_len, kv_len - qo_len + tok_last + 1) : kv_len;
      const int npairs = (kv_end + 31) >> 5;  // 32-key steps; this wavefront takes wave, wave+4, ...

      auto page_rsrc = [&](int pidx) -> rsrc_t {  // uniform: scalar loads and arithmetic
        const int page = kv_indices[pg0 + (pidx < npages ? pidx : 0)];
        return make_rsrc(kv_data + (size_t)page * (page_bytes / 2), page_bytes);
      };
      auto dma_k = [&](int pp, int buf) {
        const rsrc_t ra = page_rsrc(2 * pp), rb = page_rsrc(2 * pp + 1);
        const uint32_t dst = wlds + buf * 8192;
#pragma unroll
        for (int t4 = 0; t4 < 4; ++t4) load16_to_lds_nt(ra, k_src[t4], dst + t4 * 1024);
#pragma unroll
        for (int t4 = 0; t4 < 4; ++t4) load16_to_lds_nt(rb, k_src[t4], dst + 4096 + t4 * 1024);
      };
      auto dma_v = [&](int pp, int buf) {
        const rsrc_t ra = page_rsrc(2 * pp), rb = page_rsrc(2 * pp + 1);
        const uint32_t dst = wlds + 16384 + buf * 8192;
        // rows past the end of the sequence may hold anything (NaN x 0 = NaN): zero-fill them
        const int first_key = pp * 32 + (lane >> 4);
#pragma unroll
        for (int t4 = 0; t4 < 4; ++t4)
          load16_to_lds_nt(ra, first_key + 4 * t4 < kv_len ? v_src[t4] : kOob, dst + t4 * 1024);
#pragma unroll
        for (int t4 = 0; t4 < 4; ++t4)
          load16_to_lds_nt(rb, first_key + 16 + 4 * t4 < kv_len ? v_src[t4] : kOob, dst + 4096 + t4 * 1024);
      };
      // vmcnt(n): everything but the n youngest load instructions of this wavefront has landed
      auto wait_but = [&](int younger) {
        if (younger >= 24) __builtin_amdgcn_s_waitcnt(0x0F70 | (24 & 15) | ((24 >> 4) << 14));
        else if (younger >= 16) __builtin_amdgcn_s_waitcnt(0x0F70 | (16 & 15) | ((16 >> 4) << 14));
        else if (younger >= 8) __builtin_amdgcn_s_waitcnt(0x0F70 | 8);
        else __builtin_amdgcn_s_waitcnt(0x0F70);
      };

      // two steps in flight before the loop
      if (wave < npairs) {
        dma_k(wave, 0);
        dma_v(wave, 0);
      }
      if (wave + NW < npairs) {
        dma_k(wave + NW, 1);
        dma_v(wave + NW, 1);
      }
      // The compiler does not see the DMA loads above but does see the Q loads: left alone it waits
      // for them where Q is first used, inside the loop below, with vmcnt(0) on EVERY pass -- which
      // also waits for every K and V tile in flight and leaves the ring one step deep.  A use of Q
      // here makes it wait once, now (for Q and the tiles just requested).
#pragma unroll
      for (int j = 0; j < 4; ++j) asm volatile("" ::"v"(qf[j].w[0]));
      int buf = 0;
      for (int pp = wave; pp < npairs; pp += NW, buf ^= 1) {
        const int t_base = pp * 32;
        const bool n1 = pp + NW < npairs, n2 = pp + 2 * NW < npairs;
        const uint8_t* kt = wptr + buf * 8192;
        const uint8_t* vt = wptr + 16384 + buf * 8192;

        // ---- scores: K(pp) has landed once only V(pp), K(pp+4), V(pp+4) may still be in flight
        wait_but(n1 ? 24 : 8);
        float4_t s[2];
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
          s[blk] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const half8_t kf = *reinterpret_cast<const half8_t*>(kt + blk * 4096 + kx[j]);
            s[blk] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[j].h, s[blk], 0, 0, 0);
          }
        }
        // the K tile is free as soon as those reads have returned: s depends on them
        if (n2) {
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          dma_k(pp + 2 * NW, buf);
        }

        // ---- online softmax; lane holds keys t_base + blk*16 + g*4 + r of column c16
        float mx = -1e30f;
        bool ok[2][4];
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int t = t_base + blk * 16 + g * 4 + r;
            ok[blk][r] = t <= key_limit && t < kv_len;
            s[blk][r] *= scale_log2;
            if (ok[blk][r]) mx = fmaxf(mx, s[blk][r]);
          }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        float psum = 0.f;
        uint32_t pw[4];
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
          for (int rr = 0; rr < 2; ++rr) {
            float p0 = ok[blk][2 * rr] ? __builtin_amdgcn_exp2f(s[blk][2 * rr] - m_new) : 0.f;
            float p1 = ok[blk][2 * rr + 1] ? __builtin_amdgcn_exp2f(s[blk][2 * rr + 1] - m_new) : 0.f;
            psum += p0 + p1;  // the row sum uses the unrounded values, P.V the fp16 ones
            pw[blk * 2 + rr] = f2h_bits(p0) | (f2h_bits(p1) << 16);
          }
        H8 pf;
        pf.u = u32x4{pw[0], pw[1], pw[2], pw[3]};
        l_run = l_run * alpha + psum;

        // ---- P.V: V(pp) has landed once only K(pp+4), V(pp+4), K(pp+8) may still be in flight
        wait_but((n1 ? 16 : 0) + (n2 ? 8 : 0));
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const uint8_t* vp = vt + vx[i];
          const short4_t lo = lds_read_tr16(vp);         // keys 4g..4g+3 of the first page
          const short4_t hi = lds_read_tr16(vp + 4096);  // ... of the second page
          typedef short short8_t __attribute__((ext_vector_type(8)));
          const short8_t v8 = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          oacc[i] *= alpha;
          oacc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, v8), pf.h, oacc[i], 0, 0, 0);
        }
        if (n2) {
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          dma_v(pp + 2 * NW, buf);
        }
      }
      l_run += __shfl_xor(l_run, 16, 64);
      l_run += __shfl_xor(l_run, 32, 64);

      // ---- merge the wavefronts.  oacc[i][r] = O[column c16][feature 16i + 4g + r].  Each
      // wavefront parks its partial result in its own LDS region (its streaming is over).
      float* s_o = reinterpret_cast<float*>(wptr);             // [8][4][64]
      float* s_m = reinterpret_cast<float*>(wptr + 8192);      // [64]
      float* s_l = reinterpret_cast<float*>(wptr + 8192 + 256);
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) s_o[(i * 4 + r) * 64 + lane] = oacc[i][r];
      s_m[lane] = m_run;
      s_l[lane] = l_run;
      __syncthreads();
      float M = -1e30f, mw[NW];
#pragma unroll
      for (int ww = 0; ww < NW; ++ww) {
        mw[ww] = *reinterpret_cast<const float*>(lds + ww * WAVE_LDS + 8192 + lane * 4);
        M = fmaxf(M, mw[ww]);
      }
      float wgt[NW], L = 0.f;
#pragma unroll
      for (int ww = 0; ww < NW; ++ww) {
        wgt[ww] = __builtin_amdgcn_exp2f(mw[ww] - M);
        L += wgt[ww] * *reinterpret_cast<const float*>(lds + ww * WAVE_LDS + 8192 + 256 + lane * 4);
      }
      const float inv = L > 0.f ? 1.0f / L : 0.f;
      if (live) {
        // wavefront w finishes 8/NW of the 16-feature blocks: 4 consecutive features per lane and i
        uint16_t* op = o + ((size_t)(qo0 + tq) * Hq + kvh * GROUP + c16 % GROUP) * D;
#pragma unroll
        for (int e = 0; e < 8 / NW; ++e) {
          const int i = (8 / NW) * wave + e;
          float v[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float acc = 0.f;
#pragma unroll
            for (int ww = 0; ww < NW; ++ww)
              acc += wgt[ww] * *reinterpret_cast<const float*>(lds + ww * WAVE_LDS + ((i * 4 + r) * 64 + lane) * 4);
            v[r] = acc * inv;
          }
          u32x2 out;
          out.x = f2h_bits(v[0]) | (f2h_bits(v[1]) << 16);
          out.y = f2h_bits(v[2]) | (f2h_bits(v[3]) << 16);
          *reinterpret_cast<u32x2*>(op + 16 * i + 4 * g) = out;
        }
      }
      __syncthreads();  // the merge reads are done before the next pass streams into the rings
    }
  }
}

// max over the four 16-lane groups of a wavefront (lanes c, c + 16, c + 32, c + 48), in every lane:
// two lane-swap instructions (v_permlane32_swap, v_permlane16_swap: gfx950) and two maxima on the
// vector unit, where a shuffle would make two round trips through the LDS crossbar.
__device__ __forceinline__ float max_over_lane_groups(float v) {
  const auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float sum_over_lane_groups(float v) {
  const auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Chunked-prefill attention (causal, many rows per request).  A workgroup is one tile of
// 4 * NQB * (16 / GROUP) query tokens of one request and one kv head; each wavefront owns NQB
// blocks of 16 MFMA columns of it (a column = one token and one q head of the kv head's group).
// The K and V pages are streamed ONCE per workgroup, straight into a ring of NSTAGE LDS stages
// (32 keys x 256 bytes each for K and for V) that all four wavefronts read: every wavefront
// issues a quarter of a stage's load instructions, waits for its own, and one barrier per 32-key
// step makes the stage visible and frees the oldest one for the next loads.  LDS layout and
// operand reads are those of attn_decode_kernel.
//
// What bounds it is the LDS read port and the vector unit, not the matrix pipe: a step's K and V
// fragments (8 + 16 LDS reads per wavefront) feed 16 MFMAs per column block, and every score costs
// a maximum, a fused multiply-add, an exponential, an addition and half a conversion on the vector
// unit.  So a wavefront keeps NQB column blocks in registers and reuses each fragment NQB times,
// the scale is folded into the exponent (p = exp2(s * scale - m * scale): one instruction), maxima
// are reduced across lane groups with lane swaps instead of shuffles, and MINWG workgroups share a
// CU so that one wavefront's exponentials run under another's MFMAs.  Steps that lie wholly below
// the causal limit of a wavefront's first token need no masks (most steps of a long chunk);
// wavefronts whose tokens cannot see a step's keys skip its arithmetic but keep loading and
// meeting at the barrier.  Workgroup slot k computes tile tile_order[k / Hkv] for kv head k % Hkv:
// long tiles first (attn_plan_kernel), the heads of a tile side by side so that they find each
// other's pages in the L2.
template <int GROUP, int NQB, int NSTAGE, int MINWG>
__global__ __launch_bounds__(256, MINWG) void attn_prefill_kernel(
    const uint16_t* __restrict__ q, uint16_t* __restrict__ o, const int32_t* __restrict__ qo_indptr,
    const uint16_t* __restrict__ kv_data, const int32_t* __restrict__ kv_indptr,
    const int32_t* __restrict__ kv_indices, const int32_t* __restrict__ kv_last_page_len,
    const int32_t* __restrict__ tile_start, const int32_t* __restrict__ tile_order, int batch, int Hq, int Hkv,
    int causal, float scale_log2) {
  static_assert(NSTAGE >= 2 && NSTAGE <= 4, "the waits below count at most two younger steps");
  constexpr int TPB = 16 / GROUP;
  constexpr int WAVE_TOK = NQB * TPB;
  constexpr int WG_TOK = 4 * WAVE_TOK;
  constexpr int STAGE = 16384;  // K tile 8 KB + V tile 8 KB
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c16 = lane & 15, g = lane >> 4;
  const uint32_t page_bytes = (uint32_t)(2 * PAGE * Hkv * D * 2);
  const uint32_t v_half = (uint32_t)(PAGE * Hkv * D * 2);

  uint32_t kx[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) kx[j] = (uint32_t)(c16 * 256 + (((j * 4 + g) ^ c16) << 4));
  const int i16 = lane & 15, vx_x = ((g & 1) << 2) | ((i16 >> 2) & 3);
  uint32_t vx[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
    vx[i] = (uint32_t)((g * 4 + (i16 >> 2)) * 256 + ((i ^ vx_x) * 32) + (i16 & 3) * 8);

  const float lazy_raw = 8.0f / scale_log2;  // 2^8 in units of the unscaled scores
  const int total_tiles = tile_start[batch];
  for (long long w = blockIdx.x; w < (long long)total_tiles * Hkv; w += gridDim.x) {
    const int tile = tile_order[(int)(w / Hkv)], kvh = (int)(w % Hkv);
    int lo = 0, hi = batch;  // request = largest i with tile_start[i] <= tile
    while (hi - lo > 1) {
      int mid = (lo + hi) >> 1;
      if (tile_start[mid] <= tile) lo = mid; else hi = mid;
    }
    const int req = lo, tile_in_req = tile - tile_start[req];
    const int qo0 = qo_indptr[req];
    const int qo_len = qo_indptr[req + 1] - qo0;
    const int pg0 = kv_indptr[req];
    const int npages = kv_indptr[req + 1] - pg0;
    const int kv_len = npages > 0 ? (npages - 1) * PAGE + kv_last_page_len[req] : 0;
    const int wg_tok0 = tile_in_req * WG_TOK;
    const int tok0 = wg_tok0 + wave * WAVE_TOK;
    const bool wave_active = tok0 < qo_len;

    // this wavefront's load instructions: 2 of the 8 of a K tile and of a V tile (instruction
    // t8 = keys 4*t8 .. 4*t8+3 of the 32-key step; t8 < 4 is the first page, else the second)
    uint32_t k_src[2], v_src[2];
    int key_in_step[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int t8 = wave * 2 + e;
      const int key = 4 * (t8 & 3) + (lane >> 4), pos = lane & 15;
      const uint32_t row = (uint32_t)((key * Hkv + kvh) * D * 2);
      k_src[e] = row + (uint32_t)(((pos ^ key) & 15) << 4);
      v_src[e] = v_half + row + (uint32_t)((pos ^ ((key & 7) << 1)) << 4);
      key_in_step[e] = (t8 >> 2) * 16 + key;
    }

    float4_t oacc[NQB][8];
    float m_run[NQB], l_run[NQB];  // running maximum of the UNSCALED scores; partial row sums per lane
    H8 qf[NQB][4];
    int key_limit[NQB];
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb) {
      m_run[nb] = -1e30f;
      l_run[nb] = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) oacc[nb][i] = float4_t{0.f, 0.f, 0.f, 0.f};
      const int tq = tok0 + nb * TPB + c16 / GROUP;
      const bool live = wave_active && tq < qo_len;
      const uint16_t* qp = q + ((size_t)(qo0 + (live ? tq : 0)) * Hq + kvh * GROUP + c16 % GROUP) * D + g * 8;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        qf[nb][j].u = live ? *reinterpret_cast<const u32x4*>(qp + j * 32) : u32x4{0, 0, 0, 0};
      key_limit[nb] = causal ? kv_len - qo_len + tq : kv_len - 1;
      if (!live) key_limit[nb] = -1;
    }
    // keys the workgroup / this wavefront can see at all
    const int wg_last = min(wg_tok0 + WG_TOK, qo_len) - 1;
    const int wg_end = causal ? min(kv_len, kv_len - qo_len + wg_last + 1) : kv_len;
    const int wave_last = min(tok0 + WAVE_TOK, qo_len) - 1;
    const int wave_end = !wave_active ? 0 : (causal ? min(kv_len, kv_len - qo_len + wave_last + 1) : kv_len);
    const int npairs = (wg_end + 31) >> 5;

    // The page ids of 64 steps live in one register (lane i: the page this wavefront loads in step
    // pg_base + i), refilled every 64 steps, and a step's id is read from its lane: a scalar load per
    // step would put a trip to the scalar cache in front of every group of tile loads, and its wait
    // (scalar loads return out of order) would also wait for every LDS read in flight.
    int pg_base = 0;
    int pg_reg = 0;
    auto load_pages = [&](int base) {
      const int pidx = 2 * (base + lane) + (wave >> 1);  // waves 0,1 load the first page of a step, 2,3 the second
      pg_reg = kv_indices[pg0 + (pidx < npages ? pidx : 0)];
      pg_base = base;
    };
    auto dma = [&](int pp, int stage) {
      if (pp >= pg_base + 64) {
        load_pages(pg_base + 64);
        asm volatile("s_waitcnt vmcnt(0)" : "+v"(pg_reg)::"memory");  // once per 64 steps: the ring drains here
      }
      const int page = __builtin_amdgcn_readlane(pg_reg, pp - pg_base);
      const rsrc_t r = make_rsrc(kv_data + (size_t)page * (page_bytes / 2), page_bytes);
      const uint32_t dst = __builtin_amdgcn_readfirstlane(lds0 + stage * STAGE + wave * 2048);
#pragma unroll
      for (int e = 0; e < 2; ++e) load16_to_lds(r, k_src[e], dst + e * 1024);
#pragma unroll
      for (int e = 0; e < 2; ++e)  // rows past the end of the sequence are zero-filled
        load16_to_lds(r, pp * 32 + key_in_step[e] < kv_len ? v_src[e] : kOob, dst + 8192 + e * 1024);
    };
    load_pages(0);
    // (named in the wait so that the compiler takes the register for defined here, not by a load it
    // would wait for again, with everything else in flight, at every use inside the loop)
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(pg_reg)::"memory");

    __syncthreads();  // the previous work item's reads of every stage are done
    // Step pp lives in stage pp % NSTAGE.  The loop is software-pipelined by one step: while the
    // vector unit works through the softmax of step pp, the matrix pipe still runs the P.V MFMAs of
    // step pp-1, and the score MFMAs of step pp+1 are issued before the P.V MFMAs of step pp, so
    // that the next softmax can start as soon as the scores are there.  Iteration pp therefore
    // reads the fragments of step pp+1; the stage of step pp is free after its barrier, and the
    // loads of step pp+NSTAGE go there (NSTAGE-1 steps ahead of the stage being read).
#pragma unroll
    for (int p = 0; p < NSTAGE - 1; ++p)
      if (p < npairs) dma(p, p);
    // the compiler sees the Q loads but not the tile loads: make it wait for Q once, here, instead of
    // with vmcnt(0) where Q is first used inside the loop (which would drain the ring every step)
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb)
#pragma unroll
      for (int j = 0; j < 4; ++j) asm volatile("" ::"v"(qf[nb][j].w[0]));
    const int n_active = (wave_end + 31) >> 5;  // steps whose keys this wavefront's tokens can see: the first n_active

    half8_t kf[2][4], vf[8];
    float4_t s[NQB][2];
    auto wait_step = [&](int step) {  // this wavefront's loads of `step` have landed: all but the 4 of each younger step
      const int younger = min(NSTAGE - 2, npairs - 1 - step);
      if (younger >= 2) __builtin_amdgcn_s_waitcnt(0x0F78);       // vmcnt(8)
      else if (younger == 1) __builtin_amdgcn_s_waitcnt(0x0F74);  // vmcnt(4)
      else __builtin_amdgcn_s_waitcnt(0x0F70);                    // vmcnt(0)
    };
    auto read_k = [&](const uint8_t* kt) {
#pragma unroll
      for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int j = 0; j < 4; ++j) kf[blk][j] = *reinterpret_cast<const half8_t*>(kt + blk * 4096 + kx[j]);
    };
    auto read_v = [&](const uint8_t* vt) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const short4_t vlo = lds_read_tr16(vt + vx[i]);
        const short4_t vhi = lds_read_tr16(vt + vx[i] + 4096);
        typedef short short8_t __attribute__((ext_vector_type(8)));
        vf[i] = __builtin_bit_cast(half8_t, __builtin_shufflevector(vlo, vhi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    };
    // 2 * NQB independent accumulators, the k-chunks outermost: no MFMA waits for the one before it
    auto scores = [&]() {
#pragma unroll
      for (int nb = 0; nb < NQB; ++nb)
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) s[nb][blk] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
          for (int nb = 0; nb < NQB; ++nb)
            s[nb][blk] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[blk][j], qf[nb][j].h, s[nb][blk], 0, 0, 0);
    };

    if (npairs > 0) {  // step 0
      wait_step(0);
      __syncthreads();
      if (NSTAGE - 1 < npairs) dma(NSTAGE - 1, NSTAGE - 1);
      if (n_active > 0) {
        read_k(lds);
        read_v(lds + 8192);
        scores();
      }
    }
    int st = 0;  // pp % NSTAGE
    for (int pp = 0; pp < npairs; ++pp) {
      const int t_base = pp * 32;
      const bool next = pp + 1 < npairs, act = pp < n_active, act_next = pp + 1 < n_active;
      const int st_next = st + 1 == NSTAGE ? 0 : st + 1;
      if (next) {
        wait_step(pp + 1);
        __syncthreads();  // step pp+1 is visible to everybody, and nobody reads the stage of step pp any more
        if (pp + NSTAGE < npairs) dma(pp + NSTAGE, st);
      }
      if (act) {
        H8 pf[NQB];
        float alpha[NQB];
        float4_t sc[NQB][2];  // the scores of this step; s is about to take those of the next
#pragma unroll
        for (int nb = 0; nb < NQB; ++nb)
#pragma unroll
          for (int blk = 0; blk < 2; ++blk) sc[nb][blk] = s[nb][blk];
        if (act_next) read_k(lds + st_next * STAGE);  // on their way while the vector unit works
        // Steps that lie wholly below the causal limit of the wavefront's first token (and inside
        // the sequence) need no masks: most steps of a long chunk.  Same arithmetic either way.
        const bool unmasked = t_base + 31 <= (causal ? kv_len - qo_len + tok0 : kv_len - 1);
        auto softmax_step = [&](auto masked_c) {
          constexpr bool kMasked = decltype(masked_c)::value;
#pragma unroll
          for (int nb = 0; nb < NQB; ++nb) {
            // a lane holds keys t_base + blk*16 + g*4 + r of column c16
            float mx = -1e30f;
            bool ok[2][4];
#pragma unroll
            for (int blk = 0; blk < 2; ++blk)
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const int t = t_base + blk * 16 + g * 4 + r;
                ok[blk][r] = !kMasked || (t <= key_limit[nb] && t < kv_len);
                if (ok[blk][r]) mx = fmaxf(mx, sc[nb][blk][r]);
              }
            mx = max_over_lane_groups(mx);
            // The reference maximum follows the true one lazily: it moves only when a score exceeds it
            // by more than 2^8 after scaling, so p = exp2(...) stays below 256 (fp16 holds that with its
            // full relative precision, the sums are fp32) and the accumulators are rescaled once or twice
            // per tile instead of in most steps.  O / l is the same quotient either way.
            const float m_new = mx > m_run[nb] + lazy_raw ? mx : m_run[nb];
            alpha[nb] = __builtin_amdgcn_exp2f((m_run[nb] - m_new) * scale_log2);
            m_run[nb] = m_new;
            const float shift = -m_new * scale_log2;
            float psum = 0.f;
            uint32_t pw[4];
#pragma unroll
            for (int blk = 0; blk < 2; ++blk)
#pragma unroll
              for (int rr = 0; rr < 2; ++rr) {
                float p0 = ok[blk][2 * rr] ? __builtin_amdgcn_exp2f(__builtin_fmaf(sc[nb][blk][2 * rr], scale_log2, shift)) : 0.f;
                float p1 = ok[blk][2 * rr + 1] ? __builtin_amdgcn_exp2f(__builtin_fmaf(sc[nb][blk][2 * rr + 1], scale_log2, shift)) : 0.f;
                psum += p0 + p1;  // the row sum uses the unrounded values, P.V the fp16 ones
                pw[blk * 2 + rr] = pack_f16x2(p0, p1);
              }
            pf[nb].u = u32x4{pw[0], pw[1], pw[2], pw[3]};
            l_run[nb] = l_run[nb] * alpha[nb] + psum;
          }
        };
        if (unmasked) softmax_step(std::false_type{});
        else softmax_step(std::true_type{});
        if (act_next) scores();
        bool moved = false;
#pragma unroll
        for (int nb = 0; nb < NQB; ++nb) moved |= alpha[nb] != 1.0f;
        if (__builtin_amdgcn_ballot_w64(moved) != 0) {
          // a branch of its own: folded into the MFMA loop it becomes a multiply and a select per register and step
#pragma unroll
          for (int nb = 0; nb < NQB; ++nb)
#pragma unroll
            for (int i = 0; i < 8; ++i) oacc[nb][i] *= alpha[nb];
          asm volatile("" ::: "memory");
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
          for (int nb = 0; nb < NQB; ++nb)
            oacc[nb][i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf[i], pf[nb].h, oacc[nb][i], 0, 0, 0);
        if (act_next) read_v(lds + st_next * STAGE + 8192);
      }
      st = st_next;
    }

    // oacc[nb][i][r] = O[column c16][feature 16i + 4g + r]
    if (wave_active) {
#pragma unroll
      for (int nb = 0; nb < NQB; ++nb) {
        const float l = sum_over_lane_groups(l_run[nb]);
        const int tq = tok0 + nb * TPB + c16 / GROUP;
        if (tq >= qo_len) continue;
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        uint16_t* op = o + ((size_t)(qo0 + tq) * Hq + kvh * GROUP + c16 % GROUP) * D;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          u32x2 out;
          out.x = pack_f16x2(oacc[nb][i][0] * inv, oacc[nb][i][1] * inv);
          out.y = pack_f16x2(oacc[nb][i][2] * inv, oacc[nb][i][3] * inv);
          *reinterpret_cast<u32x2*>(op + 16 * i + 4 * g) = out;
        }
      }
    }
  }
}

template <int GROUP>
static int launch_attn(const uint16_t* q, uint16_t* o, const int32_t* qo_indptr,
                       const uint16_t* kv_data, const int32_t* kv_indptr, const int32_t* kv_indices,
                       const int32_t* kv_last_page_len, int32_t* tile_start, int batch,
                       int max_qo_rows, int Hq, int Hkv, int causal, int num_blocks,
                       hipStream_t stream) {
  const float scale_log2 = 1.4426950408889634f / sqrtf((float)D);
  constexpr int TPB = 16 / GROUP;
  // Decode mode (KV split over the wavefronts, one workgroup per request and kv head) is the
  // right shape when requests carry about one row each; it stays correct for any row count.
  const bool decode_mode = max_qo_rows <= batch;
  // Measured on chunks of 256 to 2048 tokens (alone, and the prefill chunks of a steady-state serving
  // cycle): one column block per wavefront (16-token tiles for a GQA group of 4) beats two, three and
  // four by 10-100 % -- a launch is over when its longest tile is, a tile's steps are serial (barrier,
  // tile loads, fragment reads, 24 MFMAs, softmax), and smaller tiles mean more workgroups to spread
  // over the CUs and to interleave on one; four LDS stages with two workgroups per CU beat 2 x 2 and 3 x 3.
  constexpr int NQB_PREFILL = 1, kPrefillStages = 4, kPrefillMinWg = 2;
  int32_t* tile_order = tile_start + batch + 2;
  long long bound;
  if (decode_mode) {
    bound = (long long)batch * Hkv;
  } else {
    const int wg_tok = 4 * NQB_PREFILL * TPB;
    // workgroup slots that are the first on their CU: one per CU, Hkv workgroups per slot (a capped
    // grid walks its tiles in rounds: long tiles first is the right order there)
    static int cus = 0;  // benign race: every caller computes the same value
    if (cus == 0) {
      int dev = 0, v = 0;
      if (hipGetDevice(&dev) != hipSuccess ||
          hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
        v = 256;
      cus = v;
    }
    const int first_wave = num_blocks > 0 ? 0 : cus / Hkv;
    attn_plan_kernel<<<1, 256, 0, stream>>>(qo_indptr, kv_indptr, kv_last_page_len, tile_start, tile_order, batch,
                                            wg_tok, causal, first_wave);
    bound = ((long long)batch + max_qo_rows / wg_tok) * Hkv;
  }
  if (num_blocks > 0 && bound > num_blocks) bound = num_blocks;
  if (bound > 0x7fffffffLL) bound = 0x7fffffffLL;
  if (bound < 1) bound = 1;
  if (decode_mode) {
    // wavefronts per (request, kv head) workgroup: with 2 (64 KB of LDS) two workgroups share a
    // CU, and one streams while the other starts or merges -- a few percent faster than 4 or 1.
    // A batch so small that its workgroups leave CUs empty (at most one per CU) runs with 4
    // wavefronts per workgroup instead: twice the loads in flight per request.
    auto launch = [&](auto waves_c) -> int {
      constexpr int kWaves = decltype(waves_c)::value;
      constexpr int kDecodeLds = kWaves * 32768;
      auto kern = attn_decode_kernel<GROUP, kWaves>;
      static bool attr_set = false;  // benign race: the call is idempotent
      if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kDecodeLds);
        if (e != hipSuccess) {
          set_error("attention: cannot reserve %d bytes of LDS: %s", kDecodeLds, hipGetErrorString(e));
          return NF_ERR_RUNTIME;
        }
        attr_set = true;
      }
      kern<<<(int)bound, kWaves * 64, kDecodeLds, stream>>>(q, o, qo_indptr, kv_data, kv_indptr, kv_indices,
                                                            kv_last_page_len, batch, Hq, Hkv, causal, scale_log2);
      return NF_OK;
    };
    int rc = (long long)batch * Hkv <= 256 ? launch(ic<4>{}) : launch(ic<2>{});
    if (rc) return rc;
  } else {
    auto kern = attn_prefill_kernel<GROUP, NQB_PREFILL, kPrefillStages, kPrefillMinWg>;
    static bool attr_set = false;  // benign race: the call is idempotent
    if (!attr_set) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, kPrefillStages * 16384);
      if (e != hipSuccess) {
        set_error("attention: cannot reserve %d bytes of LDS: %s", kPrefillStages * 16384, hipGetErrorString(e));
        return NF_ERR_RUNTIME;
      }
      attr_set = true;
    }
    kern<<<(int)bound, 256, kPrefillStages * 16384, stream>>>(
        q, o, qo_indptr, kv_data, kv_indptr, kv_indices, kv_last_page_len, tile_start, tile_order, batch, Hq,
        Hkv, causal, scale_log2);
  }
  return check_launch("nf_attention_paged_f16");
}

}  // namespace nf

using namespace nf;

extern "C" {

size_t nf_attention_workspace_bytes(int batch, int max_qo_rows, int num_qo_heads) {
  (void)num_qo_heads;
  if (batch < 0) batch = 0;
  if (max_qo_rows < 0) max_qo_rows = 0;
  // tile_start[batch + 1] (+ 1 of padding), then tile_order: a request has at most one tile that is
  // not full, and a full tile holds at least 8 tokens
  return (((size_t)batch + 2 + (size_t)batch + (size_t)max_qo_rows / 8 + 2) * sizeof(int32_t) + 255) & ~(size_t)255;
}

int nf_attention_paged_f16(const uint16_t* q, uint16_t* o, const int32_t* qo_indptr,
                           const uint16_t* kv_data, const int32_t* kv_indptr,
                           const int32_t* kv_indices, const int32_t* kv_last_page_len, int batch,
                           int max_qo_rows, int num_qo_heads, int num_kv_heads, int head_dim,
                           int page_size, int causal, int num_blocks, void* workspace,
                           size_t workspace_bytes, nf_stream_t stream) {
  NF_REQUIRE(head_dim == D && page_size == PAGE,
             "nf_attention_paged_f16: head_dim=%d page_size=%d, only 128/16 are built", head_dim,
             page_size);
  NF_REQUIRE(batch >= 0 && max_qo_rows >= 0 && num_qo_heads > 0 && num_kv_heads > 0 &&
                 num_qo_heads % num_kv_heads == 0,
             "nf_attention_paged_f16: bad sizes batch=%d rows=%d Hq=%d Hkv=%d", batch, max_qo_rows,
             num_qo_heads, num_kv_heads);
  if (batch == 0 || max_qo_rows == 0) return NF_OK;
  NF_REQUIRE(q && o && qo_indptr && kv_data && kv_indptr && kv_indices && kv_last_page_len,
             "nf_attention_paged_f16: null pointer");
  if (!workspace || workspace_bytes < nf_attention_workspace_bytes(batch, max_qo_rows, num_qo_heads)) {
    set_error("nf_attention_paged_f16: workspace of %zu bytes, need %zu", workspace_bytes,
              nf_attention_workspace_bytes(batch, max_qo_rows, num_qo_heads));
    return NF_ERR_WORKSPACE;
  }
  int32_t* tile_start = static_cast<int32_t*>(workspace);
  hipStream_t s = (hipStream_t)stream;
  const int group = num_qo_heads / num_kv_heads;
#define NF_ATTN_CASE(G)                                                                          \
  case G:                                                                                        \
    return launch_attn<G>(q, o, qo_indptr, kv_data, kv_indptr, kv_indices, kv_last_page_len,     \
                          tile_start, batch, max_qo_rows, num_qo_heads, num_kv_heads, causal,    \
                          num_blocks, s)
  switch (group) {
    NF_ATTN_CASE(1);
    NF_ATTN_CASE(2);
    NF_ATTN_CASE(4);
    NF_ATTN_CASE(8);
    default:
      set_error("nf_attention_paged_f16: GQA group %d not built (1, 2, 4, 8 are)", group);
      return NF_ERR_UNSUPPORTED;
  }
#undef NF_ATTN_CASE
}

}  // extern "C"
