// Row-wise HBM-bound operators of the nano-batch pipeline for gfx950:
// embedding gather, RMSNorm, last-token gather, greedy sampler, split+RoPE+paged-KV append.
// All use 16-byte vector accesses on rows that are multiples of 8 halves.
#include "common.h"

#include <cmath>
#include <cstring>

namespace nf {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

// ---------------------------------------------------------------- row gathers

// out[r,:] = src[row_of(r),:]; one workgroup per output row.
template <bool kKeepToken>
__global__ __launch_bounds__(256) void gather_rows_kernel(const int32_t* __restrict__ idx,
                                                          const u32x4* __restrict__ src,
                                                          u32x4* __restrict__ out, int vec_per_row) {
  const int r = blockIdx.x;
  const long long srow = kKeepToken ? (long long)idx[r + 1] - 1 : (long long)idx[r];
  const u32x4* s = src + srow * vec_per_row;
  u32x4* o = out + (long long)r * vec_per_row;
  for (int i = threadIdx.x; i < vec_per_row; i += blockDim.x) o[i] = s[i];
}

// ---------------------------------------------------------------- column slices, activation, transpose, sleep
// The smaller operators of the reference's vocabulary (pipeline/include/otherWrapper.cuh:183-301,
// 395-412): none of them is on the single-device schedules' path, all of them are one launch each.

// A row of up to three column ranges, copied apart: out_j[r, :] = in[r, first_j : first_j + n_j) in
// 16-byte chunks (first_0 = 0, first_1 = n_0, first_2 = n_0 + n_1); a null output skips its range.
// One workgroup per row.
__global__ __launch_bounds__(256) void split_columns_kernel(const u32x4* __restrict__ in, u32x4* __restrict__ o0,
                                                            u32x4* __restrict__ o1, u32x4* __restrict__ o2,
                                                            int in_vec_per_row, int v0, int v1, int v2) {
  const long long r = blockIdx.x;
  const u32x4* x = in + r * in_vec_per_row;
  for (int i = threadIdx.x; i < v0 + v1 + v2; i += 256) {
    if (i < v0) {
      if (o0) o0[r * v0 + i] = x[i];
    } else if (i < v0 + v1) {
      if (o1) o1[r * v1 + (i - v0)] = x[i];
    } else {
      if (o2) o2[r * v2 + (i - v0 - v1)] = x[i];
    }
  }
}

// out[r, c] = in[r, c] * silu(in[r, n + c]) for c < n: fp32 arithmetic, one rounding; the row's two
// halves in 16-byte chunks.  One workgroup per row.
__global__ __launch_bounds__(256) void silu_mul_kernel(const u32x4* __restrict__ in, u32x4* __restrict__ out,
                                                       int out_vec_per_row) {
  const long long r = blockIdx.x;
  const u32x4* x = in + r * 2 * out_vec_per_row;
  for (int i = threadIdx.x; i < out_vec_per_row; i += 256) {
    const u32x4 a = x[i], b = x[out_vec_per_row + i];
    const uint32_t pa[4] = {a.x, a.y, a.z, a.w}, pb[4] = {b.x, b.y, b.z, b.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint32_t h[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const float left = h2f_bits(e ? pa[j] >> 16 : pa[j] & 0xffffu);
        const float right = h2f_bits(e ? pb[j] >> 16 : pb[j] & 0xffffu);
        const float silu = right / (1.0f + expf(-right));
        h[e] = f2h_bits(left * silu);
      }
      o[j] = h[0] | (h[1] << 16);
    }
    out[r * out_vec_per_row + i] = u32x4{o[0], o[1], o[2], o[3]};
  }
}

// out[c, r] = in[r, c]: 64 x 64 tiles through LDS (one padding element per row), any rows / cols.
__global__ __launch_bounds__(256) void transpose_kernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out,
                                                        int rows, int cols) {
  __shared__ uint16_t tile[64][65];
  const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int y = ty; y < 64; y += 4)
    if (r0 + y < rows && c0 + tx < cols) tile[y][tx] = in[(long long)(r0 + y) * cols + c0 + tx];
  __syncthreads();
  for (int y = ty; y < 64; y += 4)
    if (c0 + y < cols && r0 + tx < rows) out[(long long)(c0 + y) * rows + r0 + tx] = tile[tx][y];
}

// One wavefront that leaves after `ticks` of the 100 MHz real-time counter.
__global__ void sleep_kernel(long long ticks) {
  const long long start = (long long)wall_clock64();
  while ((long long)wall_clock64() - start < ticks) __builtin_amdgcn_s_sleep(16);
}

// ---------------------------------------------------------------- RMSNorm

// One workgroup per row; fp32 math, single rounding on output.  Rows longer than 8192 are read a
// second time after the reduction (from L1/L2).
// kQuant: the rounded row (at most 4 x 256 chunks of 8 halves: hidden <= 8192) stays in registers
// and is also written as e4m3 bytes with one fp32 scale per row, exactly what the row quantiser
// makes of the fp16 output: the fp8-weight GEMM that follows needs no quantiser launch.
// kHeld: rows of at most 4 x 256 chunks (hidden <= 8192): a thread's chunks of the row and of the
// weight are loaded once, all of them before the first is used, and stay in registers -- the row is
// not read a second time after the reduction and the weight's latency passes under it.  The sums
// are taken in the same order either way, so both forms give the same bits.
template <bool kQuant, bool kHeld>
__global__ __launch_bounds__(256) void rmsnorm_kernel(u32x4* __restrict__ out,
                                                      const u32x4* __restrict__ in,
                                                      const u32x4* __restrict__ w, int vec_per_row,
                                                      float inv_n, float eps, uint8_t* __restrict__ q_out,
                                                      float* __restrict__ q_scale) {
  static_assert(!kQuant || kHeld, "the quantising form keeps the row in registers");
  __shared__ float s_part[4];
  __shared__ float s_max[4];
  const int r = blockIdx.x;
  const u32x4* x = in + (long long)r * vec_per_row;
  u32x4* y = out + (long long)r * vec_per_row;
  u32x4 xs[kHeld ? 4 : 1], ws[kHeld ? 4 : 1];
  if constexpr (kHeld) {
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if ((int)threadIdx.x + k * 256 < vec_per_row) xs[k] = x[threadIdx.x + k * 256];
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if ((int)threadIdx.x + k * 256 < vec_per_row) ws[k] = w[threadIdx.x + k * 256];
  }
  float ss = 0.f;
  auto square = [&](const u32x4& v) {
    const uint32_t p[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float a = h2f_bits(p[j] & 0xffffu), b = h2f_bits(p[j] >> 16);
      ss = fmaf(a, a, ss);
      ss = fmaf(b, b, ss);
    }
  };
  if constexpr (kHeld) {
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if ((int)threadIdx.x + k * 256 < vec_per_row) square(xs[k]);
  } else {
    for (int i = threadIdx.x; i < vec_per_row; i += 256) square(x[i]);
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float tot = s_part[0] + s_part[1] + s_part[2] + s_part[3];
  const float scale = 1.0f / sqrtf(tot * inv_n + eps);
  u32x4 held[kQuant ? 4 : 1];
  float amax = 0.f;
  auto normalise = [&](int i, const u32x4& v, const u32x4& g) {  // chunk i of the row: scaled, weighted, rounded once, stored
    const uint32_t p[4] = {v.x, v.y, v.z, v.w};
    const uint32_t q[4] = {g.x, g.y, g.z, g.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float a = h2f_bits(p[j] & 0xffffu) * scale * h2f_bits(q[j] & 0xffffu);
      float b = h2f_bits(p[j] >> 16) * scale * h2f_bits(q[j] >> 16);
      o[j] = f2h_bits(a) | (f2h_bits(b) << 16);
      if constexpr (kQuant) {
        amax = fmaxf(amax, fabsf(h2f_bits(o[j] & 0xffffu)));
        amax = fmaxf(amax, fabsf(h2f_bits(o[j] >> 16)));
      }
    }
    const u32x4 yv = u32x4{o[0], o[1], o[2], o[3]};
    y[i] = yv;
    return yv;
  };
  if constexpr (kHeld) {
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if ((int)threadIdx.x + k * 256 < vec_per_row) {
        const u32x4 yv = normalise(threadIdx.x + k * 256, xs[k], ws[k]);
        if constexpr (kQuant) held[k] = yv;
      }
  } else {
    for (int i = threadIdx.x; i < vec_per_row; i += 256) normalise(i, x[i], w[i]);
  }
  if constexpr (kQuant) {
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) amax = fmaxf(amax, __shfl_xor(amax, m, 64));
    if ((threadIdx.x & 63) == 0) s_max[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(s_max[0], s_max[1]), fmaxf(s_max[2], s_max[3]));
    const float s = amax > 0.f ? amax / 448.f : 1.f;
    if (threadIdx.x == 0) q_scale[r] = s;
    u32x2* dst = reinterpret_cast<u32x2*>(q_out + (size_t)r * vec_per_row * 8);
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if ((int)threadIdx.x + k * 256 < vec_per_row) dst[threadIdx.x + k * 256] = quantize_chunk_e4m3(held[k], s);
  }
}

// ---------------------------------------------------------------- greedy sampler

// Candidate order of the reference sampler: larger value wins; equal values: smaller key,
// key = bitreverse10(col mod 1024) << 20 | col.  Values <= -10000 (and NaN) never win.
struct ArgBest {
  float v;
  uint32_t key;
};
__device__ __forceinline__ bool arg_better(float v, uint32_t key, const ArgBest& b) {
  return v > b.v || (v == b.v && key < b.key);
}
__device__ __forceinline__ uint32_t arg_key(uint32_t col) {
  return ((__brev(col & 1023u) >> 22) << 20) | col;
}

__global__ __launch_bounds__(1024) void argmax_kernel(const uint16_t* __restrict__ logits,
                                                      uint16_t* __restrict__ max_vals,
                                                      int32_t* __restrict__ arg, int cols) {
  __shared__ float s_v[16];
  __shared__ uint32_t s_k[16];
  const int r = blockIdx.x;
  const uint16_t* x = logits + (long long)r * cols;
  ArgBest best{-10000.f, 0u};
  const int nvec = cols >> 3;
  const u32x4* xv = reinterpret_cast<const u32x4*>(x);
  for (int i = threadIdx.x; i < nvec; i += 1024) {
    u32x4 v = xv[i];
    const uint32_t p[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t c0 = (uint32_t)i * 8u + 2u * j;
      float a = h2f_bits(p[j] & 0xffffu), b = h2f_bits(p[j] >> 16);
      uint32_t ka = arg_key(c0), kb = arg_key(c0 + 1);
      if (a > -10000.f && arg_better(a, ka, best)) best = ArgBest{a, ka};
      if (b > -10000.f && arg_better(b, kb, best)) best = ArgBest{b, kb};
    }
  }
  for (int c = (nvec << 3) + threadIdx.x; c < cols; c += 1024) {
    float a = h2f_bits(x[c]);
    uint32_t ka = arg_key((uint32_t)c);
    if (a > -10000.f && arg_better(a, ka, best)) best = ArgBest{a, ka};
  }
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) {
    float ov = __shfl_xor(best.v, m, 64);
    uint32_t ok = __shfl_xor(best.key, m, 64);
    if (arg_better(ov, ok, best)) best = ArgBest{ov, ok};
  }
  if ((threadIdx.x & 63) == 0) {
    s_v[threadIdx.x >> 6] = best.v;
    s_k[threadIdx.x >> 6] = best.key;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    ArgBest b{s_v[0], s_k[0]};
    for (int i = 1; i < 16; ++i)
      if (arg_better(s_v[i], s_k[i], b)) b = ArgBest{s_v[i], s_k[i]};
    arg[r] = (int32_t)(b.key & 0xfffffu);
    if (max_vals) max_vals[r] = (uint16_t)f2h_bits(b.v);
  }
}

// ---------------------------------------------------------------- split + RoPE + paged append

// One workgroup per token.  The 64 rotation angles of the token (one per frequency) are
// evaluated once into LDS and shared by all heads.  A work item is (head, 8-feature chunk of
// the first half): it loads the chunk and its rotate-half partner (two 16-byte loads), and
// writes both rotated chunks.  V heads are copied.
__global__ __launch_bounds__(256) void rope_append_kernel(
    const uint16_t* __restrict__ kqv, uint16_t* __restrict__ q_out, uint16_t* __restrict__ kv_data,
    const int32_t* __restrict__ kv_indices, const int32_t* __restrict__ kv_indptr,
    const int32_t* __restrict__ rev_input_indptr, const int32_t* __restrict__ per_token_offset,
    int Hq, int Hkv, int page_size, float rope_rcp_scale, float rope_rcp_theta, float smooth_a,
    float smooth_b) {
  constexpr int D = 128;
  __shared__ float s_cos[D / 2], s_sin[D / 2];
  const int t = blockIdx.x;
  const int heads = Hq + 2 * Hkv;
  const uint16_t* row = kqv + (long long)t * heads * D;
  // the token's row first: a thread's first four items are in flight while the page is looked up
  // (three dependent loads) and the angles are evaluated
  constexpr int HELD = 4;
  u32x4 lo_held[HELD], hi_held[HELD];
#pragma unroll
  for (int k = 0; k < HELD; ++k) {
    const int item = threadIdx.x + k * 256;
    if (item < heads * 8) {
      const uint16_t* src = row + (item >> 3) * D + 8 * (item & 7);
      lo_held[k] = *reinterpret_cast<const u32x4*>(src);
      hi_held[k] = *reinterpret_cast<const u32x4*>(src + 64);
    }
  }
  const int r = rev_input_indptr[t];
  const int pos = per_token_offset[t];
  const int page = kv_indices[kv_indptr[r] + pos / page_size];
  const int entry = pos % page_size;
  if (threadIdx.x < D / 2) {
    float f = powf(rope_rcp_theta, (float)(2 * threadIdx.x) / (float)D);
    float smooth = f * smooth_a + smooth_b;
    smooth = fmaxf(0.0f, fminf(1.0f, smooth));
    f = (1.f - smooth) * (f * rope_rcp_scale) + smooth * f;
    float ang = (float)pos * f;
    s_cos[threadIdx.x] = cosf(ang);
    s_sin[threadIdx.x] = sinf(ang);
  }
  __syncthreads();
  // pool[page][kv][entry][head][feat]
  uint16_t* kdst = kv_data + ((((long long)page * 2 + 0) * page_size + entry) * Hkv) * D;
  uint16_t* vdst = kv_data + ((((long long)page * 2 + 1) * page_size + entry) * Hkv) * D;
  uint16_t* qdst = q_out + (long long)t * Hq * D;
  auto emit = [&](int item, const u32x4& lo, const u32x4& hi) {
    const int h = item >> 3, c = item & 7;  // chunk c covers features 8c..8c+7 and 64+8c..
    uint16_t* dst;
    if (h < Hkv) {
      dst = kdst + h * D;
    } else if (h < 2 * Hkv) {
      dst = vdst + (h - Hkv) * D;
      *reinterpret_cast<u32x4*>(dst + 8 * c) = lo;
      *reinterpret_cast<u32x4*>(dst + 64 + 8 * c) = hi;
      return;
    } else {
      dst = qdst + (h - 2 * Hkv) * D;
    }
    const uint32_t pl[4] = {lo.x, lo.y, lo.z, lo.w};
    const uint32_t ph[4] = {hi.x, hi.y, hi.z, hi.w};
    uint32_t ol[4], oh[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint32_t l16[2], h16[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int fi = 8 * c + 2 * j + e;
        const float cs = s_cos[fi], sn = s_sin[fi];
        const float a = h2f_bits(e ? pl[j] >> 16 : pl[j] & 0xffffu);
        const float b = h2f_bits(e ? ph[j] >> 16 : ph[j] & 0xffffu);
        l16[e] = f2h_bits(a * cs + (-b) * sn);  // i <  d/2: x[i]*cos - x[i+d/2]*sin
        h16[e] = f2h_bits(b * cs + a * sn);     // i >= d/2: x[i]*cos + x[i-d/2]*sin
      }
      ol[j] = l16[0] | (l16[1] << 16);
      oh[j] = h16[0] | (h16[1] << 16);
    }
    *reinterpret_cast<u32x4*>(dst + 8 * c) = u32x4{ol[0], ol[1], ol[2], ol[3]};
    *reinterpret_cast<u32x4*>(dst + 64 + 8 * c) = u32x4{oh[0], oh[1], oh[2], oh[3]};
  };
#pragma unroll
  for (int k = 0; k < HELD; ++k) {
    const int item = threadIdx.x + k * 256;
    if (item < heads * 8) emit(item, lo_held[k], hi_held[k]);
  }
  for (int item = threadIdx.x + HELD * 256; item < heads * 8; item += 256) {  // more than 128 heads
    const uint16_t* src = row + (item >> 3) * D + 8 * (item & 7);
    emit(item, *reinterpret_cast<const u32x4*>(src), *reinterpret_cast<const u32x4*>(src + 64));
  }
}

// Pages of the listed requests between a layer's pool and a staging buffer indexed like
// kv_indices: staging page j <-> pool page kv_indices[j] for j in [kv_indptr[r], kv_indptr[r+1])
// of every listed request r.  grid.y walks the requests, grid.x strides over a request's pages;
// a workgroup moves one page (K and V: page_chunks 16-byte chunks) at a time.
template <bool kToPool>
__global__ __launch_bounds__(256) void move_kv_pages_kernel(const int32_t* __restrict__ req_idx,
                                                            const int32_t* __restrict__ kv_indptr,
                                                            const int32_t* __restrict__ kv_indices,
                                                            u32x4* staging, u32x4* pool, int page_chunks) {
  const int r = req_idx[blockIdx.y];
  const int begin = kv_indptr[r], end = kv_indptr[r + 1];
  for (int j = begin + blockIdx.x; j < end; j += gridDim.x) {
    u32x4* s = staging + (size_t)j * page_chunks;
    u32x4* p = pool + (size_t)kv_indices[j] * page_chunks;
    for (int c = threadIdx.x; c < page_chunks; c += 256) {
      if constexpr (kToPool) p[c] = s[c];
      else s[c] = p[c];
    }
  }
}

}  // namespace nf

using namespace nf;

extern "C" {

int nf_abi_version(void) { return 1; }
const char* nf_last_error(void) { return nf::g_err; }

int nf_embedding_f16(const int32_t* tokens, const uint16_t* table, uint16_t* out, int n_tokens,
                     int hidden, nf_stream_t stream) {
  NF_REQUIRE(n_tokens >= 0 && hidden > 0 && hidden % 8 == 0,
             "nf_embedding_f16: hidden=%d must be a positive multiple of 8 (n_tokens=%d)", hidden,
             n_tokens);
  if (n_tokens == 0) return NF_OK;
  NF_REQUIRE(tokens && table && out, "nf_embedding_f16: null pointer");
  gather_rows_kernel<false><<<n_tokens, 256, 0, (hipStream_t)stream>>>(
      tokens, reinterpret_cast<const u32x4*>(table), reinterpret_cast<u32x4*>(out), hidden / 8);
  return check_launch("nf_embedding_f16");
}

int nf_keep_token_f16(const uint16_t* in, uint16_t* out, const int32_t* input_indptr, int req_num,
                      int hidden, nf_stream_t stream) {
  NF_REQUIRE(req_num >= 0 && hidden > 0 && hidden % 8 == 0,
             "nf_keep_token_f16: hidden=%d must be a positive multiple of 8 (req_num=%d)", hidden,
             req_num);
  if (req_num == 0) return NF_OK;
  NF_REQUIRE(in && out && input_indptr, "nf_keep_token_f16: null pointer");
  gather_rows_kernel<true><<<req_num, 256, 0, (hipStream_t)stream>>>(
      input_indptr, reinterpret_cast<const u32x4*>(in), reinterpret_cast<u32x4*>(out), hidden / 8);
  return check_launch("nf_keep_token_f16");
}

int nf_split_kqv_f16(const uint16_t* kqv, uint16_t* k, uint16_t* q, uint16_t* v, int rows, int k_dim, int q_dim,
                     int v_dim, nf_stream_t stream) {
  NF_REQUIRE(rows >= 0 && k_dim >= 0 && q_dim >= 0 && v_dim >= 0 && k_dim + q_dim + v_dim > 0 &&
                 k_dim % 8 == 0 && q_dim % 8 == 0 && v_dim % 8 == 0,
             "nf_split_kqv_f16: widths %d | %d | %d must be non-negative multiples of 8 (rows=%d)", k_dim, q_dim, v_dim,
             rows);
  if (rows == 0) return NF_OK;
  NF_REQUIRE(kqv && (k || !k_dim) && (q || !q_dim) && (v || !v_dim), "nf_split_kqv_f16: null pointer");
  NF_REQUIRE(((uintptr_t)kqv | (uintptr_t)k | (uintptr_t)q | (uintptr_t)v) % 16 == 0,
             "nf_split_kqv_f16: buffers must be 16-byte aligned");
  split_columns_kernel<<<rows, 256, 0, (hipStream_t)stream>>>(
      reinterpret_cast<const u32x4*>(kqv), reinterpret_cast<u32x4*>(k), reinterpret_cast<u32x4*>(q),
      reinterpret_cast<u32x4*>(v), (k_dim + q_dim + v_dim) / 8, k_dim / 8, q_dim / 8, v_dim / 8);
  return check_launch("nf_split_kqv_f16");
}

int nf_extract_rank_columns_f16(const uint16_t* in, uint16_t* out, int rows, int cols, int nranks, int rank,
                                nf_stream_t stream) {
  NF_REQUIRE(rows >= 0 && cols > 0 && cols % 8 == 0 && nranks > 0 && rank >= 0 && rank < nranks,
             "nf_extract_rank_columns_f16: cols=%d must be a positive multiple of 8, rank %d of %d (rows=%d)", cols, rank,
             nranks, rows);
  if (rows == 0) return NF_OK;
  NF_REQUIRE(in && out, "nf_extract_rank_columns_f16: null pointer");
  NF_REQUIRE(((uintptr_t)in | (uintptr_t)out) % 16 == 0, "nf_extract_rank_columns_f16: buffers must be 16-byte aligned");
  // the rank's range as the first of the row's "three": the row pointer is moved to its first column
  split_columns_kernel<<<rows, 256, 0, (hipStream_t)stream>>>(
      reinterpret_cast<const u32x4*>(in + (size_t)rank * cols), reinterpret_cast<u32x4*>(out), nullptr, nullptr,
      nranks * (cols / 8), cols / 8, 0, 0);
  return check_launch("nf_extract_rank_columns_f16");
}

int nf_silu_mul_f16(const uint16_t* in, uint16_t* out, int rows, int cols, nf_stream_t stream) {
  NF_REQUIRE(rows >= 0 && cols > 0 && cols % 8 == 0, "nf_silu_mul_f16: cols=%d must be a positive multiple of 8 (rows=%d)",
             cols, rows);
  if (rows == 0) return NF_OK;
  NF_REQUIRE(in && out, "nf_silu_mul_f16: null pointer");
  NF_REQUIRE(((uintptr_t)in | (uintptr_t)out) % 16 == 0, "nf_silu_mul_f16: buffers must be 16-byte aligned");
  silu_mul_kernel<<<rows, 256, 0, (hipStream_t)stream>>>(reinterpret_cast<const u32x4*>(in),
                                                         reinterpret_cast<u32x4*>(out), cols / 8);
  return check_launch("nf_silu_mul_f16");
}

int nf_transpose_f16(const uint16_t* in, uint16_t* out, int rows, int cols, nf_stream_t stream) {
  NF_REQUIRE(rows >= 0 && cols >= 0, "nf_transpose_f16: bad shape %d x %d", rows, cols);
  if (rows == 0 || cols == 0) return NF_OK;
  NF_REQUIRE(in && out && in != out, "nf_transpose_f16: null pointer, or in place");
  NF_REQUIRE((rows + 63) / 64 <= 65535, "nf_transpose_f16: %d rows exceed the grid", rows);
  transpose_kernel<<<dim3((cols + 63) / 64, (rows + 63) / 64), 256, 0, (hipStream_t)stream>>>(in, out, rows, cols);
  return check_launch("nf_transpose_f16");
}

int nf_sleep_us(int us, nf_stream_t stream) {
  NF_REQUIRE(us >= 0 && us <= 1000000, "nf_sleep_us: %d us not in [0, 1 s]", us);
  if (us == 0) return NF_OK;
  sleep_kernel<<<1, 64, 0, (hipStream_t)stream>>>((long long)us * 100);
  return check_launch("nf_sleep_us");
}

int nf_move_kv_pages(int req_num, const int32_t* req_idx, const int32_t* kv_indptr, const int32_t* kv_indices,
                     uint16_t* staging, uint16_t* kv_data, size_t page_bytes, int to_pool, nf_stream_t stream) {
  NF_REQUIRE(req_num >= 0 && page_bytes > 0 && page_bytes % 16 == 0 && page_bytes < ((size_t)1 << 31),
             "nf_move_kv_pages: page_bytes=%zu must be a positive multiple of 16 (req_num=%d)", page_bytes, req_num);
  if (req_num == 0) return NF_OK;
  NF_REQUIRE(req_num <= 65535, "nf_move_kv_pages: at most 65535 requests per call (%d)", req_num);
  NF_REQUIRE(req_idx && kv_indptr && kv_indices && staging && kv_data, "nf_move_kv_pages: null pointer");
  NF_REQUIRE(((uintptr_t)staging | (uintptr_t)kv_data) % 16 == 0, "nf_move_kv_pages: buffers must be 16-byte aligned");
  // 64 workgroups per request stride over its pages (a 1024-token request has 64 of them)
  const dim3 grid(64, (unsigned)req_num);
  const int chunks = (int)(page_bytes / 16);
  if (to_pool)
    move_kv_pages_kernel<true><<<grid, 256, 0, (hipStream_t)stream>>>(
        req_idx, kv_indptr, kv_indices, reinterpret_cast<u32x4*>(staging), reinterpret_cast<u32x4*>(kv_data), chunks);
  else
    move_kv_pages_kernel<false><<<grid, 256, 0, (hipStream_t)stream>>>(
        req_idx, kv_indptr, kv_indices, reinterpret_cast<u32x4*>(staging), reinterpret_cast<u32x4*>(kv_data), chunks);
  return check_launch("nf_move_kv_pages");
}

int nf_rmsnorm_f16(uint16_t* out, const uint16_t* in, const uint16_t* weight, int rows, int hidden,
                   float eps, nf_stream_t stream) {
  NF_REQUIRE(rows >= 0 && hidden > 0 && hidden % 8 == 0,
             "nf_rmsnorm_f16: hidden=%d must be a positive multiple of 8 (rows=%d)", hidden, rows);
  if (rows == 0) return NF_OK;
  NF_REQUIRE(out && in && weight, "nf_rmsnorm_f16: null pointer");
  auto kern = hidden <= 8192 ? rmsnorm_kernel<false, true> : rmsnorm_kernel<false, false>;
  kern<<<rows, 256, 0, (hipStream_t)stream>>>(
      reinterpret_cast<u32x4*>(out), reinterpret_cast<const u32x4*>(in),
      reinterpret_cast<const u32x4*>(weight), hidden / 8, 1.0f / (float)hidden, eps, nullptr, nullptr);
  return check_launch("nf_rmsnorm_f16");
}

int nf_rmsnorm_quantize_e4m3(uint16_t* out, const uint16_t* in, const uint16_t* weight, uint8_t* out_q,
                             float* row_scale, int rows, int hidden, float eps, nf_stream_t stream) {
  NF_REQUIRE(rows >= 0 && hidden > 0 && hidden % 16 == 0 && hidden <= 8192,
             "nf_rmsnorm_quantize_e4m3: hidden=%d must be a positive multiple of 16, at most 8192 (rows=%d)", hidden,
             rows);
  if (rows == 0) return NF_OK;
  NF_REQUIRE(out && in && weight && out_q && row_scale, "nf_rmsnorm_quantize_e4m3: null pointer");
  NF_REQUIRE(((uintptr_t)out | (uintptr_t)in | (uintptr_t)weight | (uintptr_t)out_q) % 16 == 0,
             "nf_rmsnorm_quantize_e4m3: operands must be 16-byte aligned");
  rmsnorm_kernel<true, true><<<rows, 256, 0, (hipStream_t)stream>>>(
      reinterpret_cast<u32x4*>(out), reinterpret_cast<const u32x4*>(in),
      reinterpret_cast<const u32x4*>(weight), hidden / 8, 1.0f / (float)hidden, eps, out_q, row_scale);
  return check_launch("nf_rmsnorm_quantize_e4m3");
}

int nf_argmax_f16(const uint16_t* logits, uint16_t* max_vals, int32_t* argmax, int rows, int cols,
                  nf_stream_t stream) {
  NF_REQUIRE(rows >= 0 && cols > 0 && cols < (1 << 20) && cols % 8 == 0,
             "nf_argmax_f16: cols=%d must be a multiple of 8 below 2^20 (rows=%d)", cols, rows);
  if (rows == 0) return NF_OK;
  NF_REQUIRE(logits && argmax, "nf_argmax_f16: null pointer");
  argmax_kernel<<<rows, 1024, 0, (hipStream_t)stream>>>(logits, max_vals, argmax, cols);
  return check_launch("nf_argmax_f16");
}

int nf_rope_append_f16(const uint16_t* kqv, uint16_t* q_out, uint16_t* kv_data,
                       const int32_t* kv_indices, const int32_t* kv_indptr,
                       const int32_t* rev_input_indptr, const int32_t* per_token_offset,
                       int n_tokens, int num_qo_heads, int num_kv_heads, int head_dim,
                       int page_size, float rope_scale, float rope_theta, float smooth_a,
                       float smooth_b, nf_stream_t stream) {
  NF_REQUIRE(head_dim == 128, "nf_rope_append_f16: head_dim=%d, only 128 is built", head_dim);
  NF_REQUIRE(n_tokens >= 0 && num_qo_heads > 0 && num_kv_heads > 0 && page_size > 0,
             "nf_rope_append_f16: bad sizes tokens=%d Hq=%d Hkv=%d page=%d", n_tokens, num_qo_heads,
             num_kv_heads, page_size);
  NF_REQUIRE(rope_scale > 0.f && rope_theta > 0.f, "nf_rope_append_f16: rope_scale/theta must be > 0");
  if (n_tokens == 0) return NF_OK;
  NF_REQUIRE(kqv && q_out && kv_data && kv_indices && kv_indptr && rev_input_indptr &&
                 per_token_offset,
             "nf_rope_append_f16: null pointer");
  rope_append_kernel<<<n_tokens, 256, 0, (hipStream_t)stream>>>(
      kqv, q_out, kv_data, kv_indices, kv_indptr, rev_input_indptr, per_token_offset, num_qo_heads,
      num_kv_heads, page_size, 1.0f / rope_scale, 1.0f / rope_theta, smooth_a, smooth_b);
  return check_launch("nf_rope_append_f16");
}

}  // extern "C"
