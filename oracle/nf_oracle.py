"""ctypes/numpy binding of the CPU oracle (oracle/nf_oracle.c).

TEST INFRASTRUCTURE ONLY.  Imported by tests/, by the smoke check and by the
benchmark's cpu_baseline leg; the shipped package never imports it.

All tensors are numpy arrays; fp16 tensors are ``np.float16`` (viewed as uint16
bit patterns on the C side).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libnf_oracle.so")


def build(force: bool = False) -> str:
    """Compile the oracle with the Makefile next to this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-s", "-C", _HERE] + (["-B"] if force else []))
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


_u16p = C.POINTER(C.c_uint16)
_i32p = C.POINTER(C.c_int32)
_f32p = C.POINTER(C.c_float)
_u8p = C.POINTER(C.c_uint8)


def _h(a):
    """fp16 array -> uint16 pointer (None passes NULL)."""
    if a is None:
        return None
    assert a.dtype == np.float16 and a.flags["C_CONTIGUOUS"], (a.dtype, a.flags)
    return a.ctypes.data_as(_u16p)


def _i(a):
    if a is None:
        return None
    assert a.dtype == np.int32 and a.flags["C_CONTIGUOUS"], (a.dtype, a.flags)
    return a.ctypes.data_as(_i32p)


class NfoModel(C.Structure):
    _fields_ = [
        ("hidden", C.c_int), ("Hq", C.c_int), ("Hkv", C.c_int), ("d", C.c_int),
        ("ffn", C.c_int), ("vocab", C.c_int), ("layers", C.c_int), ("page_size", C.c_int),
        ("eps", C.c_float), ("rope_theta", C.c_float), ("rope_scale", C.c_float),
        ("smooth_a", C.c_float), ("smooth_b", C.c_float),
        ("embedding", _u16p), ("lm_head", _u16p), ("model_norm", _u16p),
        ("w_kqv", C.POINTER(_u16p)), ("w_o", C.POINTER(_u16p)), ("w_gate", C.POINTER(_u16p)),
        ("w_up", C.POINTER(_u16p)), ("w_down", C.POINTER(_u16p)), ("ln_attn", C.POINTER(_u16p)),
        ("ln_ffn", C.POINTER(_u16p)), ("kv_data", C.POINTER(_u16p)), ("b_kqv", C.POINTER(_u16p)),
    ]


class NfoBatch(C.Structure):
    _fields_ = [
        ("decodePrefillBorder", C.c_int), ("prefillNum", C.c_int), ("prefillTokensNum", C.c_int),
        ("input_tokens", _i32p), ("input_indptr", _i32p), ("rev_input_indptr", _i32p),
        ("per_token_offset", _i32p), ("kv_indptr", _i32p), ("kv_indices", _i32p),
        ("kv_last_page_len", _i32p),
    ]


def _declare(l):
    l.nfo_num_threads.restype = C.c_int
    l.nfo_half_to_float.restype = C.c_float
    l.nfo_half_to_float.argtypes = [C.c_uint16]
    l.nfo_float_to_half.restype = C.c_uint16
    l.nfo_float_to_half.argtypes = [C.c_float]
    l.nfo_e4m3_to_float.restype = C.c_float
    l.nfo_e4m3_to_float.argtypes = [C.c_uint8]
    l.nfo_gemm_f16.restype = None
    l.nfo_gemm_f16.argtypes = [_u16p, _u16p, _u16p, _u16p, C.c_int, C.c_int, C.c_int, C.c_float,
                               C.c_float, C.c_int]
    l.nfo_dual_swiglu_f16.restype = None
    l.nfo_dual_swiglu_f16.argtypes = [_u16p, _u16p, _u16p, _u16p, _u16p, _u16p, C.c_int, C.c_int,
                                      C.c_int]
    l.nfo_float_to_e4m3.restype = C.c_uint8
    l.nfo_float_to_e4m3.argtypes = [C.c_float]
    l.nfo_quantize_rows_e4m3.restype = None
    l.nfo_quantize_rows_e4m3.argtypes = [_u16p, _u8p, _f32p, C.c_int, C.c_int]
    l.nfo_silu_mul_f16.restype = None
    l.nfo_silu_mul_f16.argtypes = [_u16p, _u16p, _u16p, C.c_size_t]
    l.nfo_gemm_f8f8_f16.restype = None
    l.nfo_gemm_f8f8_f16.argtypes = [_u8p, _f32p, _u8p, _f32p, _u16p, _u16p, C.c_int, C.c_int, C.c_int,
                                    C.c_float, C.c_float]
    l.nfo_gemm_f8w_f16.restype = None
    l.nfo_gemm_f8w_f16.argtypes = [_u16p, _u8p, _f32p, _u16p, _u16p, C.c_int, C.c_int, C.c_int,
                                   C.c_float, C.c_float]
    l.nfo_rmsnorm_f16.restype = None
    l.nfo_rmsnorm_f16.argtypes = [_u16p, _u16p, _u16p, C.c_int, C.c_int, C.c_float]
    l.nfo_embedding_f16.restype = None
    l.nfo_embedding_f16.argtypes = [_i32p, _u16p, _u16p, C.c_int, C.c_int]
    l.nfo_keep_token_f16.restype = None
    l.nfo_keep_token_f16.argtypes = [_u16p, _u16p, _i32p, C.c_int, C.c_int]
    l.nfo_argmax_f16.restype = None
    l.nfo_argmax_f16.argtypes = [_u16p, _u16p, _i32p, C.c_int, C.c_int]
    l.nfo_kv_offset.restype = C.c_int64
    l.nfo_kv_offset.argtypes = [C.c_int] * 8
    l.nfo_rope_freq.restype = C.c_float
    l.nfo_rope_freq.argtypes = [C.c_int, C.c_int, C.c_float, C.c_float, C.c_float, C.c_float]
    l.nfo_ref_llama_rope.restype = None
    l.nfo_ref_llama_rope.argtypes = [_u16p, _f32p, C.c_int, C.c_int, C.c_float, C.c_float]
    l.nfo_rope_append_f16.restype = None
    l.nfo_rope_append_f16.argtypes = [_u16p, _u16p, _u16p, _i32p, _i32p, _i32p, _i32p, C.c_int,
                                      C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float,
                                      C.c_float, C.c_float, _i32p, _i32p]
    l.nfo_attention_paged_f16.restype = None
    l.nfo_attention_paged_f16.argtypes = [_u16p, _u16p, _i32p, _u16p, _i32p, _i32p, _i32p, C.c_int,
                                          C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
    l.nfo_decoder_forward.restype = None
    l.nfo_decoder_forward.argtypes = [C.POINTER(NfoModel), C.POINTER(NfoBatch), _u16p, _u16p, _u16p,
                                      _i32p]


# ------------------------------------------------------------------ operators


def num_threads() -> int:
    return lib().nfo_num_threads()


def gemm(A, B, Cmat=None, alpha=1.0, beta=0.0, b_col_major=False):
    M, K = A.shape
    N = B.shape[0] if b_col_major else B.shape[1]
    assert (B.shape == (N, K)) if b_col_major else (B.shape == (K, N))
    D = np.empty((M, N), np.float16)
    lib().nfo_gemm_f16(_h(A), _h(B), _h(Cmat), _h(D), M, N, K, alpha, beta, int(b_col_major))
    return D


def dual_swiglu(A, Bg, Bu, return_parts=False):
    M, K = A.shape
    N = Bg.shape[1]
    assert Bg.shape == (K, N) and Bu.shape == (K, N)
    out = np.empty((M, N), np.float16)
    d0 = np.empty((M, N), np.float16) if return_parts else None
    d1 = np.empty((M, N), np.float16) if return_parts else None
    lib().nfo_dual_swiglu_f16(_h(A), _h(Bg), _h(Bu), _h(out), _h(d0), _h(d1), M, N, K)
    return (out, d0, d1) if return_parts else out


# ---- bfloat16 variants of the two GEMM operators.  The reference has no bf16 path (its GEMM
# wrappers are half only, pipeline/include/cutlassGemmWrapperImpl.cuh:24-27): PARITY UNPINNED
# against the reference; these are the closed forms D = bf16(alpha*A.B + beta*C) and
# bf16(silu(bf16(A.Bg)) * bf16(A.Bu)) in float64, on uint16 bit patterns.
def bf16_to_float(bits: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def float_to_bf16(x: np.ndarray) -> np.ndarray:
    """Round to nearest, ties to even, on the fp32 bit pattern (finite inputs)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return u.astype(np.uint16)


def gemm_bf16(A, B, Cmat=None, alpha=1.0, beta=0.0, b_col_major=False):
    a = bf16_to_float(A).astype(np.float64)
    b = bf16_to_float(B).astype(np.float64)
    d = alpha * (a @ (b.T if b_col_major else b))
    if Cmat is not None and beta != 0.0:
        d = d + beta * bf16_to_float(Cmat).astype(np.float64)
    return float_to_bf16(d.astype(np.float32))


def dual_swiglu_bf16(A, Bg, Bu):
    a = bf16_to_float(A).astype(np.float64)
    g = bf16_to_float(float_to_bf16((a @ bf16_to_float(Bg).astype(np.float64)).astype(np.float32))).astype(np.float64)
    u = bf16_to_float(float_to_bf16((a @ bf16_to_float(Bu).astype(np.float64)).astype(np.float32))).astype(np.float64)
    return float_to_bf16((g / (1.0 + np.exp(-g)) * u).astype(np.float32))


def gemm_f8w(A, Bq, scale, Cmat=None, alpha=1.0, beta=0.0):
    M, K = A.shape
    N = Bq.shape[1]
    assert Bq.dtype == np.uint8 and Bq.shape == (K, N) and scale.dtype == np.float32
    D = np.empty((M, N), np.float16)
    lib().nfo_gemm_f8w_f16(_h(A), Bq.ctypes.data_as(_u8p), scale.ctypes.data_as(_f32p), _h(Cmat),
                           _h(D), M, N, K, alpha, beta)
    return D


def e4m3_to_float(v: int) -> float:
    return lib().nfo_e4m3_to_float(v)


def float_to_e4m3(x: float) -> int:
    return int(lib().nfo_float_to_e4m3(float(x)))


def quantize_rows_e4m3(X):
    """X fp16 [M,K] -> (Xq uint8 [M,K], scale fp32 [M])."""
    M, K = X.shape
    Xq = np.empty((M, K), np.uint8)
    scale = np.empty((M,), np.float32)
    lib().nfo_quantize_rows_e4m3(_h(X), Xq.ctypes.data_as(_u8p), scale.ctypes.data_as(_f32p), M, K)
    return Xq, scale


def gemm_f8f8(Aq, sa, Bq_nk, sb, Cmat=None, alpha=1.0, beta=0.0):
    """Aq uint8 [M,K], Bq_nk uint8 [N,K] (one row per output channel), fp32 scales."""
    M, K = Aq.shape
    N = Bq_nk.shape[0]
    assert Aq.dtype == np.uint8 and Bq_nk.dtype == np.uint8 and Bq_nk.shape == (N, K)
    Aq, Bq_nk = np.ascontiguousarray(Aq), np.ascontiguousarray(Bq_nk)
    sa, sb = np.ascontiguousarray(sa, np.float32), np.ascontiguousarray(sb, np.float32)
    D = np.empty((M, N), np.float16)
    lib().nfo_gemm_f8f8_f16(Aq.ctypes.data_as(_u8p), sa.ctypes.data_as(_f32p), Bq_nk.ctypes.data_as(_u8p),
                            sb.ctypes.data_as(_f32p), _h(Cmat), _h(D), M, N, K, alpha, beta)
    return D


def silu_mul(g16, u16):
    """half(silu(g) * u) elementwise on fp16 arrays (the tail of the dual epilogue)."""
    g16, u16 = np.ascontiguousarray(g16, np.float16), np.ascontiguousarray(u16, np.float16)
    out = np.empty(g16.shape, np.float16)
    lib().nfo_silu_mul_f16(_h(g16), _h(u16), _h(out), g16.size)
    return out


def activation_silu_mul(x):
    """[M, 2N] -> [M, N]: x[:, :N] * silu(x[:, N:]) -- SiLU of the RIGHT half times the left half, fp32
    arithmetic, one rounding (silu_and_multiply_kernel, pipeline/src/small_cuda_operator.cu:100-120)."""
    N = x.shape[1] // 2
    return silu_mul(np.ascontiguousarray(x[:, N:]), np.ascontiguousarray(x[:, :N]))


def split_kqv(kqv, k_dim, q_dim, v_dim):
    """Rows of [k | q | v] copied apart, in that column order (splitKQVOutputKernel,
    pipeline/src/small_cuda_operator.cu:27-52)."""
    assert kqv.shape[1] == k_dim + q_dim + v_dim
    return (np.ascontiguousarray(kqv[:, :k_dim]), np.ascontiguousarray(kqv[:, k_dim:k_dim + q_dim]),
            np.ascontiguousarray(kqv[:, k_dim + q_dim:]))


def extract_rank_columns(x, nranks, rank):
    """[M, nranks * N] -> the rank's [M, N] (extractRankSubmatrixHalf, pipeline/src/small_cuda_operator.cu:133-151)."""
    N = x.shape[1] // nranks
    return np.ascontiguousarray(x[:, rank * N:(rank + 1) * N])


def transpose(x):
    """[rows, cols] -> [cols, rows] (transposeKernel, pipeline/src/small_cuda_operator.cu:64-83)."""
    return np.ascontiguousarray(x.T)


def quantize_weight_e4m3(W):
    """W fp16 [K,N] (the pipeline's weight orientation) -> (Wq uint8 [N,K], scale fp32 [N]): per
    output channel, scale = max|w| / 448, q = e4m3(w / scale) -- the row quantiser on the transpose."""
    return quantize_rows_e4m3(np.ascontiguousarray(W.T))


def dual_swiglu_f8f8(Aq, sa, Gq_nk, sg, Uq_nk, su):
    """The gate/up pair on fp8 operands: both products rounded to fp16, then half(silu(g) * u)."""
    return silu_mul(gemm_f8f8(Aq, sa, Gq_nk, sg), gemm_f8f8(Aq, sa, Uq_nk, su))


FP8_LAYER_WEIGHTS = ("w_kqv", "w_o", "w_gate", "w_up", "w_down")


def quantize_model_weights(weights: dict) -> dict:
    """Per-layer lists of (Wq [N,K], scale [N]) for the five GEMM weights of every layer."""
    return {k: [quantize_weight_e4m3(w) for w in weights[k]] for k in FP8_LAYER_WEIGHTS}


def decoder_forward_f8(cfg: dict, weights: dict, wq: dict, kv_data: list, batch: dict, activations="e4m3",
                       want_logits=False):
    """decoder_forward with the five per-layer GEMM weights in e4m3 (wq = quantize_model_weights);
    embedding, norms and the LM head stay fp16.  No reference implementation exists for this
    variant: parity unpinned.  activations:
      "e4m3": every fp8 GEMM quantises its input rows first (per-row scale) and multiplies
              fp8 x fp8 -- the arithmetic the device kernels do;
      "f16":  fp16 activations against dequantised weights -- the definition the 3e-2 fp8
              tolerance is stated against.
    The op order is nfo_decoder_forward's; kv_data is appended in place.  Returns
    (hidden, logits or None, sampled)."""
    assert activations in ("e4m3", "f16")
    L, Hq, Hkv, d, P = cfg["layers"], cfg["Hq"], cfg["Hkv"], cfg["d"], cfg["page_size"]
    eps = float(cfg.get("eps", 1e-5))
    b = {k: (None if batch.get(k) is None else np.ascontiguousarray(batch[k], np.int32)) for k in
         ("input_tokens", "input_indptr", "rev_input_indptr", "per_token_offset", "kv_indptr", "kv_indices",
          "kv_last_page_len")}
    nd, npre = int(batch["decodePrefillBorder"]), int(batch["prefillNum"])
    req = nd + npre

    def mm(x, key, l, Cmat=None, beta=0.0):
        q, s = wq[key][l]
        if activations == "e4m3":
            xq, xs = quantize_rows_e4m3(x)
            return gemm_f8f8(xq, xs, q, s, Cmat, 1.0, beta)
        return gemm_f8w(x, np.ascontiguousarray(q.T), s, Cmat, 1.0, beta)

    x = embedding(b["input_tokens"], weights["embedding"])
    T = x.shape[0]
    for l in range(L):
        xn = rmsnorm(x, weights["ln_attn"][l], eps)
        kqv = mm(xn, "w_kqv", l)
        qb = rope_append(kqv, kv_data[l], b["kv_indices"], b["kv_indptr"], b["rev_input_indptr"],
                         b["per_token_offset"], Hq, Hkv, d, P, float(cfg.get("rope_scale", 1.0)),
                         float(cfg.get("rope_theta", 1e4)), float(cfg.get("smooth_a", 0.0)),
                         float(cfg.get("smooth_b", 0.0)))
        ao = np.zeros((T, Hq * d), np.float16)
        if nd:
            attention_paged(qb, np.ascontiguousarray(b["input_indptr"][:nd + 1]), kv_data[l],
                            np.ascontiguousarray(b["kv_indptr"][:nd + 1]), b["kv_indices"],
                            np.ascontiguousarray(b["kv_last_page_len"][:nd]), Hq, Hkv, d, P, causal=False, out=ao)
        if npre:
            attention_paged(qb, np.ascontiguousarray(b["input_indptr"][nd:]), kv_data[l],
                            np.ascontiguousarray(b["kv_indptr"][nd:]), b["kv_indices"],
                            np.ascontiguousarray(b["kv_last_page_len"][nd:]), Hq, Hkv, d, P, causal=True, out=ao)
        xo = mm(ao, "w_o", l, x, 1.0)
        xn = rmsnorm(xo, weights["ln_ffn"][l], eps)
        act = silu_mul(mm(xn, "w_gate", l), mm(xn, "w_up", l))
        x = mm(act, "w_down", l, xo, 1.0)
    kept = keep_token(x, b["input_indptr"], req)
    logits = gemm(rmsnorm(kept, weights["model_norm"], eps), weights["lm_head"])
    sampled = argmax(logits)[0]
    return x, (logits if want_logits else None), sampled


def move_kv_pages(req_idx, kv_indptr, kv_indices, staging, kv_data, to_pool: bool):
    """Pages of the listed requests between a layer's pool [pages, ...] and a staging buffer indexed
    like kv_indices, IN PLACE (pipeline/src/offloadKernel.cu:17-34: for each listed request, for j in
    [kv_indptr[r], kv_indptr[r+1]): host page j <-> pool page kv_indices[j]).  Plain loops."""
    for r in np.asarray(req_idx).tolist():
        for j in range(int(kv_indptr[r]), int(kv_indptr[r + 1])):
            if to_pool:
                kv_data[int(kv_indices[j])] = staging[j]
            else:
                staging[j] = kv_data[int(kv_indices[j])]


def rmsnorm(x, w, eps=1e-5):
    rows, H = x.shape
    out = np.empty_like(x)
    lib().nfo_rmsnorm_f16(_h(out), _h(x), _h(w), rows, H, eps)
    return out


def embedding(tokens, table):
    T = tokens.shape[0]
    H = table.shape[1]
    out = np.empty((T, H), np.float16)
    lib().nfo_embedding_f16(_i(tokens), _h(table), _h(out), T, H)
    return out


def keep_token(x, input_indptr, req_num):
    H = x.shape[1]
    out = np.empty((req_num, H), np.float16)
    lib().nfo_keep_token_f16(_h(x), _h(out), _i(input_indptr), req_num, H)
    return out


def argmax(logits):
    rows, cols = logits.shape
    mv = np.empty((rows,), np.float16)
    arg = np.empty((rows,), np.int32)
    lib().nfo_argmax_f16(_h(logits), _h(mv), _i(arg), rows, cols)
    return arg, mv


def kv_offset(page, kv, entry, head, feat, page_size, Hkv, d):
    return lib().nfo_kv_offset(page, kv, entry, head, feat, page_size, Hkv, d)


def rope_freq(i, d, rope_scale, rope_theta, smooth_a=0.0, smooth_b=0.0):
    return lib().nfo_rope_freq(i, d, rope_scale, rope_theta, smooth_a, smooth_b)


def ref_llama_rope(x, offset, rope_scale=1.0, rope_theta=1e4):
    d = x.shape[0]
    out = np.empty((d,), np.float32)
    lib().nfo_ref_llama_rope(_h(x), out.ctypes.data_as(_f32p), d, offset, rope_scale, rope_theta)
    return out


def rope_append(kqv, kv_data, kv_indices, kv_indptr, rev_input_indptr, per_token_offset, Hq, Hkv, d,
                page_size, rope_scale=1.0, rope_theta=1e4, smooth_a=0.0, smooth_b=0.0,
                return_index=False):
    """Appends into kv_data IN PLACE; returns q_out (and (page, entry) per token)."""
    T = kqv.shape[0]
    assert kqv.shape[1] == (Hq + 2 * Hkv) * d
    q_out = np.empty((T, Hq * d), np.float16)
    pg = np.empty((T,), np.int32) if return_index else None
    en = np.empty((T,), np.int32) if return_index else None
    lib().nfo_rope_append_f16(_h(kqv), _h(q_out), _h(kv_data), _i(kv_indices), _i(kv_indptr),
                              _i(rev_input_indptr), _i(per_token_offset), T, Hq, Hkv, d, page_size,
                              rope_scale, rope_theta, smooth_a, smooth_b, _i(pg), _i(en))
    return (q_out, pg, en) if return_index else q_out


def attention_paged(q, qo_indptr, kv_data, kv_indptr, kv_indices, kv_last_page_len, Hq, Hkv, d,
                    page_size, causal, out=None):
    batch = kv_last_page_len.shape[0]
    o = np.zeros_like(q) if out is None else out
    lib().nfo_attention_paged_f16(_h(q), _h(o), _i(qo_indptr), _h(kv_data), _i(kv_indptr),
                                  _i(kv_indices), _i(kv_last_page_len), batch, Hq, Hkv, d, page_size,
                                  int(bool(causal)))
    return o


def _ptr_array(arrs):
    arr = (_u16p * len(arrs))()
    for i, a in enumerate(arrs):
        arr[i] = _h(a)
    return arr


def decoder_forward(cfg: dict, weights: dict, kv_data: list, batch: dict, hidden_in=None,
                    want_hidden=True, want_logits=False, want_sampled=True):
    """cfg: hidden,Hq,Hkv,d,ffn,vocab,layers,page_size,eps,rope_theta,rope_scale,smooth_a,smooth_b.
    weights: embedding, lm_head, model_norm and per-layer lists w_kqv,w_o,w_gate,w_up,w_down,
    ln_attn, ln_ffn, and optionally b_kqv (bias rows of the QKV projection).  kv_data: per-layer pools, appended IN PLACE.  batch: the update-data arrays.
    """
    m = NfoModel()
    for k in ("hidden", "Hq", "Hkv", "d", "ffn", "vocab", "layers", "page_size"):
        setattr(m, k, int(cfg[k]))
    for k in ("eps", "rope_theta", "rope_scale", "smooth_a", "smooth_b"):
        setattr(m, k, float(cfg.get(k, {"eps": 1e-5, "rope_theta": 1e4, "rope_scale": 1.0}.get(k, 0.0))))
    keep = []
    m.embedding = _h(weights["embedding"])
    m.lm_head = _h(weights["lm_head"])
    m.model_norm = _h(weights["model_norm"])
    for k in ("w_kqv", "w_o", "w_gate", "w_up", "w_down", "ln_attn", "ln_ffn"):
        pa = _ptr_array(weights[k])
        keep.append(pa)
        setattr(m, k, pa)
    if weights.get("b_kqv") is not None:      # the *_KQVBIAS pipeline types
        pa = _ptr_array(weights["b_kqv"])
        keep.append(pa)
        m.b_kqv = pa
    kva = _ptr_array(kv_data)
    m.kv_data = kva
    b = NfoBatch()
    b.decodePrefillBorder = int(batch["decodePrefillBorder"])
    b.prefillNum = int(batch["prefillNum"])
    b.prefillTokensNum = int(batch["prefillTokensNum"])
    for k in ("input_tokens", "input_indptr", "rev_input_indptr", "per_token_offset", "kv_indptr",
              "kv_indices", "kv_last_page_len"):
        arr = None if batch.get(k) is None else np.ascontiguousarray(batch[k], dtype=np.int32)
        keep.append(arr)  # the struct only holds raw pointers
        setattr(b, k, _i(arr))
    T = b.decodePrefillBorder + b.prefillTokensNum
    req = b.decodePrefillBorder + b.prefillNum
    hidden = np.empty((T, cfg["hidden"]), np.float16) if want_hidden else None
    logits = np.empty((req, cfg["vocab"]), np.float16) if want_logits else None
    sampled = np.empty((req,), np.int32) if want_sampled else None
    lib().nfo_decoder_forward(C.byref(m), C.byref(b), _h(hidden_in), _h(hidden), _h(logits),
                              _i(sampled))
    return hidden, logits, sampled
