"""ctypes binding of the gfx950 kernel library (C ABI: include/nanoflow_kernels.h).

Operands are torch CUDA tensors used purely as device buffers; every call enqueues on
torch's current stream and returns without synchronising.  There is no CPU or PyTorch
fallback: if the compiled library is missing or a call is rejected, an exception is raised.
"""
from __future__ import annotations

import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnf_kernels.so")

SYMBOLS = [
    "nf_abi_version", "nf_last_error", "nf_embedding_f16", "nf_rmsnorm_f16", "nf_gemm_f16", "nf_gemm_bias_f16",
    "nf_gemm_workspace_bytes", "nf_gemm_workspace_bytes_upto", "nf_gemm_f16_ws", "nf_gemm_bias_f16_ws",
    "nf_dual_swiglu_workspace_bytes", "nf_dual_swiglu_workspace_bytes_upto", "nf_dual_swiglu_f16_ws",
    "nf_dual_swiglu_f16", "nf_gemm_bf16", "nf_dual_swiglu_bf16", "nf_quantize_rows_e4m3", "nf_gemm_f8_f16", "nf_gemm_f8w_workspace_bytes",
    "nf_quantize_weight_e4m3", "nf_dual_swiglu_f8_f16", "nf_dual_swiglu_f8w_f16", "nf_move_kv_pages",
    "nf_gemm_f8w_split_workspace_bytes", "nf_gemm_f8w_split_workspace_bytes_upto",
    "nf_dual_swiglu_f8w_split_workspace_bytes", "nf_dual_swiglu_f8w_split_workspace_bytes_upto",
    "nf_gemm_f8w_f16", "nf_rope_append_f16", "nf_attention_workspace_bytes",
    "nf_attention_paged_f16", "nf_keep_token_f16", "nf_argmax_f16",
    "nf_calibrate_mfma", "nf_calibrate_hbm_read", "nf_calibrate_paged_read",
    "nf_gemm_f16_noalloc", "nf_gemm_noalloc_scratch_bytes",
    "nf_split_kqv_f16", "nf_extract_rank_columns_f16", "nf_silu_mul_f16", "nf_transpose_f16", "nf_sleep_us",
    "nf_gemm_tile_menu", "nf_gemm_tiled_workspace_bytes", "nf_gemm_f16_tiled",
    "nf_rmsnorm_quantize_e4m3", "nf_gemm_f8q_f16", "nf_dual_swiglu_f8q_f16",
]


class NanoflowKernelError(RuntimeError):
    pass


_lib = None


def lib() -> C.CDLL:
    """Loads libnf_kernels.so (built by ``make -C nanoflow_amd/csrc`` / ``__graft_entry__.build``)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise NanoflowKernelError(
                f"{LIB_PATH} is missing: build it with `make -C nanoflow_amd/csrc` "
                "(there is no fallback path)")
        l = C.CDLL(LIB_PATH)
        vp, i32, f32, sz = C.c_void_p, C.c_int, C.c_float, C.c_size_t
        l.nf_abi_version.restype = i32
        l.nf_last_error.restype = C.c_char_p
        l.nf_embedding_f16.argtypes = [vp, vp, vp, i32, i32, vp]
        l.nf_rmsnorm_f16.argtypes = [vp, vp, vp, i32, i32, f32, vp]
        l.nf_gemm_f16.argtypes = [vp, vp, vp, vp, i32, i32, i32, f32, f32, i32, vp]
        l.nf_gemm_workspace_bytes.restype = sz
        l.nf_gemm_workspace_bytes.argtypes = [i32, i32, i32]
        l.nf_gemm_workspace_bytes_upto.restype = sz
        l.nf_gemm_workspace_bytes_upto.argtypes = [i32, i32, i32]
        l.nf_gemm_f16_ws.argtypes = [vp, vp, vp, vp, i32, i32, i32, f32, f32, i32, vp, sz, vp]
        l.nf_dual_swiglu_workspace_bytes.restype = sz
        l.nf_dual_swiglu_workspace_bytes.argtypes = [i32, i32, i32]
        l.nf_dual_swiglu_workspace_bytes_upto.restype = sz
        l.nf_dual_swiglu_workspace_bytes_upto.argtypes = [i32, i32, i32]
        l.nf_dual_swiglu_f16_ws.argtypes = [vp, vp, vp, vp, i32, i32, i32, i32, vp, sz, vp]
        l.nf_gemm_bias_f16_ws.argtypes = [vp, vp, vp, vp, i32, i32, i32, f32, f32, i32, vp, sz, vp]
        l.nf_gemm_bias_f16.argtypes = [vp, vp, vp, vp, i32, i32, i32, f32, f32, i32, vp]
        l.nf_dual_swiglu_f16.argtypes = [vp, vp, vp, vp, i32, i32, i32, i32, vp]
        l.nf_gemm_bf16.argtypes = [vp, vp, vp, vp, i32, i32, i32, f32, f32, i32, vp]
        l.nf_dual_swiglu_bf16.argtypes = [vp, vp, vp, vp, i32, i32, i32, vp]
        l.nf_quantize_rows_e4m3.argtypes = [vp, vp, vp, i32, i32, vp]
        l.nf_gemm_f8_f16.argtypes = [vp, vp, vp, vp, vp, vp, i32, i32, i32, f32, f32, vp]
        l.nf_gemm_f8w_workspace_bytes.restype = C.c_size_t
        l.nf_gemm_f8w_workspace_bytes.argtypes = [i32, i32]
        l.nf_gemm_f8w_f16.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, f32, f32, vp, C.c_size_t, vp]
        for name in ("nf_gemm_f8w_split_workspace_bytes", "nf_gemm_f8w_split_workspace_bytes_upto",
                     "nf_dual_swiglu_f8w_split_workspace_bytes", "nf_dual_swiglu_f8w_split_workspace_bytes_upto"):
            getattr(l, name).restype = sz
            getattr(l, name).argtypes = [i32, i32, i32]
        l.nf_quantize_weight_e4m3.argtypes = [vp, vp, vp, i32, i32, vp]
        l.nf_rmsnorm_quantize_e4m3.argtypes = [vp, vp, vp, vp, vp, i32, i32, f32, vp]
        l.nf_gemm_f8q_f16.argtypes = [vp, vp, vp, vp, vp, vp, i32, i32, i32, f32, f32, vp, C.c_size_t, vp]
        l.nf_dual_swiglu_f8q_f16.argtypes = [vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, vp, C.c_size_t, vp]
        l.nf_dual_swiglu_f8_f16.argtypes = [vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, vp]
        l.nf_dual_swiglu_f8w_f16.argtypes = [vp, vp, vp, vp, vp, vp, i32, i32, i32, vp, C.c_size_t, vp]
        l.nf_move_kv_pages.argtypes = [i32, vp, vp, vp, vp, vp, sz, i32, vp]
        l.nf_rope_append_f16.argtypes = [vp] * 7 + [i32] * 5 + [f32] * 4 + [vp]
        l.nf_gemm_f16_noalloc.argtypes = [vp, vp, vp, vp, i32, i32, i32, f32, f32, i32, vp]
        l.nf_gemm_noalloc_scratch_bytes.restype = sz
        l.nf_gemm_noalloc_scratch_bytes.argtypes = []
        l.nf_split_kqv_f16.argtypes = [vp, vp, vp, vp, i32, i32, i32, i32, vp]
        l.nf_extract_rank_columns_f16.argtypes = [vp, vp, i32, i32, i32, i32, vp]
        l.nf_silu_mul_f16.argtypes = [vp, vp, i32, i32, vp]
        l.nf_transpose_f16.argtypes = [vp, vp, i32, i32, vp]
        l.nf_sleep_us.argtypes = [i32, vp]
        ip = C.POINTER(C.c_int)
        l.nf_gemm_tile_menu.argtypes = [i32, ip, ip, ip]
        l.nf_gemm_tiled_workspace_bytes.restype = sz
        l.nf_gemm_tiled_workspace_bytes.argtypes = [i32, i32, i32, i32]
        l.nf_gemm_f16_tiled.argtypes = [vp, vp, vp, vp, i32, i32, i32, f32, f32, i32, i32, i32, i32, i32, vp, sz, vp]
        dp = C.POINTER(C.c_double)
        l.nf_calibrate_mfma.argtypes = [i32, i32, i32, vp, sz, dp, dp, vp]
        l.nf_calibrate_hbm_read.argtypes = [vp, sz, i32, vp, sz, dp, vp]
        l.nf_calibrate_paged_read.argtypes = [vp, vp, vp, vp, i32, i32, sz, i32, vp, sz, dp, vp]
        l.nf_attention_workspace_bytes.restype = sz
        l.nf_attention_workspace_bytes.argtypes = [i32, i32, i32]
        l.nf_attention_paged_f16.argtypes = [vp] * 7 + [i32] * 8 + [vp, sz, vp]
        l.nf_keep_token_f16.argtypes = [vp, vp, vp, i32, i32, vp]
        l.nf_argmax_f16.argtypes = [vp, vp, vp, i32, i32, vp]
        for name in SYMBOLS:
            if name not in ("nf_last_error", "nf_attention_workspace_bytes", "nf_gemm_workspace_bytes",
                            "nf_gemm_workspace_bytes_upto", "nf_gemm_f8w_workspace_bytes", "nf_gemm_tiled_workspace_bytes",
                            "nf_dual_swiglu_workspace_bytes", "nf_dual_swiglu_workspace_bytes_upto",
                            "nf_gemm_f8w_split_workspace_bytes", "nf_gemm_f8w_split_workspace_bytes_upto",
                            "nf_dual_swiglu_f8w_split_workspace_bytes", "nf_dual_swiglu_f8w_split_workspace_bytes_upto"):
                getattr(l, name).restype = i32
        _lib = l
    return _lib


def _check(rc: int, what: str):
    if rc != 0:
        raise NanoflowKernelError(f"{what} failed ({rc}): {lib().nf_last_error().decode()}")


def _p(t):
    if t is None:
        return None
    assert t.is_cuda and t.is_contiguous(), "device-resident contiguous tensor required"
    return t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _f16(t):
    assert t.dtype == torch.float16, t.dtype


def _i32(t):
    assert t.dtype == torch.int32, t.dtype


def embedding(tokens, table, out=None):
    _i32(tokens); _f16(table)
    T, H = tokens.numel(), table.shape[1]
    out = torch.empty((T, H), dtype=torch.float16, device=table.device) if out is None else out
    _check(lib().nf_embedding_f16(_p(tokens), _p(table), _p(out), T, H, _stream()), "nf_embedding_f16")
    return out


def rmsnorm(x, w, eps=1e-5, out=None):
    _f16(x); _f16(w)
    rows, H = x.shape
    out = torch.empty_like(x) if out is None else out
    _check(lib().nf_rmsnorm_f16(_p(out), _p(x), _p(w), rows, H, eps, _stream()), "nf_rmsnorm_f16")
    return out


def rmsnorm_quantize_e4m3(x, w, eps=1e-5):
    """(fp16 RMSNorm output, its e4m3 bytes, fp32 row scales) from one launch."""
    _f16(x); _f16(w)
    rows, H = x.shape
    out = torch.empty_like(x)
    q = torch.empty((rows, H), dtype=torch.uint8, device=x.device)
    scale = torch.empty((rows,), dtype=torch.float32, device=x.device)
    _check(lib().nf_rmsnorm_quantize_e4m3(_p(out), _p(x), _p(w), _p(q), _p(scale), rows, H, eps, _stream()),
           "nf_rmsnorm_quantize_e4m3")
    return out, q, scale


def _elem(t, dtype):
    assert t.is_cuda and t.dtype == dtype and t.is_contiguous(), (t.dtype, t.device)


def gemm(A, B, Cmat=None, alpha=1.0, beta=0.0, b_col_major=False, out=None, bias=None):
    """fp16 operands run nf_gemm_f16, bfloat16 operands nf_gemm_bf16 (same kernels, other element type).
    bias [N] (fp16 only, instead of Cmat): beta * bias is added to every row (nf_gemm_bias_f16)."""
    dt = A.dtype
    assert dt in (torch.float16, torch.bfloat16), dt
    _elem(A, dt); _elem(B, dt)
    M, K = A.shape
    N = B.shape[0] if b_col_major else B.shape[1]
    assert tuple(B.shape) == ((N, K) if b_col_major else (K, N)), (A.shape, B.shape)
    if bias is not None:
        assert Cmat is None and dt == torch.float16 and bias.numel() == N
        _elem(bias, dt)
        out = torch.empty((M, N), dtype=dt, device=A.device) if out is None else out
        _elem(out, dt)
        _check(lib().nf_gemm_bias_f16(_p(A), _p(B), _p(bias), _p(out), M, N, K, alpha, beta, int(b_col_major),
                                      _stream()), "nf_gemm_bias_f16")
        return out
    if Cmat is not None:
        _elem(Cmat, dt)
        assert tuple(Cmat.shape) == (M, N)
    out = torch.empty((M, N), dtype=dt, device=A.device) if out is None else out
    _elem(out, dt)
    fn, name = (lib().nf_gemm_f16, "nf_gemm_f16") if dt == torch.float16 else (lib().nf_gemm_bf16, "nf_gemm_bf16")
    _check(fn(_p(A), _p(B), _p(Cmat), _p(out), M, N, K, alpha, beta, int(b_col_major), _stream()), name)
    return out


def gemm_ws(A, B, Cmat=None, alpha=1.0, beta=0.0, b_col_major=False, out=None, workspace=None, bias=None):
    """nf_gemm_f16_ws: fp16 GEMM that is split over K through a workspace when few rows against a narrow
    N would leave most of the chip idle.  Returns (out, shares_bytes) where shares_bytes is the
    workspace the shape asked for (0: not split)."""
    _f16(A); _f16(B)
    M, K = A.shape
    N = B.shape[0] if b_col_major else B.shape[1]
    assert tuple(B.shape) == ((N, K) if b_col_major else (K, N)), (A.shape, B.shape)
    if Cmat is not None:
        _f16(Cmat)
        assert tuple(Cmat.shape) == (M, N)
    need = lib().nf_gemm_workspace_bytes(M, N, K)
    if workspace is None:
        workspace = torch.empty((max(need, 16),), dtype=torch.uint8, device=A.device)
    out = torch.empty((M, N), dtype=torch.float16, device=A.device) if out is None else out
    if bias is not None:          # one row [N] added (times beta) to every row: nf_gemm_bias_f16_ws
        assert Cmat is None and bias.numel() == N
        _f16(bias)
        _check(lib().nf_gemm_bias_f16_ws(_p(A), _p(B), _p(bias), _p(out), M, N, K, alpha, beta, int(b_col_major),
                                         _p(workspace), workspace.numel(), _stream()), "nf_gemm_bias_f16_ws")
        return out, need
    _check(lib().nf_gemm_f16_ws(_p(A), _p(B), _p(Cmat), _p(out), M, N, K, alpha, beta, int(b_col_major),
                                _p(workspace), workspace.numel(), _stream()), "nf_gemm_f16_ws")
    return out, need


def gemm_tile_menu():
    """[(tile_m, tile_n, takes k-contiguous weights only)] of the tiles nf_gemm_f16_tiled chooses from."""
    m, n, c = C.c_int(), C.c_int(), C.c_int()
    out = []
    for i in range(lib().nf_gemm_tile_menu(-1, None, None, None)):
        lib().nf_gemm_tile_menu(i, C.byref(m), C.byref(n), C.byref(c))
        out.append((m.value, n.value, bool(c.value)))
    return out


def gemm_tiled(A, B, tile, split_k=1, Cmat=None, alpha=1.0, beta=0.0, b_col_major=False, out=None, bias=None,
               workspace=None):
    """nf_gemm_f16_tiled: the GEMM on the menu tile closest to ``tile`` = (m, n), K cut into ``split_k`` shares."""
    _f16(A); _f16(B)
    M, K = A.shape
    N = B.shape[0] if b_col_major else B.shape[1]
    assert tuple(B.shape) == ((N, K) if b_col_major else (K, N))
    need = lib().nf_gemm_tiled_workspace_bytes(M, N, K, split_k)
    if workspace is None:
        workspace = torch.empty((max(need, 16),), dtype=torch.uint8, device=A.device)
    out = torch.empty((M, N), dtype=torch.float16, device=A.device) if out is None else out
    c = bias if bias is not None else Cmat
    _check(lib().nf_gemm_f16_tiled(_p(A), _p(B), _p(c), _p(out), M, N, K, alpha, beta, int(b_col_major),
                                   int(bias is not None), tile[0], tile[1], split_k, _p(workspace), workspace.numel(),
                                   _stream()), "nf_gemm_f16_tiled")
    return out


def dual_swiglu_ws(A, Bg, Bu, out=None, workspace=None, b_col_major=False):
    """nf_dual_swiglu_f16_ws; returns (out, bytes of workspace the shape asks for: 0 = not split).
    b_col_major: Bg / Bu are [N, K] (k contiguous) instead of [K, N]."""
    _f16(A); _f16(Bg); _f16(Bu)
    M, K = A.shape
    N = Bg.shape[0] if b_col_major else Bg.shape[1]
    assert tuple(Bg.shape) == ((N, K) if b_col_major else (K, N)) and Bu.shape == Bg.shape
    need = lib().nf_dual_swiglu_workspace_bytes(M, N, K)
    if workspace is None:
        workspace = torch.empty((max(need, 16),), dtype=torch.uint8, device=A.device)
    out = torch.empty((M, N), dtype=torch.float16, device=A.device) if out is None else out
    _check(lib().nf_dual_swiglu_f16_ws(_p(A), _p(Bg), _p(Bu), _p(out), M, N, K, int(b_col_major), _p(workspace),
                                       workspace.numel(), _stream()), "nf_dual_swiglu_f16_ws")
    return out, need


def dual_swiglu(A, Bg, Bu, out=None, b_col_major=False):
    """b_col_major (fp16 only): Bg / Bu are [N, K] (k contiguous) instead of [K, N]."""
    dt = A.dtype
    assert dt in (torch.float16, torch.bfloat16), dt
    _elem(A, dt); _elem(Bg, dt); _elem(Bu, dt)
    M, K = A.shape
    N = Bg.shape[0] if b_col_major else Bg.shape[1]
    assert tuple(Bg.shape) == ((N, K) if b_col_major else (K, N)) and Bu.shape == Bg.shape
    out = torch.empty((M, N), dtype=dt, device=A.device) if out is None else out
    _elem(out, dt)
    if dt == torch.float16:
        _check(lib().nf_dual_swiglu_f16(_p(A), _p(Bg), _p(Bu), _p(out), M, N, K, int(b_col_major), _stream()),
               "nf_dual_swiglu_f16")
    else:
        assert not b_col_major, "the bf16 pair takes [K, N] weights only"
        _check(lib().nf_dual_swiglu_bf16(_p(A), _p(Bg), _p(Bu), _p(out), M, N, K, _stream()), "nf_dual_swiglu_bf16")
    return out


def quantize_rows_e4m3(X):
    """fp16 [M,K] -> (e4m3 bytes [M,K], fp32 row scales [M])."""
    _f16(X)
    M, K = X.shape
    Xq = torch.empty((M, K), dtype=torch.uint8, device=X.device)
    scale = torch.empty((M,), dtype=torch.float32, device=X.device)
    _check(lib().nf_quantize_rows_e4m3(_p(X), _p(Xq), _p(scale), M, K, _stream()), "nf_quantize_rows_e4m3")
    return Xq, scale


def gemm_f8(Aq, a_scale, Bq_nk, b_scale, Cmat=None, alpha=1.0, beta=0.0, out=None):
    """Aq e4m3 bytes [M,K], Bq_nk e4m3 bytes [N,K] (one row per output channel)."""
    assert Aq.dtype == torch.uint8 and Bq_nk.dtype == torch.uint8
    assert a_scale.dtype == torch.float32 and b_scale.dtype == torch.float32
    M, K = Aq.shape
    N = Bq_nk.shape[0]
    assert tuple(Bq_nk.shape) == (N, K) and a_scale.numel() == M and b_scale.numel() == N
    assert Aq.is_contiguous() and Bq_nk.is_contiguous()
    out = torch.empty((M, N), dtype=torch.float16, device=Aq.device) if out is None else out
    _check(lib().nf_gemm_f8_f16(_p(Aq), _p(a_scale), _p(Bq_nk), _p(b_scale), _p(Cmat), _p(out), M, N, K,
                                alpha, beta, _stream()), "nf_gemm_f8_f16")
    return out


def gemm_f8w(A, Bq_nk, b_scale, Cmat=None, alpha=1.0, beta=0.0, out=None, workspace=None):
    """fp16 activations [M,K] against e4m3 weights [N,K] with per-output-channel scales."""
    _f16(A)
    assert Bq_nk.dtype == torch.uint8 and b_scale.dtype == torch.float32 and Bq_nk.is_contiguous()
    M, K = A.shape
    N = Bq_nk.shape[0]
    assert tuple(Bq_nk.shape) == (N, K) and b_scale.numel() == N
    need = lib().nf_gemm_f8w_split_workspace_bytes(M, N, K)      # quantised rows (+ the sums of a split over K)
    if workspace is None:
        workspace = torch.empty((max(need, 16),), dtype=torch.uint8, device=A.device)
    out = torch.empty((M, N), dtype=torch.float16, device=A.device) if out is None else out
    _check(lib().nf_gemm_f8w_f16(_p(A), _p(Bq_nk), _p(b_scale), _p(Cmat), _p(out), M, N, K, alpha, beta,
                                 _p(workspace), workspace.numel() * workspace.element_size(), _stream()),
           "nf_gemm_f8w_f16")
    return out


def gemm_f8q(Aq, a_scale, Bq_nk, b_scale, Cmat=None, alpha=1.0, beta=0.0, out=None, workspace=None):
    """nf_gemm_f8w_f16 on rows that are quantised already; the workspace only holds the sums of a split over K."""
    M, K = Aq.shape
    N = Bq_nk.shape[0]
    need = lib().nf_gemm_f8w_split_workspace_bytes(M, N, K)
    if workspace is None:
        workspace = torch.empty((max(need, 16),), dtype=torch.uint8, device=Aq.device)
    out = torch.empty((M, N), dtype=torch.float16, device=Aq.device) if out is None else out
    _check(lib().nf_gemm_f8q_f16(_p(Aq), _p(a_scale), _p(Bq_nk), _p(b_scale), _p(Cmat), _p(out), M, N, K, alpha, beta,
                                 _p(workspace), workspace.numel(), _stream()), "nf_gemm_f8q_f16")
    return out


def dual_swiglu_f8q(Aq, a_scale, Gq, g_scale, Uq, u_scale, out=None, workspace=None):
    M, Kd = Aq.shape
    N = Gq.shape[0]
    need = lib().nf_dual_swiglu_f8w_split_workspace_bytes(M, N, Kd)
    if workspace is None:
        workspace = torch.empty((max(need, 16),), dtype=torch.uint8, device=Aq.device)
    out = torch.empty((M, N), dtype=torch.float16, device=Aq.device) if out is None else out
    _check(lib().nf_dual_swiglu_f8q_f16(_p(Aq), _p(a_scale), _p(Gq), _p(g_scale), _p(Uq), _p(u_scale), _p(out), M, N,
                                        Kd, _p(workspace), workspace.numel(), _stream()), "nf_dual_swiglu_f8q_f16")
    return out


def quantize_weight_e4m3(W):
    """W fp16 [K,N] (the pipeline's weight orientation) -> (Wq e4m3 bytes [N,K], col_scale fp32 [N])."""
    _f16(W)
    Kd, N = W.shape
    Wq = torch.empty((N, Kd), dtype=torch.uint8, device=W.device)
    scale = torch.empty((N,), dtype=torch.float32, device=W.device)
    _check(lib().nf_quantize_weight_e4m3(_p(W), _p(Wq), _p(scale), Kd, N, _stream()), "nf_quantize_weight_e4m3")
    return Wq, scale


def dual_swiglu_f8(Aq, a_scale, Gq, g_scale, Uq, u_scale, out=None):
    assert Aq.dtype == torch.uint8 and Gq.dtype == torch.uint8 and Uq.dtype == torch.uint8
    M, Kd = Aq.shape
    N = Gq.shape[0]
    assert tuple(Gq.shape) == (N, Kd) and tuple(Uq.shape) == (N, Kd)
    assert a_scale.numel() == M and g_scale.numel() == N and u_scale.numel() == N
    out = torch.empty((M, N), dtype=torch.float16, device=Aq.device) if out is None else out
    _check(lib().nf_dual_swiglu_f8_f16(_p(Aq), _p(a_scale), _p(Gq), _p(g_scale), _p(Uq), _p(u_scale), _p(out),
                                       M, N, Kd, _stream()), "nf_dual_swiglu_f8_f16")
    return out


def dual_swiglu_f8w(A, Gq, g_scale, Uq, u_scale, out=None, workspace=None):
    """fp16 activations [M,K] against e4m3 gate/up weights [N,K] with per-output-channel scales."""
    _f16(A)
    M, Kd = A.shape
    N = Gq.shape[0]
    assert tuple(Gq.shape) == (N, Kd) and tuple(Uq.shape) == (N, Kd)
    need = lib().nf_dual_swiglu_f8w_split_workspace_bytes(M, N, Kd)
    if workspace is None:
        workspace = torch.empty((max(need, 16),), dtype=torch.uint8, device=A.device)
    out = torch.empty((M, N), dtype=torch.float16, device=A.device) if out is None else out
    _check(lib().nf_dual_swiglu_f8w_f16(_p(A), _p(Gq), _p(g_scale), _p(Uq), _p(u_scale), _p(out), M, N, Kd,
                                        _p(workspace), workspace.numel() * workspace.element_size(), _stream()),
           "nf_dual_swiglu_f8w_f16")
    return out


def rope_append(kqv, kv_data, kv_indices, kv_indptr, rev_input_indptr, per_token_offset, Hq, Hkv,
                d=128, page_size=16, rope_scale=1.0, rope_theta=1e4, smooth_a=0.0, smooth_b=0.0,
                q_out=None, n_tokens=None):
    """Appends K/V into kv_data IN PLACE and returns the rotated Q rows."""
    _f16(kqv); _f16(kv_data)
    for t in (kv_indices, kv_indptr, rev_input_indptr, per_token_offset):
        _i32(t)
    T = kqv.shape[0] if n_tokens is None else n_tokens
    assert kqv.shape[1] == (Hq + 2 * Hkv) * d
    q_out = torch.empty((kqv.shape[0], Hq * d), dtype=torch.float16, device=kqv.device) \
        if q_out is None else q_out
    _check(lib().nf_rope_append_f16(_p(kqv), _p(q_out), _p(kv_data), _p(kv_indices), _p(kv_indptr),
                                    _p(rev_input_indptr), _p(per_token_offset), T, Hq, Hkv, d,
                                    page_size, rope_scale, rope_theta, smooth_a, smooth_b, _stream()),
           "nf_rope_append_f16")
    return q_out


def attention_paged(q, qo_indptr, kv_data, kv_indptr, kv_indices, kv_last_page_len, Hq, Hkv, d=128,
                    page_size=16, causal=False, out=None, batch=None, max_qo_rows=None,
                    num_blocks=0, workspace=None):
    _f16(q); _f16(kv_data)
    for t in (qo_indptr, kv_indptr, kv_indices, kv_last_page_len):
        _i32(t)
    batch = kv_last_page_len.numel() if batch is None else batch
    max_qo_rows = q.shape[0] if max_qo_rows is None else max_qo_rows
    out = torch.zeros_like(q) if out is None else out
    need = lib().nf_attention_workspace_bytes(batch, max_qo_rows, Hq)
    if workspace is None:
        workspace = torch.empty((max(need, 1),), dtype=torch.uint8, device=q.device)
    _check(lib().nf_attention_paged_f16(_p(q), _p(out), _p(qo_indptr), _p(kv_data), _p(kv_indptr),
                                        _p(kv_indices), _p(kv_last_page_len), batch, max_qo_rows,
                                        Hq, Hkv, d, page_size, int(bool(causal)), num_blocks,
                                        _p(workspace), workspace.numel(), _stream()),
           "nf_attention_paged_f16")
    return out


def move_kv_pages(req_idx, kv_indptr, kv_indices, staging, kv_data, to_pool: bool):
    """Pages of the requests in req_idx between one layer's pool kv_data [pages, 2, page, Hkv, d] and
    staging [len(kv_indices), 2, page, Hkv, d] (page j of staging <-> pool page kv_indices[j])."""
    for t in (req_idx, kv_indptr, kv_indices):
        _i32(t)
    _f16(staging); _f16(kv_data)
    page_bytes = kv_data[0].numel() * 2
    assert staging[0].numel() * 2 == page_bytes and staging.shape[0] >= kv_indices.numel()
    _check(lib().nf_move_kv_pages(req_idx.numel(), _p(req_idx), _p(kv_indptr), _p(kv_indices), _p(staging),
                                  _p(kv_data), page_bytes, int(bool(to_pool)), _stream()), "nf_move_kv_pages")


def split_kqv(kqv, k_dim, q_dim, v_dim):
    """(k, q, v): the three column ranges of kqv [rows, k_dim + q_dim + v_dim], in that order."""
    _f16(kqv)
    rows = kqv.shape[0]
    assert kqv.shape[1] == k_dim + q_dim + v_dim
    outs = [torch.empty((rows, d), dtype=torch.float16, device=kqv.device) for d in (k_dim, q_dim, v_dim)]
    _check(lib().nf_split_kqv_f16(_p(kqv), *[_p(o) if o.numel() else None for o in outs], rows, k_dim, q_dim, v_dim,
                                  _stream()), "nf_split_kqv_f16")
    return tuple(outs)


def extract_rank_columns(x, nranks, rank):
    _f16(x)
    rows, cols = x.shape[0], x.shape[1] // nranks
    assert x.shape[1] == nranks * cols
    out = torch.empty((rows, cols), dtype=torch.float16, device=x.device)
    _check(lib().nf_extract_rank_columns_f16(_p(x), _p(out), rows, cols, nranks, rank, _stream()),
           "nf_extract_rank_columns_f16")
    return out


def silu_mul(x):
    """[rows, 2 * cols] -> [rows, cols]: x[:, :cols] * silu(x[:, cols:])."""
    _f16(x)
    rows, cols = x.shape[0], x.shape[1] // 2
    assert x.shape[1] == 2 * cols
    out = torch.empty((rows, cols), dtype=torch.float16, device=x.device)
    _check(lib().nf_silu_mul_f16(_p(x), _p(out), rows, cols, _stream()), "nf_silu_mul_f16")
    return out


def transpose(x):
    _f16(x)
    rows, cols = x.shape
    out = torch.empty((cols, rows), dtype=torch.float16, device=x.device)
    _check(lib().nf_transpose_f16(_p(x), _p(out), rows, cols, _stream()), "nf_transpose_f16")
    return out


def sleep_us(us):
    _check(lib().nf_sleep_us(int(us), _stream()), "nf_sleep_us")


def keep_token(x, input_indptr, req_num, out=None):
    _f16(x); _i32(input_indptr)
    H = x.shape[1]
    out = torch.empty((req_num, H), dtype=torch.float16, device=x.device) if out is None else out
    _check(lib().nf_keep_token_f16(_p(x), _p(out), _p(input_indptr), req_num, H, _stream()),
           "nf_keep_token_f16")
    return out


def argmax(logits, rows=None):
    _f16(logits)
    rows = logits.shape[0] if rows is None else rows
    cols = logits.shape[1]
    mv = torch.empty((rows,), dtype=torch.float16, device=logits.device)
    arg = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    _check(lib().nf_argmax_f16(_p(logits), _p(mv), _p(arg), rows, cols, _stream()), "nf_argmax_f16")
    return arg, mv


# ---------------------------------------------------------------- calibration micro-benchmarks

def calibrate_mfma(fp8: bool = False, random_operands=True, iters: int = 20000):
    """(TFLOP/s, shader clock in MHz) of an MFMA loop on this device.  random_operands: False = zero
    operands in registers, True = pseudo-random ones, 2 = pseudo-random ones re-read from LDS before
    every 16 MFMAs (fp16 only), as a GEMM's main loop reads its fragments, 3 = with the operand loads
    of a 256x256 tile (L2 -> LDS) beside them as well, 4 = as True with 16x16 MFMAs."""
    scratch = torch.zeros(8192 + ((8 << 20) if int(random_operands) == 3 else 0), dtype=torch.uint8, device="cuda")
    tf, mhz = C.c_double(), C.c_double()
    _check(lib().nf_calibrate_mfma(int(fp8), int(random_operands), iters, scratch.data_ptr(), scratch.numel(),
                                   C.byref(tf), C.byref(mhz), _stream()), "nf_calibrate_mfma")
    return tf.value, mhz.value


def calibrate_hbm_read(gib: float = 8.0, reps: int = 4) -> float:
    """GB/s of all CUs streaming a buffer of `gib` GiB (freed again before returning)."""
    n = int(gib * (1 << 30)) // 16 * 16
    buf = torch.empty(n, dtype=torch.uint8, device="cuda")
    buf.random_()   # touched: every page is backed
    scratch = torch.zeros(8192, dtype=torch.uint8, device="cuda")
    g = C.c_double()
    _check(lib().nf_calibrate_hbm_read(buf.data_ptr(), n, reps, scratch.data_ptr(), scratch.numel(), C.byref(g), _stream()),
           "nf_calibrate_hbm_read")
    del buf
    torch.cuda.empty_cache()
    return g.value


def calibrate_paged_read(pool, kv_indptr, kv_indices, kv_last_page_len, batch: int, num_kv_heads: int,
                         kv_bytes: int, reps: int = 10) -> float:
    """GB/s of paged decode attention's load pattern with the arithmetic removed."""
    scratch = torch.zeros(8192, dtype=torch.uint8, device="cuda")
    g = C.c_double()
    _check(lib().nf_calibrate_paged_read(pool.data_ptr(), kv_indptr.data_ptr(), kv_indices.data_ptr(),
                                         kv_last_page_len.data_ptr(), batch, num_kv_heads, kv_bytes, reps,
                                         scratch.data_ptr(), scratch.numel(), C.byref(g), _stream()), "nf_calibrate_paged_read")
    return g.value
