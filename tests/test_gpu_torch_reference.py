"""A second, oracle-independent check of the floating-point kernels: plain PyTorch fp32 on the GPU.

The oracle (oracle/nf_oracle.c) is the parity reference everywhere else; these few cases guard
against a mistake shared by a kernel and the oracle's restatement of the same formula.  Tolerance:
2e-3 relative to the largest magnitude, the bound stated for fp16 operators with fp32 accumulation.
"""
import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

from nanoflow_amd import synth  # noqa: E402

RTOL = 2e-3


def _close(got, ref, rtol=RTOL):
    err = (got.float() - ref).abs().max().item()
    assert err <= rtol * ref.abs().max().item(), (err, ref.abs().max().item())


@pytest.fixture(scope="module")
def K():
    from nanoflow_amd import kernels
    kernels.lib()
    return kernels


def test_gemm_against_torch_fp32(K):
    g = torch.Generator(device="cuda").manual_seed(1)
    for M, N, Kd in [(300, 1160, 520), (64, 4096, 4096), (2048, 6144, 512)]:
        A = torch.empty(M, Kd, dtype=torch.float16, device="cuda").normal_(0, 1, generator=g)
        B = torch.empty(Kd, N, dtype=torch.float16, device="cuda").normal_(0, 0.02, generator=g)
        C = torch.empty(M, N, dtype=torch.float16, device="cuda").normal_(0, 1, generator=g)
        ref = 0.5 * (A.float() @ B.float()) + 2.0 * C.float()
        _close(K.gemm(A, B, C, alpha=0.5, beta=2.0), ref)
        _close(K.gemm_ws(A, B, C, alpha=0.5, beta=2.0)[0], ref)                       # split over K where it applies
        _close(K.gemm(A, B.t().contiguous(), C, alpha=0.5, beta=2.0, b_col_major=True), ref)
        bias = torch.empty(N, dtype=torch.float16, device="cuda").normal_(0, 1, generator=g)
        _close(K.gemm(A, B, bias=bias, alpha=1.0, beta=1.0), A.float() @ B.float() + bias.float()[None, :])


def test_dual_swiglu_and_rmsnorm_against_torch_fp32(K):
    g = torch.Generator(device="cuda").manual_seed(2)
    M, N, Kd = 200, 2048, 1024
    A = torch.empty(M, Kd, dtype=torch.float16, device="cuda").normal_(0, 1, generator=g)
    Bg = torch.empty(Kd, N, dtype=torch.float16, device="cuda").normal_(0, 0.04, generator=g)
    Bu = torch.empty(Kd, N, dtype=torch.float16, device="cuda").normal_(0, 0.04, generator=g)
    gate, up = A.float() @ Bg.float(), A.float() @ Bu.float()
    ref = torch.nn.functional.silu(gate) * up
    # the kernel rounds both products to fp16 before SiLU-mul (the reference's epilogue types): two
    # more roundings than the fp32 formula, hence twice the tolerance
    _close(K.dual_swiglu(A, Bg, Bu), ref, 2 * RTOL)
    _close(K.dual_swiglu_ws(A, Bg, Bu)[0], ref, 2 * RTOL)
    x = torch.empty(77, 4096, dtype=torch.float16, device="cuda").normal_(0, 3, generator=g)
    w = torch.empty(4096, dtype=torch.float16, device="cuda").normal_(1, 0.02, generator=g)
    xf = x.float()
    _close(K.rmsnorm(x, w, 1e-5), xf * torch.rsqrt((xf * xf).mean(dim=1, keepdim=True) + 1e-5) * w.float())


@pytest.mark.parametrize("Hq,Hkv", [(32, 8), (64, 8), (8, 8)])
def test_paged_attention_against_torch_sdpa(K, Hq, Hkv):
    """Decode rows (non-causal, one row per request) and a causal prefill chunk against
    scaled_dot_product_attention on the keys and values gathered from the pages."""
    rng = np.random.default_rng(Hq)
    d, P = 128, 16
    shape = synth.ModelShape(Hq=Hq, Hkv=Hkv, hidden=Hq * d)
    b = synth.make_batch([300, 17, 1024, 64], [(40, 50)], vocab=10, seed=3, extra_pages=5)
    pool = synth.make_kv_pool(b.num_pages, shape, rng)
    q = synth.normal_f16(rng, (b.tokens, Hq * d))
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    nd = b.decodePrefillBorder
    dq, dpool = dev(q), dev(pool)
    out = torch.zeros_like(dq)
    K.attention_paged(dq, dev(b.input_indptr[:nd + 1]), dpool, dev(b.kv_indptr[:nd + 1]), dev(b.kv_indices),
                      dev(b.kv_last_page_len[:nd]), Hq, Hkv, causal=False, out=out, batch=nd, max_qo_rows=nd)
    K.attention_paged(dq, dev(b.input_indptr[nd:]), dpool, dev(b.kv_indptr[nd:]), dev(b.kv_indices),
                      dev(b.kv_last_page_len[nd:]), Hq, Hkv, causal=True, out=out, batch=b.req_num - nd,
                      max_qo_rows=b.tokens - nd)
    torch.cuda.synchronize()
    for r in range(b.req_num):
        pages = torch.from_numpy(b.kv_indices[b.kv_indptr[r]:b.kv_indptr[r + 1]].astype(np.int64)).cuda()
        L = int(b.kv_len[r])
        k = dpool[pages, 0].reshape(-1, Hkv, d)[:L].float()          # [L, Hkv, d]
        v = dpool[pages, 1].reshape(-1, Hkv, d)[:L].float()
        rows = slice(int(b.input_indptr[r]), int(b.input_indptr[r + 1]))
        qr = dq[rows].float().reshape(-1, Hq, d)                     # [n, Hq, d]
        n = qr.shape[0]
        kk = k.repeat_interleave(Hq // Hkv, dim=1).permute(1, 0, 2)  # [Hq, L, d]
        vv = v.repeat_interleave(Hq // Hkv, dim=1).permute(1, 0, 2)
        mask = None
        if r >= nd:      # row i of the chunk sees keys up to L - n + i
            mask = torch.arange(L, device="cuda")[None, :] <= (L - n + torch.arange(n, device="cuda"))[:, None]
        ref = torch.nn.functional.scaled_dot_product_attention(qr.permute(1, 0, 2), kk, vv, attn_mask=mask)
        _close(out[rows].reshape(n, Hq, d).permute(1, 0, 2), ref)
