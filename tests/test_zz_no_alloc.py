"""nf_gemm_f16_noalloc (partial sums of a GEMM split over K in the library's static device array,
no allocation inside the call) against nf_gemm_f16_ws with a caller workspace, through the C ABI:
two calls in a row, the second on a smaller input, so that whatever the first left in the array is
in the second one's way; bit-identical to the existing entry point (same kernels, same split) and
within the fp16 GEMM tolerance of the oracle."""
import ctypes as C

import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

from nanoflow_amd import synth  # noqa: E402

RTOL = 2e-3


def _call_noalloc(l, A, B, Cm, out, alpha, beta):
    M, K_ = A.shape
    N = B.shape[1]
    rc = l.nf_gemm_f16_noalloc(A.data_ptr(), B.data_ptr(), None if Cm is None else Cm.data_ptr(), out.data_ptr(),
                               M, N, K_, alpha, beta, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, l.nf_last_error().decode()


def test_gemm_noalloc_matches_the_workspace_entry_point_on_two_calls_in_a_row(oracle):
    from nanoflow_amd import kernels as K
    l = K.lib()
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    rng = np.random.default_rng(12)
    cap = l.nf_gemm_noalloc_scratch_bytes()
    assert cap == 32 << 20
    # (M, N, K, beta): split shapes, larger first; the last one is not split at all
    for M, N, K_, beta in [(200, 6144, 4096, 0.0), (64, 4096, 14336, 1.0), (16, 1024, 1024, 0.0), (700, 512, 256, 1.0)]:
        need = l.nf_gemm_workspace_bytes(M, N, K_)
        assert need <= cap
        print(f"noalloc gemm {M}x{N}x{K_} beta={beta} split workspace {need} B", flush=True)
        A = synth.normal_f16(rng, (M, K_))
        B = synth.normal_f16(rng, (K_, N), 0.02)
        Cm = synth.normal_f16(rng, (M, N)) if beta else None
        dA, dB, dC = dev(A), dev(B), (dev(Cm) if beta else None)
        out = torch.empty((M, N), dtype=torch.float16, device="cuda")
        _call_noalloc(l, dA, dB, dC, out, 1.0, beta)
        want, _ = K.gemm_ws(dA, dB, dC, alpha=1.0, beta=beta)
        torch.cuda.synchronize()
        assert torch.equal(out, want), (M, N, K_)
        ref = oracle.gemm(A, B, Cm, 1.0, beta).astype(np.float64)
        err = np.abs(out.cpu().numpy().astype(np.float64) - ref).max()
        assert err <= RTOL * np.abs(ref).max() * 2, (M, N, K_, err)


def test_gemm_noalloc_rejects_what_the_static_array_cannot_hold():
    from nanoflow_amd import kernels as K
    l = K.lib()
    # 512 rows x 8192 columns split 4 ways over K = 28672: four shares of 16 MiB of partial sums
    M, N, K_ = 512, 8192, 28672
    assert l.nf_gemm_workspace_bytes(M, N, K_) > l.nf_gemm_noalloc_scratch_bytes()
    A = torch.zeros((M, K_), dtype=torch.float16, device="cuda")
    B = torch.zeros((K_, N), dtype=torch.float16, device="cuda")
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    rc = l.nf_gemm_f16_noalloc(A.data_ptr(), B.data_ptr(), None, out.data_ptr(), M, N, K_, 1.0, 0.0, 0, None)
    assert rc == -1 and b"static" in l.nf_last_error()
