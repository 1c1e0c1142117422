"""Parity of every HIP operator (through the C ABI) with the CPU oracle on the same seeded
inputs.  Integer/index/copy results are compared bit-exactly; floating-point results within
2e-3 relative (fp16 storage, fp32 accumulate)."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

from nanoflow_amd import synth  # noqa: E402

RTOL = 2e-3


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def assert_close(got, ref, rtol=RTOL, what=""):
    """|got-ref| <= rtol*|ref| + rtol*rms(ref) elementwise, and max-norm relative <= rtol."""
    g = got.astype(np.float64)
    r = ref.astype(np.float64)
    assert np.isfinite(g).all(), f"{what}: non-finite output"
    scale = max(np.sqrt((r ** 2).mean()), 1e-6)
    err = np.abs(g - r)
    bad = err > rtol * np.abs(r) + rtol * scale
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} elements off, max err {err.max():.3e} (rms {scale:.3e})"
    assert err.max() <= rtol * max(np.abs(r).max(), 1e-6) * 2, f"{what}: max-norm error {err.max():.3e}"


@pytest.fixture(scope="module")
def K():
    from nanoflow_amd import kernels
    assert torch.cuda.is_available()
    kernels.lib()
    return kernels


# ---------------------------------------------------------------- copies / sampler (bit-exact)

def test_embedding_and_keep_token_bit_exact(K, oracle):
    rng = np.random.default_rng(0)
    table = synth.normal_f16(rng, (1000, 4096))
    tok = rng.integers(0, 1000, size=77, dtype=np.int32)
    assert np.array_equal(host(K.embedding(dev(tok), dev(table))), oracle.embedding(tok, table))
    x = synth.normal_f16(rng, (77, 4096))
    indptr = np.concatenate([[0], np.sort(rng.choice(np.arange(1, 77), 9, replace=False)), [77]]).astype(np.int32)
    got = host(K.keep_token(dev(x), dev(indptr), 10))
    assert np.array_equal(got, oracle.keep_token(x, indptr, 10))


def test_smaller_operators_of_the_reference_vocabulary(K, oracle):
    """SplitKQVOutput / SplitTensor / Transpose move data (bit-exact against the oracle, tails included);
    Activation is left * silu(right) of a [M, 2N] row, one fp16 rounding; the sleep kernel holds its stream."""
    rng = np.random.default_rng(3)
    kqv = synth.normal_f16(rng, (333, 1024 + 4096 + 1024))
    for got, want in zip(K.split_kqv(dev(kqv), 1024, 4096, 1024), oracle.split_kqv(kqv, 1024, 4096, 1024)):
        assert np.array_equal(host(got), want)
    k, q, v = K.split_kqv(dev(kqv[:, :48]), 8, 40, 0)                   # a range may be empty
    assert np.array_equal(host(k), kqv[:, :8]) and np.array_equal(host(q), kqv[:, 8:48]) and v.shape == (333, 0)
    wide = synth.normal_f16(rng, (77, 4 * 2056))
    for rank in range(4):
        assert np.array_equal(host(K.extract_rank_columns(dev(wide), 4, rank)), oracle.extract_rank_columns(wide, 4, rank))
    for rows, cols in ((2048, 4096), (70, 131), (1, 513), (300, 8)):
        x = synth.normal_f16(rng, (rows, cols))
        assert np.array_equal(host(K.transpose(dev(x))), oracle.transpose(x)), (rows, cols)
    gu = synth.normal_f16(rng, (257, 2 * 14336), 2.0)
    assert_close(host(K.silu_mul(dev(gu))), oracle.activation_silu_mul(gu), what="activation")
    z = gu.copy()
    z[:, 14336:] = 0                                                     # silu is taken of the right half
    assert not host(K.silu_mul(dev(z))).any()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    K.sleep_us(10)
    start.record()
    K.sleep_us(2000)
    stop.record()
    torch.cuda.synchronize()
    assert 1.9 <= start.elapsed_time(stop) < 50.0
    with pytest.raises(K.NanoflowKernelError):
        K.sleep_us(2_000_000)                                            # bounded: at most a second
    with pytest.raises(K.NanoflowKernelError):
        K.split_kqv(dev(kqv[:, :44]), 8, 32, 4)                          # widths in 16-byte chunks


def test_smaller_operator_wrappers_run_as_a_schedule_drives_them():
    """The C++ wrapper classes (SplitKQVOutput, SplitTensor, Activation, Transpose, CopyTensor,
    SleepWrapper) through init / config / setStream / run, each result against host loops: the checker
    program built with the libraries."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "nanoflow_amd", "test_other_wrappers")
    assert os.path.exists(exe), "nanoflow_amd/test_other_wrappers is built by make -C nanoflow_amd/csrc"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count(" ok ") == 6 and "WRONG" not in r.stdout


def test_embedding_empty_batch(K):
    table = dev(np.zeros((4, 64), np.float16))
    out = K.embedding(torch.zeros(0, dtype=torch.int32, device="cuda"), table)
    assert out.shape == (0, 64)


def test_argmax_matches_reference_tie_order(K, oracle):
    rng = np.random.default_rng(1)
    x = synth.normal_f16(rng, (9, 128256))
    x[1, [7, 1031, 100000]] = 9.0            # ties across scanner slots
    x[2, [512, 256, 768]] = 9.0
    x[3, :] = -20000.0                       # nothing above the -10000 start
    x[4, :] = np.float16(-1.5)               # all equal
    x[5, 128255] = 11.0                      # last column
    x[6, ::1024] = 8.0                       # same slot, many times
    want_i, want_v = oracle.argmax(x)
    got_i, got_v = K.argmax(dev(x))
    assert np.array_equal(host(got_i), want_i)
    assert np.array_equal(host(got_v), want_v)


# ---------------------------------------------------------------- RMSNorm

@pytest.mark.parametrize("rows,H", [(1, 4096), (64, 4096), (7, 256), (3, 8192)])
def test_rmsnorm(K, oracle, rows, H):
    rng = np.random.default_rng(2)
    x = synth.normal_f16(rng, (rows, H), 2.0)
    w = synth.normal_f16(rng, (H,), 0.02, 1.0)
    assert_close(host(K.rmsnorm(dev(x), dev(w), 1e-5)), oracle.rmsnorm(x, w, 1e-5), what="rmsnorm")


# ---------------------------------------------------------------- GEMM family

GEMM_SHAPES = [
    (64, 6144, 4096),     # config-1 QKV (short-M tile)
    (64, 4096, 14336),    # config-1 down projection, long K
    (1, 256, 64),         # single row
    (33, 136, 200),       # ragged M, N, K (K % 8 == 0 only)
    (130, 384, 256),      # 128-row tiles with an M tail
    (257, 512, 128),      # M tail of one row
    (384, 4096, 4096),    # nano-batch O projection
    (1408, 6144, 512),    # 256x256 tiles with an M tail, XCD-remapped grid
    (2048, 6144, 256),    # 192 tiles of 256x256: three quarters of a round (the QKV projection of a full batch)
    (1930, 5000, 264),    # the same with M, N and K tails
    (2048, 10240, 136),   # 320 tiles of 256x256: one round, then 64 tiles as two 128-row halves each
    (1950, 10200, 72),    # the same with M, N and K tails
    (267, 1160, 520),     # a few hundred rows (the KV-bound 70B serving regime), N and K tails
]


@pytest.mark.parametrize("M,N,K_", GEMM_SHAPES)
def test_gemm_plain_and_residual(K, oracle, M, N, K_):
    rng = np.random.default_rng(3)
    A = synth.normal_f16(rng, (M, K_))
    B = synth.normal_f16(rng, (K_, N), 0.02)
    Cm = synth.normal_f16(rng, (M, N))
    assert_close(host(K.gemm(dev(A), dev(B))), oracle.gemm(A, B), what="gemm beta=0")
    assert_close(host(K.gemm(dev(A), dev(B), dev(Cm), alpha=1.0, beta=1.0)),
                 oracle.gemm(A, B, Cm, 1.0, 1.0), what="gemm beta=1")


@pytest.mark.parametrize("M", [128, 768])
def test_gemm_at_the_lm_head_shape(K, oracle, M):
    """The LM head as the pipelines launch it (pipeline_local.cu:305-307,819-820): sampled rows padded
    to 128 against the [4096, 128256] transposed lm_head, beta = 0.  1.05 GB of weights, 501 column
    tiles of 256 (the last one 64 columns wide), 32-bit buffer offsets up to 1.05e9.  128 rows are
    checked against the oracle in full; 768 rows against the oracle on column bands at the start, in
    the middle and over the ragged last tile, and in full against fp32 PyTorch on the device."""
    N, K_ = 128256, 4096
    rng = np.random.default_rng(9)
    A = synth.normal_f16(rng, (M, K_))
    g = torch.Generator(device="cuda").manual_seed(10)
    Bd = torch.empty((K_, N), dtype=torch.float16, device="cuda").normal_(0, 0.02, generator=g)
    print(f"LM head GEMM M={M}", flush=True)
    got_d = K.gemm(dev(A), Bd)
    got = host(got_d)
    assert got.shape == (M, N)
    if M <= 128:
        B = host(Bd)
        assert_close(got, oracle.gemm(A, B), what="LM head gemm")
    else:
        for lo, hi in ((0, 512), (64000, 64512), (127744, N)):
            Bb = np.ascontiguousarray(host(Bd[:, lo:hi]))
            assert_close(got[:, lo:hi], oracle.gemm(A, Bb), what=f"LM head gemm columns {lo}:{hi}")
    ref32 = dev(A).float() @ Bd.float()
    err = (got_d.float() - ref32).abs().max().item()
    assert err <= RTOL * ref32.abs().max().item() * 2, err
    del ref32


def test_gemm_alpha_beta_and_in_place_residual(K, oracle):
    rng = np.random.default_rng(4)
    A = synth.normal_f16(rng, (96, 256))
    B = synth.normal_f16(rng, (256, 264), 0.05)
    Cm = synth.normal_f16(rng, (96, 264))
    want = oracle.gemm(A, B, Cm, 0.5, -2.0)
    d = dev(Cm)
    K.gemm(dev(A), dev(B), d, alpha=0.5, beta=-2.0, out=d)     # C aliases D
    assert_close(host(d), want, what="gemm in place")


def test_gemm_column_major_weights(K, oracle):
    rng = np.random.default_rng(5)
    for (M, N, K_) in [(64, 512, 256), (300, 384, 320), (1930, 5000, 264), (1950, 10200, 72)]:
        A = synth.normal_f16(rng, (M, K_))
        Bt = synth.normal_f16(rng, (N, K_), 0.05)
        assert_close(host(K.gemm(dev(A), dev(Bt), b_col_major=True)),
                     oracle.gemm(A, Bt, b_col_major=True), what="gemm col-major B")


@pytest.mark.parametrize("M,N,K_", [(64, 6144, 512), (33, 136, 200), (257, 512, 128), (1408, 6144, 256),
                                    (2048, 10240, 128), (1930, 5000, 264)])
def test_gemm_with_bias_row_equals_gemm_with_replicated_bias(K, oracle, M, N, K_):
    """The QKV projection of the bias pipelines: the reference adds the bias as a C operand holding
    one copy of it per row (pipeline.cu:1048-1058); reading the one row in the epilogue must give
    the same bits as that, and agree with the oracle."""
    rng = np.random.default_rng(7)
    A = synth.normal_f16(rng, (M, K_))
    B = synth.normal_f16(rng, (K_, N), 0.02)
    bias = synth.normal_f16(rng, (N,))
    rep = np.ascontiguousarray(np.broadcast_to(bias, (M, N)))
    got = host(K.gemm(dev(A), dev(B), bias=dev(bias), alpha=1.0, beta=1.0))
    assert np.array_equal(got, host(K.gemm(dev(A), dev(B), dev(rep), alpha=1.0, beta=1.0)))
    assert_close(got, oracle.gemm(A, B, rep, 1.0, 1.0), what="gemm + bias row")
    got = host(K.gemm(dev(A), dev(B.T.copy()), bias=dev(bias), alpha=0.5, beta=-1.5, b_col_major=True))
    assert_close(got, oracle.gemm(A, B, rep, 0.5, -1.5), what="gemm + bias row, col-major B")


@pytest.mark.parametrize("M,N,K_", [(16, 6144, 4096), (64, 4096, 14336), (128, 4096, 4096), (200, 6144, 4096),
                                    (64, 1160, 2056), (1, 1024, 1024), (256, 2048, 8200),
                                    (267, 4096, 12288), (300, 1160, 4112), (320, 6144, 4096),   # one 320-row tile
                                    (421, 1160, 12304), (512, 2048, 14336)])                    # 256-row tiles
def test_gemm_split_over_k_matches_oracle(K, oracle, M, N, K_):
    """Few rows against a narrow N: the launch is split over K into shares whose fp32 sums meet in a
    workspace.  Same tolerance as the unsplit kernel; residual operand, column-major weights and
    the no-workspace fallback included."""
    from nanoflow_amd import kernels
    rng = np.random.default_rng(M + N)
    A = synth.normal_f16(rng, (M, K_))
    B = synth.normal_f16(rng, (K_, N), 0.02)
    Cm = synth.normal_f16(rng, (M, N))
    got, need = K.gemm_ws(dev(A), dev(B))
    assert need > 0 and need % (M * N * 4) == 0 and need // (M * N * 4) >= 2, "this shape is meant to be split"
    assert_close(host(got), oracle.gemm(A, B), what="split-K gemm beta=0")
    got, _ = K.gemm_ws(dev(A), dev(B), dev(Cm), alpha=0.5, beta=1.0)
    assert_close(host(got), oracle.gemm(A, B, Cm, 0.5, 1.0), what="split-K gemm beta=1")
    d = dev(Cm)
    K.gemm_ws(dev(A), dev(B), d, alpha=1.0, beta=1.0, out=d)            # C aliases D (the residual stream)
    assert_close(host(d), oracle.gemm(A, B, Cm, 1.0, 1.0), what="split-K gemm in place")
    got, _ = K.gemm_ws(dev(A), dev(np.ascontiguousarray(B.T)), b_col_major=True)
    assert_close(host(got), oracle.gemm(A, B), what="split-K gemm col-major B")
    bias = synth.normal_f16(rng, (N,))
    rep = np.ascontiguousarray(np.broadcast_to(bias, (M, N)))
    got, _ = K.gemm_ws(dev(A), dev(B), bias=dev(bias), alpha=1.0, beta=1.0)
    assert np.array_equal(host(got), host(K.gemm_ws(dev(A), dev(B), dev(rep), alpha=1.0, beta=1.0)[0]))   # bias row = replicated C
    # a workspace that is too small: the unsplit kernel, bit for bit
    short, _ = K.gemm_ws(dev(A), dev(B), workspace=torch.empty(16, dtype=torch.uint8, device="cuda"))
    assert np.array_equal(host(short), host(K.gemm(dev(A), dev(B))))


def test_gemm_with_workspace_is_the_plain_kernel_for_large_shapes(K):
    from nanoflow_amd import kernels
    rng = np.random.default_rng(8)
    for M, N, K_ in [(2048, 6144, 256), (300, 4096, 512), (64, 14336, 512), (64, 4096, 512), (520, 4096, 2048)]:
        A = synth.normal_f16(rng, (M, K_))
        B = synth.normal_f16(rng, (K_, N), 0.02)
        got, need = K.gemm_ws(dev(A), dev(B))
        assert need == 0, (M, N, K_)
        assert np.array_equal(host(got), host(K.gemm(dev(A), dev(B))))


def test_gemm_identity_is_exact(K):
    rng = np.random.default_rng(6)
    A = synth.normal_f16(rng, (70, 128))
    I = np.eye(128, dtype=np.float16)
    assert np.array_equal(host(K.gemm(dev(A), dev(I))), A)


@pytest.mark.parametrize("M,N,K_", [(64, 14336, 4096), (5, 136, 72), (200, 512, 256), (640, 2048, 512),
                                    (2048, 14336, 128),    # 3.5 rounds of 256-row tiles: two tile heights in one launch
                                    (1992, 14328, 200),    # the same with M, N and K tails
                                    (267, 1160, 264),      # a few hundred rows, N and K tails
                                    (267, 24584, 328),     # 257 .. 320 rows against 193 column panels: the
                                    (320, 24576, 128),     # 320-row tile on eight wavefronts (N and K tails; exact fit)
                                    (257, 28672, 72)])
def test_dual_swiglu(K, oracle, M, N, K_):
    rng = np.random.default_rng(7)
    A = synth.normal_f16(rng, (M, K_))
    Bg = synth.normal_f16(rng, (K_, N), 0.04)
    Bu = synth.normal_f16(rng, (K_, N), 0.04)
    assert_close(host(K.dual_swiglu(dev(A), dev(Bg), dev(Bu))), oracle.dual_swiglu(A, Bg, Bu),
                 what="dual swiglu")


@pytest.mark.parametrize("M,N,K_", [(16, 14336, 4096), (64, 1160, 2056), (128, 14336, 1024), (200, 2048, 4096),
                                    (300, 14336, 1024), (267, 1160, 2056)])    # the 320-row tile, split
def test_dual_swiglu_split_over_k_matches_oracle(K, oracle, M, N, K_):
    """Few rows: both products of the gate/up pair are split over K, summed in fp32, rounded to fp16 and
    put through SiLU-mul by the reduction.  Twice the fp16 tolerance, as for the bf16 and fp8 pairs: a
    product on an fp16 rounding boundary may round the other way than in the oracle."""
    rng = np.random.default_rng(M + N)
    A = synth.normal_f16(rng, (M, K_))
    Bg = synth.normal_f16(rng, (K_, N), 0.02)
    Bu = synth.normal_f16(rng, (K_, N), 0.02)
    got, need = K.dual_swiglu_ws(dev(A), dev(Bg), dev(Bu))
    assert need > 0 and need % (2 * M * N * 4) == 0 and need // (2 * M * N * 4) >= 2, "this shape is meant to be split"
    assert_close(host(got), oracle.dual_swiglu(A, Bg, Bu), 2 * RTOL, what="split-K dual swiglu")
    assert not np.array_equal(host(got), host(K.dual_swiglu_ws(dev(A), dev(Bu), dev(Bg))[0]))     # gate is the first
    short, _ = K.dual_swiglu_ws(dev(A), dev(Bg), dev(Bu), workspace=torch.empty(16, dtype=torch.uint8, device="cuda"))
    assert np.array_equal(host(short), host(K.dual_swiglu(dev(A), dev(Bg), dev(Bu))))
    _, need = K.dual_swiglu_ws(dev(A[:, :512]), dev(Bg[:512]), dev(Bu[:512]))                     # K < 1024: not split
    assert need == 0


@pytest.mark.parametrize("b_col", [False, True])
@pytest.mark.parametrize("M,N,K_", [(2048, 4096, 14336), (1500, 4088, 8200)])
def test_gemm_dense_rows_split_in_two_over_a_long_contraction(K, oracle, M, N, K_, b_col):
    """More than 512 rows whose 256 x 256 tiles fill half the chip or less against K >= 8192 (the 8B down
    projection) run as two shares of K when the caller brings the workspace: against the oracle, with
    the residual operand; without the workspace the unsplit launch runs."""
    rng = np.random.default_rng(M + K_)
    A = synth.normal_f16(rng, (M, K_))
    B = synth.normal_f16(rng, (K_, N), 0.02)
    Cm = synth.normal_f16(rng, (M, N))
    dB = dev(np.ascontiguousarray(B.T)) if b_col else dev(B)
    ref = oracle.gemm(A, B, Cm, 1.0, 1.0)
    got, need = K.gemm_ws(dev(A), dB, dev(Cm), 1.0, 1.0, b_col_major=b_col)
    assert need == 2 * M * N * 4, "this shape is meant to be split in two"
    assert_close(host(got), ref, what="dense split-K")
    plain = K.gemm(dev(A), dB, dev(Cm), 1.0, 1.0, b_col_major=b_col)
    assert_close(host(plain), ref, what="unsplit")
    short, _ = K.gemm_ws(dev(A), dB, dev(Cm), 1.0, 1.0, b_col_major=b_col, workspace=torch.empty(16, dtype=torch.uint8, device="cuda"))
    assert np.array_equal(host(short), host(plain))


@pytest.mark.parametrize("b_col", [False, True])
@pytest.mark.parametrize("M,N,K_", [(640, 1160, 264), (513, 6144, 512), (37, 520, 200), (2048, 4096, 448)])
def test_gemm_on_a_caller_chosen_tile_and_split(K, oracle, M, N, K_, b_col):
    """nf_gemm_f16_tiled -- what a GEMM tag's cta_m x cta_n and split_k select -- on every tile of the
    menu, unsplit and cut into 2 and 3 shares of K, both weight layouts, with M / N / K tails, the
    residual operand and the bias row: against the oracle.  A tile that is not in the menu runs on
    the closest one; a split without its workspace is refused."""
    from nanoflow_amd import kernels
    rng = np.random.default_rng(M + N + K_)
    A = synth.normal_f16(rng, (M, K_))
    B = synth.normal_f16(rng, (K_, N), 0.05)
    Cm = synth.normal_f16(rng, (M, N))
    bias = synth.normal_f16(rng, (N,))
    dB = dev(np.ascontiguousarray(B.T)) if b_col else dev(B)
    ref = oracle.gemm(A, B, Cm, 1.0, 1.0)
    ref_bias = oracle.gemm(A, B, np.ascontiguousarray(np.broadcast_to(bias, (M, N))), 1.0, 1.0)
    menu = K.gemm_tile_menu()
    assert (256, 256, False) in menu and (128, 256, False) in menu and (256, 192, True) in menu and len(menu) >= 5
    for tm, tn, col_only in menu:
        for split in (1, 2, 3):
            got = host(K.gemm_tiled(dev(A), dB, (tm, tn), split, Cmat=dev(Cm), beta=1.0, b_col_major=b_col))
            assert_close(got, ref, what=f"tile {tm}x{tn} split {split} {'[N][K]' if b_col else '[K][N]'}")
        got = host(K.gemm_tiled(dev(A), dB, (tm, tn), 2, bias=dev(bias), beta=1.0, b_col_major=b_col))
        assert_close(got, ref_bias, what=f"tile {tm}x{tn} with a bias row")
    # 100 x 100 is not in the menu: the closest entry (128 x 128) runs, with the same bits
    assert np.array_equal(host(K.gemm_tiled(dev(A), dB, (100, 100), 1, b_col_major=b_col)),
                          host(K.gemm_tiled(dev(A), dB, (128, 128), 1, b_col_major=b_col)))
    assert K.lib().nf_gemm_tiled_workspace_bytes(M, N, K_, 1) == 0
    k_per = -(-(-(-K_ // 3)) // 64) * 64                   # a share is a whole number of 64-deep slabs
    assert K.lib().nf_gemm_tiled_workspace_bytes(M, N, K_, 3) == -(-K_ // k_per) * M * N * 4
    with pytest.raises(kernels.NanoflowKernelError, match="workspace"):
        K.gemm_tiled(dev(A), dB, (128, 128), 2, b_col_major=b_col, workspace=torch.empty(16, dtype=torch.uint8, device="cuda"))


@pytest.mark.parametrize("M,N,K_", [(5, 136, 72), (64, 14336, 256), (200, 1160, 264), (267, 24584, 328), (300, 14336, 1024),
                                    (16, 14336, 4096), (2048, 14336, 256), (1992, 14328, 200), (1792, 28672, 128)])
def test_dual_swiglu_with_k_contiguous_weights(K, oracle, M, N, K_):
    """The gate/up pair on [N][K] weights (the layout a GEMM tag calls ColumnMajor for B), plain and
    split over K: against the oracle, and bit for bit what the [K][N] path gives for the same
    matrices (the same products summed in the same order; only the way the fragments reach the
    registers differs)."""
    rng = np.random.default_rng(M + N + K_)
    A = synth.normal_f16(rng, (M, K_))
    Bg = synth.normal_f16(rng, (K_, N), 0.03)
    Bu = synth.normal_f16(rng, (K_, N), 0.03)
    gt, ut = dev(np.ascontiguousarray(Bg.T)), dev(np.ascontiguousarray(Bu.T))
    ref = oracle.dual_swiglu(A, Bg, Bu)
    got = host(K.dual_swiglu(dev(A), gt, ut, b_col_major=True))
    assert_close(got, ref, what="dual swiglu, [N][K] weights")
    assert np.array_equal(got, host(K.dual_swiglu(dev(A), dev(Bg), dev(Bu))))
    got_ws, need = K.dual_swiglu_ws(dev(A), gt, ut, b_col_major=True)
    row_ws, need_row = K.dual_swiglu_ws(dev(A), dev(Bg), dev(Bu))
    assert need == need_row
    assert_close(host(got_ws), ref, 2 * RTOL if need else RTOL, what="dual swiglu with workspace, [N][K] weights")
    assert np.array_equal(host(got_ws), host(row_ws))
    assert not np.array_equal(got, host(K.dual_swiglu(dev(A), ut, gt, b_col_major=True)))     # gate is the first


def test_dual_known_answer_inputs(K, oracle):
    # inputs of the reference's dual-GEMM test program (all operands (j+k)/2560, 128^3)
    j, k = np.meshgrid(np.arange(128), np.arange(128), indexing="ij")
    X = ((j + k).astype(np.float32) / 20 / 128).astype(np.float16)
    assert_close(host(K.dual_swiglu(dev(X), dev(X), dev(X))), oracle.dual_swiglu(X, X, X), what="dual KAT")


# ---------------------------------------------------------------- bf16 variants of the GEMM family

BF16_RTOL = 8e-3   # one bf16 ulp (2^-8 = 3.9e-3 relative) either side of the float64 closed form


def _bf16_dev(bits):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).cuda().view(torch.bfloat16)


def _bf16_host(t):
    torch.cuda.synchronize()
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("M,N,K_", [(64, 512, 256), (33, 136, 200), (300, 384, 320), (2048, 6144, 256), (1408, 6144, 512),
                                    (2048, 10240, 72)])
def test_gemm_bf16(K, oracle, M, N, K_):
    rng = np.random.default_rng(31)
    A = oracle.float_to_bf16(rng.standard_normal((M, K_), dtype=np.float32))
    B = oracle.float_to_bf16(rng.standard_normal((K_, N), dtype=np.float32) * 0.05)
    Cm = oracle.float_to_bf16(rng.standard_normal((M, N), dtype=np.float32))
    got = _bf16_host(K.gemm(_bf16_dev(A), _bf16_dev(B)))
    assert_close(oracle.bf16_to_float(got), oracle.bf16_to_float(oracle.gemm_bf16(A, B)), BF16_RTOL, "gemm bf16")
    got = _bf16_host(K.gemm(_bf16_dev(A), _bf16_dev(B), _bf16_dev(Cm), alpha=0.5, beta=1.0))
    assert_close(oracle.bf16_to_float(got), oracle.bf16_to_float(oracle.gemm_bf16(A, B, Cm, 0.5, 1.0)), BF16_RTOL,
                 "gemm bf16 beta=1")
    Bt = np.ascontiguousarray(B.T)
    got_t = _bf16_host(K.gemm(_bf16_dev(A), _bf16_dev(Bt), b_col_major=True))
    assert_close(oracle.bf16_to_float(got_t), oracle.bf16_to_float(oracle.gemm_bf16(A, B)), BF16_RTOL, "gemm bf16 col-major B")


def test_gemm_bf16_exact_on_small_integers(K, oracle):
    rng = np.random.default_rng(32)
    A = rng.integers(-4, 5, (130, 64)).astype(np.float32)
    B = rng.integers(-4, 5, (64, 264)).astype(np.float32)
    got = oracle.bf16_to_float(_bf16_host(K.gemm(_bf16_dev(oracle.float_to_bf16(A)), _bf16_dev(oracle.float_to_bf16(B)))))
    assert np.array_equal(got, oracle.bf16_to_float(oracle.float_to_bf16(A @ B)))


@pytest.mark.parametrize("M,N,K_", [(5, 136, 72), (200, 512, 256), (2048, 14336, 128)])
def test_dual_swiglu_bf16(K, oracle, M, N, K_):
    rng = np.random.default_rng(33)
    A = oracle.float_to_bf16(rng.standard_normal((M, K_), dtype=np.float32))
    Bg = oracle.float_to_bf16(rng.standard_normal((K_, N), dtype=np.float32) * 0.04)
    Bu = oracle.float_to_bf16(rng.standard_normal((K_, N), dtype=np.float32) * 0.04)
    got = _bf16_host(K.dual_swiglu(_bf16_dev(A), _bf16_dev(Bg), _bf16_dev(Bu)))
    # the two products are rounded to bf16 before SiLU-mul: a product that lands on the other side
    # of a rounding boundary moves the result by up to two ulps
    assert_close(oracle.bf16_to_float(got), oracle.bf16_to_float(oracle.dual_swiglu_bf16(A, Bg, Bu)), 2 * BF16_RTOL,
                 "dual swiglu bf16")


# ---------------------------------------------------------------- KV pages to and from a staging buffer

def test_move_kv_pages_is_bit_exact_and_round_trips(K, oracle):
    rng = np.random.default_rng(17)
    shape = synth.LLAMA3_8B                                     # 64 KB pages (K and V of 16 tokens, 8 heads)
    b = synth.make_batch([1023, 17, 300, 64, 1], [(0, 33)], vocab=10, seed=4, extra_pages=7)
    pool = synth.make_kv_pool(b.num_pages, shape, rng)
    n_idx = b.kv_indices.shape[0]
    listed = np.array([4, 0, 5, 2], np.int32)                   # out of order, not all requests
    staging_ref = np.zeros((n_idx,) + pool.shape[1:], np.float16)
    oracle.move_kv_pages(listed, b.kv_indptr, b.kv_indices, staging_ref, pool, to_pool=False)
    staging = torch.zeros(staging_ref.shape, dtype=torch.float16, device="cuda")
    d_idx, d_indptr, d_indices, d_pool = dev(listed), dev(b.kv_indptr), dev(b.kv_indices), dev(pool)
    K.move_kv_pages(d_idx, d_indptr, d_indices, staging, d_pool, to_pool=False)
    assert np.array_equal(host(staging), staging_ref)
    assert np.array_equal(host(d_pool), pool)                   # the pool is only read
    # back into a pool whose page table has been re-drawn (the requests own other pages now)
    perm = rng.permutation(b.num_pages).astype(np.int32)
    indices2 = perm[b.kv_indices]
    pool2_ref = np.zeros_like(pool)
    oracle.move_kv_pages(listed, b.kv_indptr, indices2, staging_ref, pool2_ref, to_pool=True)
    d_pool2 = torch.zeros_like(d_pool)
    K.move_kv_pages(d_idx, d_indptr, dev(indices2), staging, d_pool2, to_pool=True)
    assert np.array_equal(host(d_pool2), pool2_ref)
    for r in listed:                                            # every listed request got its pages back
        for j in range(b.kv_indptr[r], b.kv_indptr[r + 1]):
            assert np.array_equal(pool2_ref[indices2[j]], pool[b.kv_indices[j]])
    # an empty list is a no-op
    K.move_kv_pages(dev(np.zeros(0, np.int32)), d_indptr, d_indices, staging, d_pool, to_pool=True)


# ---------------------------------------------------------------- RoPE + paged append

F8_RTOL = 3e-2   # fp8 path: activations rounded to e4m3 (3 mantissa bits) on the way in


def _quantize_weights_nk(W):
    """fp32 [N,K] -> (e4m3 bytes [N,K], per-output-channel fp32 scales), scale = amax / 448."""
    sc = (np.abs(W).max(axis=1) / 448.0).astype(np.float32)
    q = torch.from_numpy(W / sc[:, None]).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    return q, sc


# row lengths on both sides of what the quantiser keeps in registers (8192 and 32768 halves)
@pytest.mark.parametrize("M,K_", [(1, 16), (5, 4096), (33, 144), (64, 28672), (7, 8192), (6, 8208), (9, 14336),
                                  (4, 32768), (3, 32784), (3, 40960)])
def test_quantize_rows_e4m3_bit_exact(K, oracle, M, K_):
    rng = np.random.default_rng(M * 7 + K_)
    X = (rng.normal(0, 1, (M, K_)) * rng.uniform(0.01, 20, (M, 1))).astype(np.float16)
    if M > 2:
        X[2] = 0                                  # all-zero row: scale 1, codes 0
        X[1, ::3] = 0
    q_ref, s_ref = oracle.quantize_rows_e4m3(X)
    q, s = K.quantize_rows_e4m3(dev(X))
    assert np.array_equal(host(s), s_ref)
    assert np.array_equal(host(q), q_ref)


@pytest.mark.parametrize("M,N,K_", [(1, 8, 16), (37, 136, 144), (130, 520, 1040), (300, 264, 4096),
                                     (64, 1024, 512), (256, 256, 128), (512, 2048, 384)])
def test_gemm_f8_exact_products(K, oracle, M, N, K_):
    """fp8 x fp8 with fp32 accumulation: the products are exact, so the result matches the
    oracle (double accumulation) to fp16 rounding."""
    rng = np.random.default_rng(M + N + K_)
    fin = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], np.uint8)
    Aq, Bq = rng.choice(fin, (M, K_)), rng.choice(fin, (N, K_))
    # keep magnitudes moderate so that the sum does not ride on a few 448*448 products
    Aq, Bq = (Aq & 0xBF).astype(np.uint8), (Bq & 0xBF).astype(np.uint8)
    sa = rng.uniform(0.5, 2, M).astype(np.float32)
    sb = rng.uniform(0.5, 2, N).astype(np.float32)
    Cm = rng.normal(0, 1, (M, N)).astype(np.float16)
    for alpha, beta in ((1.0, 0.0), (0.5, 1.0)):
        ref = oracle.gemm_f8f8(Aq, sa, Bq, sb, Cm if beta else None, alpha=alpha, beta=beta)
        got = K.gemm_f8(dev(Aq), dev(sa), dev(Bq), dev(sb), dev(Cm) if beta else None, alpha=alpha, beta=beta)
        assert_close(host(got), ref, what=f"gemm_f8 {M}x{N}x{K_} a={alpha} b={beta}")


@pytest.mark.parametrize("M,N,K_", [(48, 256, 512), (200, 1024, 4096), (1, 4096, 4096)])
def test_gemm_f8w_within_fp8_tolerance_of_dequantised_reference(K, oracle, M, N, K_):
    rng = np.random.default_rng(N + K_)
    A = rng.normal(0, 1, (M, K_)).astype(np.float16)
    W = rng.normal(0, 0.02, (N, K_)).astype(np.float32)
    Wq, sc = _quantize_weights_nk(W)
    Cm = rng.normal(0, 1, (M, N)).astype(np.float16)
    ref = oracle.gemm_f8w(A, np.ascontiguousarray(Wq.T), sc, Cm, alpha=1.0, beta=1.0)   # oracle takes [K,N]
    got = host(K.gemm_f8w(dev(A), dev(Wq), dev(sc), dev(Cm), alpha=1.0, beta=1.0))
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    assert np.isfinite(got).all()
    assert err.max() <= F8_RTOL * np.abs(ref).max(), (err.max(), np.abs(ref).max())
    # and the two-step form gives the same bits as the fused entry point
    q, s = K.quantize_rows_e4m3(dev(A))
    two = host(K.gemm_f8(q, s, dev(Wq), dev(sc), dev(Cm), alpha=1.0, beta=1.0))
    assert np.array_equal(two, got)


@pytest.mark.parametrize("Kd,N", [(16, 8), (144, 136), (512, 6144), (4096, 1000), (1040, 72)])
def test_quantize_weight_e4m3_is_bit_exact(K, oracle, Kd, N):
    rng = np.random.default_rng(Kd + N)
    W = (rng.normal(0, 0.02, (Kd, N)) * rng.uniform(0.1, 10, (1, N))).astype(np.float16)
    if N > 3:
        W[:, 3] = 0                                # all-zero output channel: scale 1, codes 0
    q_ref, s_ref = oracle.quantize_weight_e4m3(W)
    q, s = K.quantize_weight_e4m3(dev(W))
    assert np.array_equal(host(s), s_ref)
    assert np.array_equal(host(q), q_ref)


@pytest.mark.parametrize("M,N,K_", [(1, 8, 16), (37, 136, 144), (64, 512, 256), (130, 520, 1040), (300, 264, 4096),
                                     (256, 24576, 128), (1930, 3200, 272), (2048, 3072, 128)])
def test_dual_swiglu_f8_matches_oracle(K, oracle, M, N, K_):
    """The fp8 gate/up pair: products exact, fp32 accumulation, both rounded to fp16 before
    SiLU-mul.  A product that lands on an fp16 rounding boundary may round the other way than the
    oracle's double-precision sum, which moves g or u by a whole fp16 step (2^-10 relative) and
    the output with it: bounded at twice the fp16 GEMM tolerance, as for the bf16 pair."""
    rng = np.random.default_rng(M + N + K_)
    fin = np.array([c for c in range(256) if (c & 0x7F) < 0x50], np.uint8)       # magnitudes below 8
    Aq, Gq, Uq = rng.choice(fin, (M, K_)), rng.choice(fin, (N, K_)), rng.choice(fin, (N, K_))
    sa = rng.uniform(0.05, 0.2, M).astype(np.float32)
    sg = (rng.uniform(0.5, 2, N) / np.sqrt(K_)).astype(np.float32)
    su = (rng.uniform(0.5, 2, N) / np.sqrt(K_)).astype(np.float32)
    ref = oracle.dual_swiglu_f8f8(Aq, sa, Gq, sg, Uq, su)
    got = host(K.dual_swiglu_f8(dev(Aq), dev(sa), dev(Gq), dev(sg), dev(Uq), dev(su)))
    assert_close(got, ref, 2 * RTOL, what=f"dual_swiglu_f8 {M}x{N}x{K_}")
    # swapping gate and up must change the result (silu is taken of the first)
    if M * N > 64:
        assert not np.array_equal(got, host(K.dual_swiglu_f8(dev(Aq), dev(sa), dev(Uq), dev(su), dev(Gq), dev(sg))))


def test_dual_swiglu_f8w_is_quantise_then_dual(K, oracle):
    rng = np.random.default_rng(11)
    M, N, K_ = 200, 1024, 4096
    A = rng.normal(0, 1, (M, K_)).astype(np.float16)
    Wg = rng.normal(0, 0.02, (K_, N)).astype(np.float16)
    Wu = rng.normal(0, 0.02, (K_, N)).astype(np.float16)
    Gq, sg = K.quantize_weight_e4m3(dev(Wg))
    Uq, su = K.quantize_weight_e4m3(dev(Wu))
    got = host(K.dual_swiglu_f8w(dev(A), Gq, sg, Uq, su))
    q, s = K.quantize_rows_e4m3(dev(A))
    assert np.array_equal(got, host(K.dual_swiglu_f8(q, s, Gq, sg, Uq, su)))
    # against fp16 activations on the dequantised weights: the output is a product of two GEMM
    # results that are each within the fp8 tolerance, so it is held to twice that
    g = oracle.gemm_f8w(A, np.ascontiguousarray(host(Gq).T), host(sg))
    u = oracle.gemm_f8w(A, np.ascontiguousarray(host(Uq).T), host(su))
    ref = oracle.silu_mul(g, u)
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    assert err.max() <= 2 * F8_RTOL * np.abs(ref).max(), (err.max(), np.abs(ref).max())


@pytest.mark.parametrize("M,N,K_", [(16, 6144, 4096), (64, 4096, 14336), (128, 4096, 4096), (200, 1160, 4112)])
def test_gemm_f8w_split_over_k_matches_the_unsplit_kernel_and_the_oracle(K, oracle, M, N, K_):
    """Few rows: nf_gemm_f8w_f16 splits the contraction when its workspace has room for the sums.
    Same quantised operands as the unsplit path (the row quantiser is bit-exact), fp32 sums taken
    share by share: the fp16 tolerance against the oracle's double-precision sum."""
    from nanoflow_amd import kernels
    rng = np.random.default_rng(M + N)
    A = rng.normal(0, 1, (M, K_)).astype(np.float16)
    W = rng.normal(0, 0.02, (K_, N)).astype(np.float16)
    Cm = rng.normal(0, 1, (M, N)).astype(np.float16)
    Wq, sc = K.quantize_weight_e4m3(dev(W))
    l = kernels.lib()
    assert l.nf_gemm_f8w_split_workspace_bytes(M, N, K_) > l.nf_gemm_f8w_workspace_bytes(M, K_), "meant to be split"
    got = host(K.gemm_f8w(dev(A), Wq, sc, dev(Cm), alpha=0.5, beta=1.0))
    q, s = oracle.quantize_rows_e4m3(A)
    ref = oracle.gemm_f8f8(q, s, host(Wq), host(sc), Cm, alpha=0.5, beta=1.0)
    assert_close(got, ref, what="split-K fp8 gemm")
    small = torch.empty(l.nf_gemm_f8w_workspace_bytes(M, K_), dtype=torch.uint8, device="cuda")   # no room: unsplit
    unsplit = host(K.gemm_f8w(dev(A), Wq, sc, dev(Cm), alpha=0.5, beta=1.0, workspace=small))
    assert_close(unsplit, ref, what="unsplit fp8 gemm")
    assert_close(got, unsplit, what="split vs unsplit")


@pytest.mark.parametrize("M,N,K_", [(16, 14336, 4096), (64, 1160, 4112), (128, 14336, 2048)])
def test_dual_swiglu_f8w_split_over_k_matches_oracle(K, oracle, M, N, K_):
    from nanoflow_amd import kernels
    rng = np.random.default_rng(M + N + 1)
    A = rng.normal(0, 1, (M, K_)).astype(np.float16)
    Wg = rng.normal(0, 0.02, (K_, N)).astype(np.float16)
    Wu = rng.normal(0, 0.02, (K_, N)).astype(np.float16)
    Gq, sg = K.quantize_weight_e4m3(dev(Wg))
    Uq, su = K.quantize_weight_e4m3(dev(Wu))
    l = kernels.lib()
    assert l.nf_dual_swiglu_f8w_split_workspace_bytes(M, N, K_) > l.nf_gemm_f8w_workspace_bytes(M, K_), "meant to be split"
    got = host(K.dual_swiglu_f8w(dev(A), Gq, sg, Uq, su))
    q, s = oracle.quantize_rows_e4m3(A)
    ref = oracle.dual_swiglu_f8f8(q, s, host(Gq), host(sg), host(Uq), host(su))
    assert_close(got, ref, 2 * RTOL, what="split-K fp8 gate/up pair")       # two fp16 roundings before SiLU-mul
    small = torch.empty(l.nf_gemm_f8w_workspace_bytes(M, K_), dtype=torch.uint8, device="cuda")
    assert_close(host(K.dual_swiglu_f8w(dev(A), Gq, sg, Uq, su, workspace=small)), ref, 2 * RTOL, what="unsplit pair")


@pytest.mark.parametrize("rows,H", [(1, 16), (5, 4096), (130, 8192), (33, 1040), (64, 2048)])
def test_rmsnorm_quantize_is_rmsnorm_then_the_row_quantiser(K, oracle, rows, H):
    """The fused launch writes the fp16 output of nf_rmsnorm_f16 bit for bit, and the e4m3 bytes and
    row scales that nf_quantize_rows_e4m3 makes of it (the oracle's quantiser applied to the output)."""
    rng = np.random.default_rng(rows + H)
    x = (rng.normal(0, 1, (rows, H)) * rng.uniform(0.01, 30, (rows, 1))).astype(np.float16)
    if rows > 2:
        x[2] = 0                                   # an all-zero row: output 0, scale 1, codes 0
    w = (1 + rng.normal(0, 0.1, H)).astype(np.float16)
    y = K.rmsnorm(dev(x), dev(w))
    out, q, s = K.rmsnorm_quantize_e4m3(dev(x), dev(w))
    assert np.array_equal(host(out).view(np.uint16), host(y).view(np.uint16))
    q_ref, s_ref = oracle.quantize_rows_e4m3(host(y))
    assert np.array_equal(host(s), s_ref)
    assert np.array_equal(host(q), q_ref)
    assert_close(host(out), oracle.rmsnorm(x, w), what="rmsnorm in the fused launch")


def test_rmsnorm_quantize_refuses_rows_it_cannot_hold(K):
    from nanoflow_amd import kernels
    x = torch.zeros((2, 8208), dtype=torch.float16, device="cuda")
    with pytest.raises(kernels.NanoflowKernelError, match="8192"):
        K.rmsnorm_quantize_e4m3(x, torch.ones(8208, dtype=torch.float16, device="cuda"))


@pytest.mark.parametrize("M,N,K_", [(16, 6144, 4096), (200, 1160, 4112), (700, 1024, 4096)])
def test_f8q_entries_equal_the_f8w_entries_on_prequantised_rows(K, M, N, K_):
    """nf_gemm_f8q_f16 / nf_dual_swiglu_f8q_f16 take rows that are quantised already: same bits as the
    f8w entries that quantise them themselves, split over K (few rows) or not."""
    rng = np.random.default_rng(M + N + 3)
    A = dev(rng.normal(0, 1, (M, K_)).astype(np.float16))
    Cm = dev(rng.normal(0, 1, (M, N)).astype(np.float16))
    Wq, sc = K.quantize_weight_e4m3(dev(rng.normal(0, 0.02, (K_, N)).astype(np.float16)))
    Uq, su = K.quantize_weight_e4m3(dev(rng.normal(0, 0.02, (K_, N)).astype(np.float16)))
    q, s = K.quantize_rows_e4m3(A)
    assert np.array_equal(host(K.gemm_f8q(q, s, Wq, sc, Cm, alpha=0.5, beta=1.0)),
                          host(K.gemm_f8w(A, Wq, sc, Cm, alpha=0.5, beta=1.0)))
    assert np.array_equal(host(K.dual_swiglu_f8q(q, s, Wq, sc, Uq, su)), host(K.dual_swiglu_f8w(A, Wq, sc, Uq, su)))


def test_gemm_f8w_rejects_short_workspace(K):
    from nanoflow_amd import kernels
    A = torch.zeros((8, 64), dtype=torch.float16, device="cuda")
    Wq = torch.zeros((16, 64), dtype=torch.uint8, device="cuda")
    sc = torch.ones(16, dtype=torch.float32, device="cuda")
    with pytest.raises(kernels.NanoflowKernelError, match="workspace"):
        K.gemm_f8w(A, Wq, sc, workspace=torch.empty(16, dtype=torch.uint8, device="cuda"))


@pytest.mark.parametrize("Hq,Hkv,theta,scale,sa,sb", [
    (32, 8, 5e5, 1.0, 0.0, 0.0),
    (8, 2, 1e4, 1.0, 0.0, 0.0),
    (64, 8, 5e5, 8.0, 8192 / (2 * np.pi * 3), -1.0 / 3),   # Llama-3.1 smoothing
])
def test_rope_append(K, oracle, Hq, Hkv, theta, scale, sa, sb):
    rng = np.random.default_rng(8)
    d, P = 128, 16
    b = synth.make_batch(rng.integers(0, 1500, size=20), [(0, 40), (123, 17)], vocab=10, seed=3,
                         extra_pages=7)
    kqv = synth.normal_f16(rng, (b.tokens, (Hq + 2 * Hkv) * d))
    shape = synth.ModelShape(Hq=Hq, Hkv=Hkv)
    pool0 = synth.make_kv_pool(b.num_pages, shape, rng)
    pool_ref = pool0.copy()
    q_ref = oracle.rope_append(kqv, pool_ref, b.kv_indices, b.kv_indptr, b.rev_input_indptr,
                               b.per_token_offset, Hq, Hkv, d, P, scale, theta, sa, sb)
    pool_dev = dev(pool0)
    q_dev = K.rope_append(dev(kqv), pool_dev, dev(b.kv_indices), dev(b.kv_indptr),
                          dev(b.rev_input_indptr), dev(b.per_token_offset), Hq, Hkv, d, P, scale,
                          theta, sa, sb)
    pool_got = host(pool_dev)
    # index rule bit-exact: exactly the same pool slots changed, V rows bit-identical
    changed_ref = (pool_ref != pool0).any(axis=(3, 4))
    changed_got = (pool_got != pool0).any(axis=(3, 4))
    assert np.array_equal(changed_ref, changed_got)
    assert np.array_equal(pool_got[:, 1], pool_ref[:, 1])
    assert_close(pool_got[:, 0], pool_ref[:, 0], what="rope K pages")
    assert_close(host(q_dev), q_ref, what="rope Q")


# ---------------------------------------------------------------- attention

def _attn_case(K, oracle, Hq, Hkv, decode_lens, prefill, seed, num_blocks=0):
    rng = np.random.default_rng(seed)
    d, P = 128, 16
    b = synth.make_batch(decode_lens, prefill, vocab=10, seed=seed, extra_pages=3)
    shape = synth.ModelShape(Hq=Hq, Hkv=Hkv)
    pool = synth.make_kv_pool(b.num_pages, shape, rng)
    # poison the unused tail of every request's last page: results must not depend on it
    for r in range(b.req_num):
        last = b.kv_indices[b.kv_indptr[r + 1] - 1]
        pool[last, :, b.kv_last_page_len[r]:] = np.float16(np.nan)
    q = synth.normal_f16(rng, (b.tokens, Hq * d))
    nd = b.decodePrefillBorder
    ref = np.zeros_like(q)
    got = torch.zeros(q.shape, dtype=torch.float16, device="cuda")
    dq, dpool, dind = dev(q), dev(pool), dev(b.kv_indices)
    if nd:
        oracle.attention_paged(q, b.input_indptr[:nd + 1], pool, b.kv_indptr[:nd + 1], b.kv_indices,
                               b.kv_last_page_len[:nd], Hq, Hkv, d, P, causal=False, out=ref)
        K.attention_paged(dq, dev(b.input_indptr[:nd + 1]), dpool, dev(b.kv_indptr[:nd + 1]), dind,
                          dev(b.kv_last_page_len[:nd]), Hq, Hkv, causal=False, out=got, batch=nd,
                          max_qo_rows=nd, num_blocks=num_blocks)
    if b.prefillNum:
        oracle.attention_paged(q, b.input_indptr[nd:], pool, b.kv_indptr[nd:], b.kv_indices,
                               b.kv_last_page_len[nd:], Hq, Hkv, d, P, causal=True, out=ref)
        K.attention_paged(dq, dev(b.input_indptr[nd:]), dpool, dev(b.kv_indptr[nd:]), dind,
                          dev(b.kv_last_page_len[nd:]), Hq, Hkv, causal=True, out=got,
                          batch=b.prefillNum, max_qo_rows=b.tokens, num_blocks=num_blocks)
    assert_close(host(got), ref, what=f"attention Hq={Hq} Hkv={Hkv}")


@pytest.mark.parametrize("Hq,Hkv", [(32, 8), (64, 8), (8, 4), (4, 4)])
def test_attention_decode(K, oracle, Hq, Hkv):
    lens = [0, 1, 15, 16, 17, 31, 32, 33, 63, 64, 100, 127, 128, 129, 500, 1023]
    _attn_case(K, oracle, Hq, Hkv, lens, [], seed=11)


@pytest.mark.parametrize("Hq,Hkv", [(32, 8), (64, 8), (8, 4), (4, 4)])
def test_attention_decode_many_requests(K, oracle, Hq, Hkv):
    # more (request, kv head) pairs than CUs: the launch with two wavefronts per workgroup
    # (smaller batches, as above, run with four)
    lens = [int(x) for x in np.random.default_rng(16).integers(1, 260, size=72)]
    assert len(lens) * Hkv > 256
    _attn_case(K, oracle, Hq, Hkv, lens, [], seed=16)


@pytest.mark.parametrize("Hq,Hkv,n", [(32, 8, 77), (8, 8, 13), (4, 2, 139), (32, 8, 5)])
def test_attention_decode_request_counts_off_the_group_of_eight(K, oracle, Hq, Hkv, n):
    """The decode kernel orders its work items (head, request) inside groups of 8 requests and
    (request, head) past the last whole group: counts that leave a remainder, fewer than 8
    requests, and kv-head counts other than 8."""
    lens = [int(x) for x in np.random.default_rng(17).integers(1, 200, size=n)]
    _attn_case(K, oracle, Hq, Hkv, lens, [], seed=17)


@pytest.mark.parametrize("Hq,Hkv", [(32, 8), (64, 8), (8, 4), (4, 4)])
def test_attention_chunked_prefill(K, oracle, Hq, Hkv):
    _attn_case(K, oracle, Hq, Hkv, [], [(0, 1), (0, 37), (100, 64), (5, 130), (256, 3)], seed=12)


def test_attention_mixed_batch_with_capped_workgroups(K, oracle):
    # persistent-grid path: fewer workgroups than work items
    _attn_case(K, oracle, 32, 8, list(range(40, 72)), [(64, 200)], seed=13, num_blocks=24)


def test_attention_long_context_prefill(K, oracle):
    _attn_case(K, oracle, 8, 2, [], [(1900, 147)], seed=14)


def test_attention_page_permutation_invariance(K):
    rng = np.random.default_rng(15)
    Hq, Hkv, d, P = 32, 8, 128, 16
    shape = synth.ModelShape(Hq=Hq, Hkv=Hkv)
    b = synth.make_batch([300, 77, 1000], [], vocab=10, seed=15, extra_pages=9)
    pool = synth.make_kv_pool(b.num_pages, shape, rng)
    q = synth.normal_f16(rng, (3, Hq * d))
    perm = rng.permutation(b.num_pages)
    pool_p = np.empty_like(pool)
    pool_p[perm] = pool
    args = (dev(b.input_indptr), )
    o1 = K.attention_paged(dev(q), dev(b.input_indptr), dev(pool), dev(b.kv_indptr), dev(b.kv_indices),
                           dev(b.kv_last_page_len), Hq, Hkv, max_qo_rows=3)
    o2 = K.attention_paged(dev(q), dev(b.input_indptr), dev(pool_p), dev(b.kv_indptr),
                           dev(perm[b.kv_indices].astype(np.int32)), dev(b.kv_last_page_len), Hq, Hkv,
                           max_qo_rows=3)
    assert np.array_equal(host(o1), host(o2))


# ---------------------------------------------------------------- calibration micro-benchmarks

def test_calibration_loops_report_rates_this_part_can_have(K):
    """The ceilings bench.py reports its rates against: every mode runs and reports a rate and a clock
    this part can have (nothing above the published peaks), bad modes are refused.  How the modes order
    depends on clocks and the power cap, so it is recorded in the bench line, not asserted here."""
    from nanoflow_amd import kernels
    rates = {}
    for name, fp8, mode in (("zero", False, False), ("random", False, True), ("from LDS", False, 2), ("+ loads", False, 3),
                            ("16x16x32", False, 4), ("fp8", True, True), ("fp8 16x16x128", True, 4)):
        tf, mhz = K.calibrate_mfma(fp8, mode, 4000)
        rates[name] = tf
        assert np.isfinite(tf) and 300 < tf <= (5200 if fp8 else 2600), (name, tf)
        assert 800 < mhz < 2600, (name, mhz)
    print("mfma loops, TFLOP/s: " + ", ".join(f"{k} {v:.0f}" for k, v in rates.items()), flush=True)
    for bad in (5, 10, -1):
        with pytest.raises(kernels.NanoflowKernelError, match="random_operands"):
            K.calibrate_mfma(False, bad, 100)
    with pytest.raises(kernels.NanoflowKernelError, match="random_operands"):
        K.calibrate_mfma(True, 2, 100)


def test_calibration_read_streams(K):
    gbps = K.calibrate_hbm_read(2.0, 2)
    shape = synth.ModelShape()
    b = synth.config2_batch(seed=0, n_decode=128, lo=256, hi=512, prefill_chunk=16)
    nd = b.decodePrefillBorder
    pool = torch.randn(b.num_pages * 2 * shape.page_size * shape.Hkv * shape.d // 2, device="cuda").view(torch.float16)
    assert pool.numel() == b.num_pages * 2 * shape.page_size * shape.Hkv * shape.d
    kvb = int(2 * b.kv_len[:nd].astype(np.int64).sum() * shape.Hkv * shape.d * 2)
    paged = K.calibrate_paged_read(pool, dev(b.kv_indptr[:nd + 1]), dev(b.kv_indices), dev(b.kv_last_page_len[:nd]), nd,
                                   shape.Hkv, kvb, reps=5)
    print(f"read stream {gbps:.0f} GB/s, paged read of 128 requests {paged:.0f} GB/s", flush=True)
    assert 2000 < gbps < 8000 and 300 < paged < 8000
