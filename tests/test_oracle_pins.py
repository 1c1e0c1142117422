"""Pins the CPU oracle (oracle/nf_oracle.c) against what fixes its answers
independently of its own formulas: float64 closed forms, brute force on tiny
inputs, invariants, and the known-answer inputs of the reference's own test
programs.  No GPU needed."""
import math

import numpy as np
import pytest

from nanoflow_amd import synth


def f64(a):
    return a.astype(np.float64)


def rel_err(got, ref):
    ref = f64(ref)
    return np.abs(f64(got) - ref).max() / max(np.abs(ref).max(), 1e-30)


# ------------------------------------------------------------------ fp16 helpers

def test_half_roundtrip_all_bit_patterns(oracle):
    l = oracle.lib()
    pats = np.arange(65536, dtype=np.uint16)
    as_f = pats.view(np.float16).astype(np.float32)
    for p in list(range(0, 65536, 257)) + [0, 1, 0x3ff, 0x400, 0x7bff, 0x7c00, 0x8000, 0xfbff]:
        v = l.nfo_half_to_float(p)
        if math.isnan(as_f[p]):
            assert math.isnan(v)
        else:
            assert v == as_f[p]
            assert l.nfo_float_to_half(v) == p


def test_float_to_half_rounding_matches_numpy(oracle):
    l = oracle.lib()
    rng = np.random.default_rng(0)
    xs = np.concatenate([rng.standard_normal(2000).astype(np.float32) * s
                         for s in (1e-7, 1e-4, 1.0, 100.0, 7e4)])
    xs = np.concatenate([xs, np.float32([65504, 65519.9, 65520, 1e-8, 5.96e-8, 2.98e-8, 2.9802326e-8])])
    for x in xs:
        with np.errstate(over="ignore"):
            want = np.float32(x).astype(np.float16).view(np.uint16)
        assert l.nfo_float_to_half(float(x)) == int(want), x


# ------------------------------------------------------------------ GEMM

@pytest.mark.parametrize("M,N,K", [(1, 8, 16), (7, 24, 40), (33, 130, 257), (128, 64, 512)])
def test_gemm_closed_form(oracle, M, N, K):
    rng = np.random.default_rng(1)
    A = synth.normal_f16(rng, (M, K))
    B = synth.normal_f16(rng, (K, N), 0.05)
    Cm = synth.normal_f16(rng, (M, N))
    ref = f64(A) @ f64(B)
    D = oracle.gemm(A, B)
    assert rel_err(D, ref) < 1e-3
    D2 = oracle.gemm(A, B, Cm, alpha=0.5, beta=1.0)
    assert rel_err(D2, 0.5 * ref + f64(Cm)) < 1e-3
    # transposed-weight storage gives the same product
    D3 = oracle.gemm(A, np.ascontiguousarray(B.T), b_col_major=True)
    assert rel_err(D3, ref) < 1e-3


def test_gemm_identity_and_operand_order(oracle):
    # A.I == A exactly; a non-symmetric case fails if operands were transposed/swapped
    rng = np.random.default_rng(2)
    A = synth.normal_f16(rng, (5, 16))
    I = np.eye(16, dtype=np.float16)
    assert np.array_equal(oracle.gemm(A, I), A)
    B = np.zeros((16, 8), np.float16)
    B[3, 5] = 2.0  # picks column 3 of A into output column 5
    D = oracle.gemm(A, B)
    want = np.zeros((5, 8), np.float16)
    want[:, 5] = (A[:, 3].astype(np.float32) * 2).astype(np.float16)
    assert np.array_equal(D, want)


def test_gemm_residual_beta_one_is_single_rounding(oracle):
    # D = half(acc + C): one rounding, not half(half(acc) + C)
    A = np.array([[1.0]], np.float16)
    B = np.array([[2.0 ** -12]], np.float16)          # acc = 2^-12, below half ulp of 1.0 ... kept in fp32
    Cm = np.array([[1.0 + 2.0 ** -10]], np.float16)
    D = oracle.gemm(A, B, Cm, beta=1.0)
    want = np.float16(np.float32(2.0 ** -12) + np.float32(Cm[0, 0]))
    assert D[0, 0] == want


# ------------------------------------------------------------------ dual GEMM (gate/up SwiGLU)

def test_dual_known_answer_from_reference_test_inputs(oracle):
    """Inputs of pipeline/src/test_dual.cu:13-22: every operand is the 128x128 matrix
    X[j][k] = half((j+k)/2560); expected values computed here analytically in float64
    from the rounded inputs (the program itself only prints)."""
    M = N = K = 128
    j, k = np.meshgrid(np.arange(M), np.arange(N), indexing="ij")
    X = ((j + k).astype(np.float32) / 20 / 128).astype(np.float16)
    out, d0, d1 = oracle.dual_swiglu(X, X, X, return_parts=True)
    acc = f64(X) @ f64(X)
    assert rel_err(d0, acc) < 1e-3 and rel_err(d1, acc) < 1e-3
    g = f64(acc.astype(np.float16))
    want = g / (1 + np.exp(-g)) * g
    assert rel_err(out, want) < 1e-3
    # spot values that a swapped gate/up or a missing SiLU would miss by far more
    assert abs(float(out[0, 0]) - want[0, 0]) <= 1e-3 * abs(want[0, 0]) + 1e-6
    assert abs(float(out[127, 127]) - want[127, 127]) <= 1e-3 * abs(want[127, 127])


def test_dual_gate_is_first_weight(oracle):
    rng = np.random.default_rng(3)
    A = synth.normal_f16(rng, (9, 32))
    Bg = synth.normal_f16(rng, (32, 16), 0.3)
    Bu = synth.normal_f16(rng, (32, 16), 0.3)
    out = oracle.dual_swiglu(A, Bg, Bu)
    g = f64((f64(A) @ f64(Bg)).astype(np.float16))
    u = f64((f64(A) @ f64(Bu)).astype(np.float16))
    assert rel_err(out, g / (1 + np.exp(-g)) * u) < 2e-3
    swapped = u / (1 + np.exp(-u)) * g
    assert rel_err(out, swapped) > 5e-2


# ------------------------------------------------------------------ fp8 weights

def test_e4m3_decode_table(oracle):
    # OCP e4m3fn: bias 7, no inf, max 448, subnormal step 2^-9
    assert oracle.e4m3_to_float(0x00) == 0.0
    assert oracle.e4m3_to_float(0x01) == 2.0 ** -9
    assert oracle.e4m3_to_float(0x08) == 2.0 ** -6
    assert oracle.e4m3_to_float(0x38) == 1.0
    assert oracle.e4m3_to_float(0x7e) == 448.0
    assert oracle.e4m3_to_float(0xfe) == -448.0
    assert math.isnan(oracle.e4m3_to_float(0x7f))
    import torch
    t = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    for v in range(256):
        got = oracle.e4m3_to_float(v)
        assert (math.isnan(got) and math.isnan(t[v])) or got == t[v]


def test_gemm_f8w_is_dequantise_then_gemm(oracle):
    import torch
    rng = np.random.default_rng(4)
    M, N, K = 6, 24, 64
    A = synth.normal_f16(rng, (M, K))
    W = rng.standard_normal((K, N)).astype(np.float32) * 0.02
    scale = (np.abs(W).max(axis=0) / 448.0).astype(np.float32)
    Wq = torch.from_numpy(W / scale).to(torch.float8_e4m3fn)
    Bq = Wq.view(torch.uint8).numpy()
    deq = Wq.to(torch.float32).numpy().astype(np.float64) * scale
    D = oracle.gemm_f8w(A, Bq, scale)
    assert rel_err(D, f64(A) @ deq) < 1e-3


# ------------------------------------------------------------------ row ops

def _finite_codes():
    return [c for c in range(256) if (c & 0x7F) != 0x7F]


def test_e4m3_encode_roundtrip_ties_and_saturation(oracle):
    dec = {c: oracle.e4m3_to_float(c) for c in _finite_codes()}
    # every finite code is a fixed point of decode -> encode (the sign of zero included)
    for c, v in dec.items():
        assert oracle.float_to_e4m3(v) == c, hex(c)
    # between neighbours: nearest wins, the midpoint goes to the even code
    for c in range(0, 0x7E):
        lo, hi = dec[c], dec[c + 1]
        mid = (lo + hi) / 2                           # exact in binary
        even = c if c % 2 == 0 else c + 1
        assert oracle.float_to_e4m3(mid) == even, hex(c)
        assert oracle.float_to_e4m3(np.nextafter(np.float32(mid), np.float32(0))) == c
        assert oracle.float_to_e4m3(np.nextafter(np.float32(mid), np.float32(1e9))) == c + 1
        assert oracle.float_to_e4m3(-mid) == 0x80 | even
    # saturation instead of NaN codes
    for x, want in [(448.0, 0x7E), (463.9, 0x7E), (464.0, 0x7E), (1e6, 0x7E), (-1e6, 0xFE),
                    (float("inf"), 0x7E), (2.0 ** -10, 0x00), (2.0 ** -10 * 1.01, 0x01), (1.0, 0x38)]:
        assert oracle.float_to_e4m3(x) == want, x
    # agrees with torch's converter wherever that one does not produce NaN
    import torch
    xs = np.random.default_rng(0).normal(0, 50, size=4000).astype(np.float32)
    xs = xs[np.abs(xs) < 448]
    t = torch.from_numpy(xs).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert [oracle.float_to_e4m3(float(x)) for x in xs] == t.tolist()


def test_quantize_rows_e4m3_closed_form(oracle):
    # a row made of representable values times a power of two, with 448 * 2^j present, quantises
    # exactly: scale = 2^j and the codes are the values' own codes
    codes = np.array([0x7E, 0x38, 0xB8, 0x01, 0x00, 0x45, 0xC9, 0x08] * 2, np.uint8)
    vals = np.array([oracle.e4m3_to_float(int(c)) for c in codes], np.float32)
    X = np.stack([vals * 2.0 ** -5, vals * 2.0 ** 3, np.zeros_like(vals)]).astype(np.float16)
    assert np.array_equal(X[0].astype(np.float32), vals * 2.0 ** -5)      # fp16 holds them exactly
    Xq, sc = oracle.quantize_rows_e4m3(X)
    assert sc.tolist() == [2.0 ** -5, 2.0 ** 3, 1.0]
    assert np.array_equal(Xq[0], codes) and np.array_equal(Xq[1], codes)
    assert not Xq[2].any()
    # general rows: |x - scale * decode(q)| <= half a step of the code's binade, max maps to 448
    rng = np.random.default_rng(1)
    X = (rng.normal(0, 1, (5, 64)) * np.array([[1e-3], [1], [30], [0.2], [7]])).astype(np.float16)
    Xq, sc = oracle.quantize_rows_e4m3(X)
    deq = np.vectorize(oracle.e4m3_to_float)(Xq) * sc[:, None]
    assert np.array_equal((Xq & 0x7F).max(axis=1), np.full(5, 0x7E))
    rel = np.abs(deq - X.astype(np.float32)) / np.maximum(np.abs(X.astype(np.float32)), sc[:, None] * 2.0 ** -6)
    assert rel.max() <= 2.0 ** -4 + 1e-6


def test_gemm_f8f8_matches_float64(oracle):
    rng = np.random.default_rng(2)
    M, N, K = 9, 24, 80
    fin = np.array(_finite_codes(), np.uint8)
    Aq, Bq = rng.choice(fin, (M, K)), rng.choice(fin, (N, K))
    sa, sb = rng.uniform(0.01, 0.1, M).astype(np.float32), rng.uniform(0.001, 0.01, N).astype(np.float32)
    Cm = rng.normal(0, 1, (M, N)).astype(np.float16)
    lut = np.array([oracle.e4m3_to_float(c) if (c & 0x7F) != 0x7F else 0.0 for c in range(256)])
    ref = 0.5 * (sa[:, None] * sb[None, :]).astype(np.float64) * (lut[Aq] @ lut[Bq].T) + 2.0 * Cm.astype(np.float64)
    got = oracle.gemm_f8f8(Aq, sa, Bq, sb, Cm, alpha=0.5, beta=2.0).astype(np.float64)
    assert np.abs(got - ref).max() <= 1e-3 * np.abs(ref).max()
    # transposing the roles of the operands transposes the result
    g1 = oracle.gemm_f8f8(Aq, sa, Bq, sb)
    g2 = oracle.gemm_f8f8(Bq, sb, Aq, sa)
    assert np.array_equal(g1, g2.T)


def test_silu_mul_and_fp8_dual_closed_form(oracle):
    rng = np.random.default_rng(4)
    g = rng.normal(0, 3, 4096).astype(np.float16)
    u = rng.normal(0, 3, 4096).astype(np.float16)
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    ref = g64 / (1 + np.exp(-g64)) * u64
    got = oracle.silu_mul(g, u).astype(np.float64)
    assert np.abs(got - ref).max() <= 1e-3 * np.abs(ref).max()
    assert np.array_equal(oracle.silu_mul(np.zeros(8, np.float16), u[:8]), np.zeros(8, np.float16))   # silu(0) = 0
    # the order of the operands matters: silu is taken of the first
    assert not np.array_equal(oracle.silu_mul(g, u), oracle.silu_mul(u, g))
    # the fp8 gate/up pair = the two fp8 products, rounded to fp16, through that function; against
    # float64 on the dequantised operands
    M, N, K = 7, 24, 96
    fin = np.array(_finite_codes(), np.uint8)
    small = fin[(fin & 0x7F) < 0x50]                       # magnitudes below 8: keeps products in fp16 range
    Aq, Gq, Uq = rng.choice(small, (M, K)), rng.choice(small, (N, K)), rng.choice(small, (N, K))
    sa = rng.uniform(0.05, 0.2, M).astype(np.float32)
    sg, su = rng.uniform(0.01, 0.05, N).astype(np.float32), rng.uniform(0.01, 0.05, N).astype(np.float32)
    lut = np.array([oracle.e4m3_to_float(c) if (c & 0x7F) != 0x7F else 0.0 for c in range(256)])
    g64 = (sa[:, None] * sg[None, :]).astype(np.float64) * (lut[Aq] @ lut[Gq].T)
    u64 = (sa[:, None] * su[None, :]).astype(np.float64) * (lut[Aq] @ lut[Uq].T)
    ref = g64 / (1 + np.exp(-g64)) * u64
    got = oracle.dual_swiglu_f8f8(Aq, sa, Gq, sg, Uq, su).astype(np.float64)
    assert np.abs(got - ref).max() <= 3e-3 * np.abs(ref).max()


def test_smaller_operators_against_plain_loops(oracle):
    """The activation between separate gate / up and down projections takes SiLU of the RIGHT half of a
    row and multiplies by the left half; the column splits and the transpose against element loops."""
    rng = np.random.default_rng(12)
    M, N = 5, 16
    x = rng.normal(0, 2, (M, 2 * N)).astype(np.float16)
    got = oracle.activation_silu_mul(x).astype(np.float64)
    for r in range(M):
        for c in range(N):
            left, right = float(x[r, c]), float(x[r, N + c])
            want = left * (right / (1.0 + np.exp(-right)))
            assert abs(got[r, c] - want) <= 1e-3 * abs(want) + 1e-6, (r, c)
    z = x.copy()
    z[:, N:] = 0                                      # silu(0) = 0: a zero right half gives zeros, a zero left half too
    assert not oracle.activation_silu_mul(z).any()
    z = x.copy()
    z[:, :N] = 0
    assert not oracle.activation_silu_mul(z).any()
    sw = np.concatenate([x[:, N:], x[:, :N]], axis=1)  # and the halves are not interchangeable
    assert not np.array_equal(oracle.activation_silu_mul(sw), oracle.activation_silu_mul(x))
    kqv = rng.normal(0, 1, (7, 8 + 24 + 16)).astype(np.float16)
    k, q, v = oracle.split_kqv(kqv, 8, 24, 16)
    for r in range(7):
        assert [k[r, c] for c in range(8)] == [kqv[r, c] for c in range(8)]
        assert [q[r, c] for c in range(24)] == [kqv[r, 8 + c] for c in range(24)]
        assert [v[r, c] for c in range(16)] == [kqv[r, 32 + c] for c in range(16)]
    wide = rng.normal(0, 1, (6, 3 * 8)).astype(np.float16)
    for rank in range(3):
        part = oracle.extract_rank_columns(wide, 3, rank)
        assert part.shape == (6, 8) and all(part[r, c] == wide[r, rank * 8 + c] for r in range(6) for c in range(8))
    t = oracle.transpose(wide)
    assert t.shape == (24, 6) and all(t[c, r] == wide[r, c] for r in range(6) for c in range(24))


def test_quantize_weight_is_the_row_quantiser_on_the_transpose(oracle):
    rng = np.random.default_rng(5)
    W = rng.normal(0, 0.02, (48, 24)).astype(np.float16)         # [K, N]
    W[:, 3] = 0                                                   # an all-zero output channel
    Wq, sc = oracle.quantize_weight_e4m3(W)
    assert Wq.shape == (24, 48) and sc.shape == (24,)
    amax = np.abs(W.astype(np.float32)).max(axis=0)
    assert sc[3] == 1.0 and not Wq[3].any()
    live = np.arange(24) != 3
    assert np.array_equal(sc[live], (amax / np.float32(448.0))[live])
    assert np.array_equal((Wq[live] & 0x7F).max(axis=1), np.full(23, 0x7E))    # each channel's max maps to 448
    deq = np.vectorize(oracle.e4m3_to_float)(Wq) * sc[:, None]                  # [N, K]
    assert np.abs(deq.T - W.astype(np.float32)).max() <= amax.max() * 2.0 ** -4


def test_decoder_forward_f8_vs_float64_model_on_dequantised_weights(oracle):
    """Both activation modes of the fp8 forward against the independent float64 model run on the
    dequantised weights: fp16 activations within the fp16 pipeline's own error; fp8 activations
    (each GEMM input re-quantised per row, 3 mantissa bits) within 3e-2 per GEMM, which chained
    through the 8 fp8 GEMMs of two layers is bounded here at 1e-1 of the largest magnitude."""
    shape = synth.tiny_shape(layers=2, vocab=512, Hq=4, Hkv=2, ffn=384, hidden=256)
    w = synth.make_weights(shape, seed=0)
    for k in ("w_kqv", "w_o", "w_gate", "w_up", "w_down"):
        w[k] = [(a.astype(np.float32) * 3).astype(np.float16) for a in w[k]]
    w["embedding"] = (w["embedding"].astype(np.float32) * 30).astype(np.float16)
    wq = oracle.quantize_model_weights(w)
    lut = np.array([oracle.e4m3_to_float(c) for c in range(256)], np.float64)
    w_deq = dict(w)
    for k in oracle.FP8_LAYER_WEIGHTS:
        w_deq[k] = [(lut[q] * s[:, None].astype(np.float64)).T for q, s in wq[k]]      # float64 [K, N]
    b = synth.make_batch([17, 40, 3], [(0, 21), (16, 10)], vocab=shape.vocab, seed=7, extra_pages=2)
    rng = np.random.default_rng(1)
    pools = [synth.make_kv_pool(b.num_pages, shape, rng) for _ in range(shape.layers)]
    ref_x, ref_logits = _numpy_decoder_f64(shape, w_deq, [p.copy() for p in pools], b)
    cfg = shape.as_dict()
    h16, l16, _ = oracle.decoder_forward_f8(cfg, w, wq, [p.copy() for p in pools], b.as_dict(), "f16", want_logits=True)
    assert rel_err(h16, ref_x) < 4e-3 and rel_err(l16, ref_logits) < 6e-3
    h8, l8, s8 = oracle.decoder_forward_f8(cfg, w, wq, [p.copy() for p in pools], b.as_dict(), "e4m3", want_logits=True)
    assert 1e-2 < rel_err(h8, ref_x) < 1e-1 and rel_err(l8, ref_logits) < 1e-1
    # the quantisation is visible: the fp16-weight forward differs from both by more than fp16 noise
    h_plain, _, _ = oracle.decoder_forward(cfg, w, [p.copy() for p in pools], b.as_dict())
    assert rel_err(h_plain, ref_x) > 6e-3


def test_move_kv_pages_hand_case(oracle):
    # 3 requests owning pages [4, 1], [0], [3, 2, 5]; requests 2 and 0 are listed
    indptr = np.array([0, 2, 3, 6], np.int32)
    indices = np.array([4, 1, 0, 3, 2, 5], np.int32)
    pool = np.arange(6 * 4, dtype=np.float16).reshape(6, 4)
    staging = np.full((6, 4), -1, np.float16)
    oracle.move_kv_pages([2, 0], indptr, indices, staging, pool, to_pool=False)
    want = np.full((6, 4), -1, np.float16)
    want[0], want[1], want[3], want[4], want[5] = pool[4], pool[1], pool[3], pool[2], pool[5]   # slot 2 (request 1) untouched
    assert np.array_equal(staging, want)
    pool2 = np.zeros_like(pool)
    oracle.move_kv_pages([2, 0], indptr, indices, staging, pool2, to_pool=True)
    assert np.array_equal(pool2[[1, 2, 3, 4, 5]], pool[[1, 2, 3, 4, 5]]) and not pool2[0].any()   # page 0 is request 1's


def test_rmsnorm_closed_form(oracle):
    rng = np.random.default_rng(5)
    x = synth.normal_f16(rng, (11, 256), 3.0)
    w = synth.normal_f16(rng, (256,), 0.02, 1.0)
    got = oracle.rmsnorm(x, w, 1e-5)
    xf = f64(x)
    want = xf / np.sqrt((xf ** 2).mean(axis=1, keepdims=True) + 1e-5) * f64(w)
    assert rel_err(got, want) < 1e-3
    # eps matters for a zero row: output must be exactly 0, not NaN
    z = np.zeros((1, 256), np.float16)
    assert np.array_equal(oracle.rmsnorm(z, w), z)


def test_embedding_keep_token_bruteforce(oracle):
    rng = np.random.default_rng(6)
    table = synth.normal_f16(rng, (50, 64))
    tok = rng.integers(0, 50, size=13, dtype=np.int32)
    assert np.array_equal(oracle.embedding(tok, table), table[tok])
    x = synth.normal_f16(rng, (13, 64))
    indptr = np.array([0, 1, 2, 7, 13], np.int32)
    assert np.array_equal(oracle.keep_token(x, indptr, 4), x[[0, 1, 6, 12]])


def _argmax_literal(row):
    """Literal python transcription of the 1024-slot scan + halving tree."""
    NT = 1024
    sval = [-10000.0] * NT
    sidx = [0] * NT
    for i, v in enumerate(row):
        t = i % NT
        if float(v) > sval[t]:
            sval[t] = float(v)
            sidx[t] = i
    s = NT // 2
    while s > 0:
        for t in range(s):
            if sval[t] < sval[t + s]:
                sval[t] = sval[t + s]
                sidx[t] = sidx[t + s]
        s //= 2
    return sidx[0], sval[0]


def test_argmax_unique_max_and_ties(oracle):
    rng = np.random.default_rng(7)
    x = synth.normal_f16(rng, (6, 3000))
    arg, mv = oracle.argmax(x)
    assert np.array_equal(arg, x.astype(np.float32).argmax(axis=1))
    assert np.array_equal(mv, x.max(axis=1))
    # ties: equal maxima at several columns -> the reference's scan/tree order decides
    t = np.full((4, 2500), -1.0, np.float16)
    t[0, [5, 1029, 6]] = 3.0          # same slot 5 twice (first wins), slot 6
    t[1, [512, 256, 768]] = 3.0       # bit-reversed priority: 512 (0b1000000000) wins over 256
    t[2, [1, 2]] = 3.0                # even slot wins the last tree level
    t[3, :] = -20000.0                # nothing above the -10000 start: index 0
    arg, mv = oracle.argmax(t)
    for r in range(4):
        want_i, want_v = _argmax_literal(t[r])
        assert arg[r] == want_i, (r, arg[r], want_i)
        assert float(mv[r]) == np.float16(want_v)
    assert arg[1] == 512 and arg[2] == 2 and arg[3] == 0


# ------------------------------------------------------------------ RoPE + paged append

def test_kv_offset_layout(oracle):
    # pool[page][kv][entry][head][feat]; V half sits page_size*Hkv*d elements after K
    P, Hkv, d = 16, 8, 128
    pool = np.arange(3 * 2 * P * Hkv * d).reshape(3, 2, P, Hkv, d)
    for idx in [(0, 0, 0, 0, 0), (2, 1, 15, 7, 127), (1, 0, 3, 2, 5), (1, 1, 3, 2, 5)]:
        assert oracle.kv_offset(*idx, P, Hkv, d) == pool[idx]
    assert oracle.kv_offset(1, 1, 3, 2, 5, P, Hkv, d) - oracle.kv_offset(1, 0, 3, 2, 5, P, Hkv, d) == P * Hkv * d


def _rope_f64(x, pos, theta, d, scale=1.0):
    i = np.arange(d)
    inv = (pos / scale) / theta ** (2.0 * (i % (d // 2)) / d)
    perm = np.where(i < d // 2, -np.roll(f64(x), -d // 2), np.roll(f64(x), d // 2))
    return np.cos(inv) * f64(x) + np.sin(inv) * perm


def test_rope_matches_reference_cpu_rule_and_float64(oracle):
    rng = np.random.default_rng(8)
    d = 128
    for pos in (0, 1, 17, 1023, 1535):
        x = synth.normal_f16(rng, (d,))
        ref32 = oracle.ref_llama_rope(x, pos, 1.0, 5e5)
        want = _rope_f64(x, pos, 5e5, d)
        assert np.abs(ref32 - want).max() < 2e-3 * np.abs(want).max()


def test_rope_append_indices_values_and_invariants(oracle):
    rng = np.random.default_rng(9)
    Hq, Hkv, d, P = 8, 2, 128, 16
    b = synth.make_batch([5, 31, 16, 0], [(0, 20), (37, 9)], vocab=100, page_size=P, seed=1,
                         extra_pages=3)
    T = b.tokens
    kqv = synth.normal_f16(rng, (T, (Hq + 2 * Hkv) * d))
    pool = np.zeros((b.num_pages, 2, P, Hkv, d), np.float16)
    q, pg, en = oracle.rope_append(kqv, pool, b.kv_indices, b.kv_indptr, b.rev_input_indptr,
                                   b.per_token_offset, Hq, Hkv, d, P, 1.0, 5e5, return_index=True)
    touched = np.zeros((b.num_pages, P), bool)
    for t in range(T):
        r, p = b.rev_input_indptr[t], b.per_token_offset[t]
        page = b.kv_indices[b.kv_indptr[r] + p // P]
        assert (pg[t], en[t]) == (page, p % P)                      # bit-exact index rule
        assert not touched[page, p % P]
        touched[page, p % P] = True
        row = kqv[t].reshape(Hq + 2 * Hkv, d)
        assert np.array_equal(pool[page, 1, p % P], row[Hkv:2 * Hkv])  # V copied bit-exact
        for h in range(Hkv):
            want = _rope_f64(row[h], p, 5e5, d)
            assert np.abs(f64(pool[page, 0, p % P, h]) - want).max() < 2e-3 * np.abs(want).max() + 1e-3
        for h in range(Hq):
            want = _rope_f64(row[2 * Hkv + h], p, 5e5, d)
            got = q[t].reshape(Hq, d)[h]
            assert np.abs(f64(got) - want).max() < 2e-3 * np.abs(want).max() + 1e-3
            # rotation preserves the norm of each (i, i+d/2) pair
            n_in = f64(row[2 * Hkv + h][:64]) ** 2 + f64(row[2 * Hkv + h][64:]) ** 2
            n_out = f64(got[:64]) ** 2 + f64(got[64:]) ** 2
            assert np.abs(n_in - n_out).max() < 2e-2 * max(n_in.max(), 1.0)
        if p == 0:  # position 0 is the identity
            assert np.array_equal(pool[page, 0, 0], row[:Hkv])
            assert np.array_equal(q[t].reshape(Hq, d), row[2 * Hkv:])
    # nothing else in the pool was written
    untouched = np.transpose(pool, (0, 2, 1, 3, 4))[~touched]
    assert not untouched.any()
    assert touched.sum() == T


def test_rope_llama31_smoothing_matches_wavelength_form(oracle):
    # Llama-3.1 rule written over wavelengths (the published form) vs the reference's
    # smooth_a/smooth_b form (pipeline/include/config.h:101-110)
    factor, low, high, orig, theta, d = 8.0, 1.0, 4.0, 8192, 5e5, 128
    smooth_a = orig / (2 * math.pi * high - 2 * math.pi * low)
    smooth_b = -1.0 / (high / low - 1.0)
    for i in range(d):
        f = theta ** (-2.0 * (i % (d // 2)) / d)
        wavelen = 2 * math.pi / f
        if wavelen < orig / high:
            want = f
        elif wavelen > orig / low:
            want = f / factor
        else:
            s = (orig / wavelen - low) / (high - low)
            want = (1 - s) * f / factor + s * f
        got = oracle.rope_freq(i, d, factor, theta, smooth_a, smooth_b)
        assert abs(got - want) <= 2e-5 * want, (i, got, want)
    # no scaling: plain theta^(-2i/d)
    assert abs(oracle.rope_freq(3, d, 1.0, theta) - theta ** (-6.0 / d)) < 1e-6


# ------------------------------------------------------------------ attention

def _dense_attention_f64(q, k, v, causal, group):
    # q [qo, Hq, d], k/v [kv, Hkv, d]
    qo, Hq, d = q.shape
    kv = k.shape[0]
    out = np.zeros((qo, Hq, d))
    for h in range(Hq):
        s = f64(q[:, h]) @ f64(k[:, h // group]).T / math.sqrt(d)
        if causal:
            qi, ki = np.meshgrid(np.arange(qo), np.arange(kv), indexing="ij")
            s = np.where(ki > kv + qi - qo, -np.inf, s)
        p = np.exp(s - s.max(axis=1, keepdims=True))
        p /= p.sum(axis=1, keepdims=True)
        out[:, h] = p @ f64(v[:, h // group])
    return out


def _gather_kv(pool, b, r, P):
    pages = b.kv_indices[b.kv_indptr[r]:b.kv_indptr[r + 1]]
    L = b.kv_len[r]
    k = pool[pages, 0].reshape(-1, *pool.shape[3:])[:L]
    v = pool[pages, 1].reshape(-1, *pool.shape[3:])[:L]
    return k, v


@pytest.mark.parametrize("Hq,Hkv", [(8, 2), (8, 1), (4, 4)])
def test_attention_vs_dense_float64(oracle, Hq, Hkv):
    rng = np.random.default_rng(10)
    d, P = 128, 16
    b = synth.make_batch([15, 16, 40], [(0, 20), (21, 13)], vocab=10, page_size=P, seed=2, extra_pages=2)
    pool = synth.make_kv_pool(b.num_pages, synth.ModelShape(Hq=Hq, Hkv=Hkv), rng)
    q = synth.normal_f16(rng, (b.tokens, Hq * d))
    nd = b.decodePrefillBorder
    o = oracle.attention_paged(q, b.input_indptr[:nd + 1], pool, b.kv_indptr[:nd + 1], b.kv_indices,
                               b.kv_last_page_len[:nd], Hq, Hkv, d, P, causal=False)
    o = oracle.attention_paged(q, b.input_indptr[nd:], pool, b.kv_indptr[nd:], b.kv_indices,
                               b.kv_last_page_len[nd:], Hq, Hkv, d, P, causal=True, out=o)
    for r in range(b.req_num):
        k, v = _gather_kv(pool, b, r, P)
        rows = slice(b.input_indptr[r], b.input_indptr[r + 1])
        want = _dense_attention_f64(q[rows].reshape(-1, Hq, d), k, v, causal=r >= nd, group=Hq // Hkv)
        got = f64(o[rows]).reshape(-1, Hq, d)
        assert np.abs(got - want).max() < 2e-3 * np.abs(want).max() + 1e-3, r


def test_attention_invariants(oracle):
    rng = np.random.default_rng(11)
    Hq, Hkv, d, P = 8, 2, 128, 16
    shape = synth.ModelShape(Hq=Hq, Hkv=Hkv)
    # (1) all keys equal -> uniform softmax -> output = mean of V
    b = synth.make_batch([36], [], vocab=10, page_size=P, seed=3)
    pool = synth.make_kv_pool(b.num_pages, shape, rng)
    pool[:, 0] = pool[0, 0, 0]
    q = synth.normal_f16(rng, (1, Hq * d))
    o = oracle.attention_paged(q, b.input_indptr, pool, b.kv_indptr, b.kv_indices, b.kv_last_page_len,
                               Hq, Hkv, d, P, causal=False)
    k, v = _gather_kv(pool, b, 0, P)
    want = np.repeat(f64(v).mean(axis=0), Hq // Hkv, axis=0).reshape(-1)
    assert np.abs(f64(o[0]) - want).max() < 2e-3

    # (2) one-hot: one key aligned with q and huge -> output = that V row
    pool2 = synth.make_kv_pool(b.num_pages, shape, rng)
    pool2[:, 0] = 0
    pg, en = b.kv_indices[1], 3                       # token 19 of the request
    qv = np.zeros((1, Hq, d), np.float16)
    qv[..., 0] = 30.0
    pool2[pg, 0, en, :, 0] = 30.0
    o = oracle.attention_paged(qv.reshape(1, -1), b.input_indptr, pool2, b.kv_indptr, b.kv_indices,
                               b.kv_last_page_len, Hq, Hkv, d, P, causal=False)
    want = np.repeat(f64(pool2[pg, 1, en]), Hq // Hkv, axis=0).reshape(-1)
    assert np.abs(f64(o[0]) - want).max() < 2e-3

    # (3) page-table permutation invariance: move pages, same result
    b3 = synth.make_batch([50, 20], [(0, 33)], vocab=10, page_size=P, seed=4, extra_pages=5)
    pool3 = synth.make_kv_pool(b3.num_pages, shape, rng)
    q3 = synth.normal_f16(rng, (b3.tokens, Hq * d))
    o_a = oracle.attention_paged(q3, b3.input_indptr, pool3, b3.kv_indptr, b3.kv_indices,
                                 b3.kv_last_page_len, Hq, Hkv, d, P, causal=True)
    perm = rng.permutation(b3.num_pages)
    pool3p = np.empty_like(pool3)
    pool3p[perm] = pool3
    o_b = oracle.attention_paged(q3, b3.input_indptr, pool3p, b3.kv_indptr,
                                 perm[b3.kv_indices].astype(np.int32), b3.kv_last_page_len, Hq, Hkv,
                                 d, P, causal=True)
    assert np.array_equal(o_a, o_b)

    # (4) decode == prefill with qo_len 1 (causal flag irrelevant for a single last row)
    b4 = synth.make_batch([29], [], vocab=10, page_size=P, seed=5)
    pool4 = synth.make_kv_pool(b4.num_pages, shape, rng)
    q4 = synth.normal_f16(rng, (1, Hq * d))
    args = (q4, b4.input_indptr, pool4, b4.kv_indptr, b4.kv_indices, b4.kv_last_page_len, Hq, Hkv, d, P)
    assert np.array_equal(oracle.attention_paged(*args, causal=False),
                          oracle.attention_paged(*args, causal=True))


def test_chunked_prefill_equals_single_prefill(oracle):
    """A 45-token prompt in chunks 20+25 (second chunk sees the first's KV) gives the
    same rows as one 45-token causal prefill."""
    rng = np.random.default_rng(12)
    Hq, Hkv, d, P = 4, 2, 128, 16
    shape = synth.ModelShape(Hq=Hq, Hkv=Hkv)
    full = synth.make_batch([], [(0, 45)], vocab=10, page_size=P, seed=6, permute=False)
    pool = synth.make_kv_pool(full.num_pages, shape, rng)
    q = synth.normal_f16(rng, (45, Hq * d))
    o_full = oracle.attention_paged(q, full.input_indptr, pool, full.kv_indptr, full.kv_indices,
                                    full.kv_last_page_len, Hq, Hkv, d, P, causal=True)
    c1 = synth.make_batch([], [(0, 20)], vocab=10, page_size=P, seed=6, permute=False)
    o1 = oracle.attention_paged(q[:20].copy(), c1.input_indptr, pool, c1.kv_indptr, c1.kv_indices,
                                c1.kv_last_page_len, Hq, Hkv, d, P, causal=True)
    c2 = synth.make_batch([], [(20, 25)], vocab=10, page_size=P, seed=6, permute=False)
    o2 = oracle.attention_paged(q[20:].copy(), c2.input_indptr, pool, c2.kv_indptr, c2.kv_indices,
                                c2.kv_last_page_len, Hq, Hkv, d, P, causal=True)
    assert np.array_equal(o_full[:20], o1)
    assert np.array_equal(o_full[20:], o2)


# ------------------------------------------------------------------ whole decoder

def _numpy_decoder_f64(shape, w, pools, b):
    """Independent float64 forward of the same model (no fp16 rounding between ops)."""
    d, Hq, Hkv, P = shape.d, shape.Hq, shape.Hkv, shape.page_size
    x = f64(w["embedding"][b.input_tokens])
    pools = [f64(p) for p in pools]

    def norm(v, g):
        return v / np.sqrt((v ** 2).mean(axis=1, keepdims=True) + shape.eps) * f64(g)

    for l in range(shape.layers):
        kqv = norm(x, w["ln_attn"][l]) @ f64(w["w_kqv"][l])
        if w.get("b_kqv") is not None:        # q/k/v projections with a bias: y = x W + b
            kqv = kqv + f64(w["b_kqv"][l])[None, :]
        attn = np.zeros((b.tokens, Hq * d))
        qrot = np.zeros((b.tokens, Hq, d))
        for t in range(b.tokens):
            r, p = b.rev_input_indptr[t], b.per_token_offset[t]
            page = b.kv_indices[b.kv_indptr[r] + p // P]
            row = kqv[t].reshape(Hq + 2 * Hkv, d)
            for h in range(Hkv):
                pools[l][page, 0, p % P, h] = _rope_f64(row[h], p, shape.rope_theta, d)
                pools[l][page, 1, p % P, h] = row[Hkv + h]
            for h in range(Hq):
                qrot[t, h] = _rope_f64(row[2 * Hkv + h], p, shape.rope_theta, d)
        for r in range(b.req_num):
            pages = b.kv_indices[b.kv_indptr[r]:b.kv_indptr[r + 1]]
            L = b.kv_len[r]
            k = pools[l][pages, 0].reshape(-1, Hkv, d)[:L]
            v = pools[l][pages, 1].reshape(-1, Hkv, d)[:L]
            rows = slice(b.input_indptr[r], b.input_indptr[r + 1])
            attn[rows] = _dense_attention_f64(qrot[rows], k, v, r >= b.decodePrefillBorder,
                                              Hq // Hkv).reshape(-1, Hq * d)
        xo = attn @ f64(w["w_o"][l]) + x
        h = norm(xo, w["ln_ffn"][l])
        g = h @ f64(w["w_gate"][l])
        u = h @ f64(w["w_up"][l])
        x = (g / (1 + np.exp(-g)) * u) @ f64(w["w_down"][l]) + xo
    last = x[b.input_indptr[1:] - 1]
    logits = norm(last, w["model_norm"]) @ f64(w["lm_head"])
    return x, logits


@pytest.mark.parametrize("kqv_bias", [False, True])
def test_decoder_forward_vs_independent_float64_model(oracle, kqv_bias):
    shape = synth.tiny_shape(layers=2, vocab=512, Hq=4, Hkv=2, ffn=384, hidden=256)
    # larger-than-init weights so the residual stream is not dominated by the embedding
    w = synth.make_weights(shape, seed=0, kqv_bias=kqv_bias)
    for k in ("w_kqv", "w_o", "w_gate", "w_up", "w_down"):
        w[k] = [(a.astype(np.float32) * 3).astype(np.float16) for a in w[k]]
    w["embedding"] = (w["embedding"].astype(np.float32) * 30).astype(np.float16)
    b = synth.make_batch([17, 40, 3], [(0, 21), (16, 10)], vocab=shape.vocab, seed=7, extra_pages=2)
    rng = np.random.default_rng(1)
    pools = [synth.make_kv_pool(b.num_pages, shape, rng) for _ in range(shape.layers)]
    pools_in = [p.copy() for p in pools]
    hidden, logits, sampled = oracle.decoder_forward(shape.as_dict(), w, pools, b.as_dict(),
                                                     want_logits=True)
    ref_x, ref_logits = _numpy_decoder_f64(shape, w, pools_in, b)
    if kqv_bias:    # dropping the bias must fail the comparison below by a wide margin
        no_bias, _ = _numpy_decoder_f64(shape, {k: v for k, v in w.items() if k != "b_kqv"}, pools_in, b)
        assert rel_err(no_bias, ref_x) > 0.1
    assert rel_err(hidden, ref_x) < 4e-3
    assert rel_err(logits, ref_logits) < 6e-3
    # sampled ids agree wherever the float64 top-1/top-2 gap is clear of fp16 noise
    top2 = np.sort(ref_logits, axis=1)[:, -2:]
    clear = (top2[:, 1] - top2[:, 0]) > 1e-2 * np.abs(ref_logits).max()
    assert clear.sum() >= 1
    assert np.array_equal(sampled[clear], ref_logits.argmax(axis=1)[clear])
    # the pools changed only at the appended slots
    for l in range(shape.layers):
        diff = (pools[l] != pools_in[l]).any(axis=(1, 3, 4))
        assert diff.sum() == b.tokens


# ---------------------------------------------------------------- bf16 helpers of the oracle

def test_bf16_conversions_agree_with_torch_and_round_to_even():
    torch = pytest.importorskip("torch")
    from oracle import nf_oracle as O
    rng = np.random.default_rng(11)
    x = (rng.standard_normal(20000) * np.exp(rng.uniform(-20, 20, 20000))).astype(np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.float_to_bf16(x), want)
    assert np.array_equal(O.bf16_to_float(want), torch.from_numpy(want.view(np.int16)).view(torch.bfloat16).float().numpy())
    # ties: 1 + 2^-8 lies halfway between 1 and 1 + 2^-7 -> even (1.0); 1 + 3*2^-8 -> 1 + 2^-6
    assert O.bf16_to_float(O.float_to_bf16(np.array([1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8], np.float32))).tolist() == [1.0, 1 + 2.0 ** -6]


def test_bf16_gemm_closed_form_on_exact_inputs():
    from oracle import nf_oracle as O
    # small integers are exact in bf16 and so are their dot products: the result is the integer matmul
    rng = np.random.default_rng(12)
    A = rng.integers(-4, 5, (9, 16)).astype(np.float32)
    B = rng.integers(-4, 5, (16, 24)).astype(np.float32)
    got = O.bf16_to_float(O.gemm_bf16(O.float_to_bf16(A), O.float_to_bf16(B)))
    assert np.array_equal(got, A @ B)
    Cm = rng.integers(-3, 4, (9, 24)).astype(np.float32)
    got = O.bf16_to_float(O.gemm_bf16(O.float_to_bf16(A), O.float_to_bf16(B), O.float_to_bf16(Cm), 0.5, 2.0))
    assert np.array_equal(got, O.bf16_to_float(O.float_to_bf16((0.5 * (A @ B) + 2.0 * Cm).astype(np.float32))))
    Bt = np.ascontiguousarray(B.T)
    assert np.array_equal(O.gemm_bf16(O.float_to_bf16(A), O.float_to_bf16(Bt), b_col_major=True),
                          O.gemm_bf16(O.float_to_bf16(A), O.float_to_bf16(B)))
