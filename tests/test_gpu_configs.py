"""Parity at the shapes of the benchmark configurations themselves.

* one full-size Llama-3-8B decoder layer on 64 decode tokens with KV lengths U[512,1024] (the
  reference-path parity case) and one Llama-3-70B-shaped layer, against the oracle: residual stream
  within tolerance, the KV slots written bit-exactly the ones the oracle writes, their values within
  tolerance;
* the one-iteration workload (1792 decode + 256 prefill tokens) at full width through the three
  schedules: size-independent properties (schedule independence, page-permutation invariance);
* fp8 GEMM at the 70B FFN shape, and one 70B-shaped layer with e4m3 weights through the pipeline
  (the shape and weight format of the fp8 benchmark configuration).
"""
import os

import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

from nanoflow_amd import synth  # noqa: E402

LAYER_RTOL = 2e-3   # the per-operator bound, held end to end through one decoder layer as well


def _max_rel(got, ref):
    ref = ref.astype(np.float64)
    return np.abs(got.astype(np.float64) - ref).max() / np.abs(ref).max()


def _decode_layer_case(oracle, shape, kv_lens, seed, pipelines, weight_format="f16", weight_layout="row"):
    """Iteration 0 prefills the last prompt token of every request (so that the decode iteration
    is fed distinct tokens: the samples of iteration 0); iteration 1 is the decode step under test."""
    from nanoflow_amd import engine, pllm_python as P
    rng = np.random.default_rng(seed)
    w = synth.make_weights(shape, seed=0)
    w["embedding"] = synth.normal_f16(rng, (shape.vocab, shape.hidden), 1.0)   # hidden input ~ N(0, 1)
    n = len(kv_lens)
    b0 = synth.make_batch([], [(int(L) - 1, 1) for L in kv_lens], vocab=shape.vocab, seed=seed, extra_pages=n)
    pools0 = [synth.make_kv_pool(b0.num_pages, shape, rng) for _ in range(shape.layers)]
    # iteration 1: every request decodes one token at position L; it may need one more page
    free = [p for p in range(b0.num_pages) if p not in set(b0.kv_indices.tolist())]
    indices, indptr = [], [0]
    for r in range(n):
        pg = b0.kv_indices[b0.kv_indptr[r]:b0.kv_indptr[r + 1]].tolist()
        if (int(kv_lens[r]) + 1 + 15) // 16 > len(pg):
            pg.append(free.pop())
        indices += pg
        indptr.append(len(indices))
    L = np.asarray(kv_lens, np.int64)

    def decode_batch(tokens):
        return synth.Batch(decodePrefillBorder=n, prefillNum=0, prefillTokensNum=0,
                           input_tokens=tokens.astype(np.int32), input_indptr=np.arange(n + 1, dtype=np.int32),
                           rev_input_indptr=np.arange(n, dtype=np.int32), per_token_offset=L.astype(np.int32),
                           kv_indptr=np.array(indptr, np.int32), kv_indices=np.array(indices, np.int32),
                           kv_last_page_len=(L % 16 + 1).astype(np.int32), kv_len=(L + 1).astype(np.int32),
                           num_pages=b0.num_pages)

    for pt in pipelines:
        print(f"shape hidden={shape.hidden} pipeline={pt.name} weight layout={weight_layout}", flush=True)
        T = max(64, (n + 63) // 64 * 64)
        with engine.Engine(shape, pt, global_batch=T, nano1=T // 2, kqv1=T // 4, kqv3=T // 4, kv_pages=b0.num_pages,
                           weights=w, kv_pools=pools0, weight_format=weight_format, weight_layout=weight_layout) as e:
            e.update(b0, keep_token_list=np.zeros(0, np.int32))
            s0 = e.run()
            kv_after0 = [p[:b0.num_pages].cpu().numpy() for p in e.kv]
            b1 = decode_batch(s0)
            e.update(b1, keep_token_list=np.ones(n, np.int32))
            e.run()
            hid = e.buffer("hidden").cpu().numpy()[:n]
            inter = {}
            if pt == P.PipelineType.NON_OVERLAP_LOCAL:
                inter = {k: e.buffer(k).cpu().numpy()[:n] for k in ("ln_attn", "kqv", "attn_out", "o_out", "ln_ffn", "act")}
            kv = [p[:b0.num_pages].cpu().numpy() for p in e.kv]
        # the oracle runs the decode iteration from the GPU's state after iteration 0
        pools_ref = [p.copy() for p in kv_after0]
        if weight_format == "e4m3":
            P.setWeightFormat(P.WeightFormat.F16)
            wq = oracle.quantize_model_weights(w)
            # (1) teacher-forced, per GEMM: the oracle is given the rows the device operator read
            # (the last layer's operator inputs), so re-quantisation noise cannot accumulate.
            # fp8 x fp8 on identical quantised rows: 2e-3; against the definition the fp8 tolerance
            # is stated for (fp16 activations x dequantised weights): 3e-2.
            x_in = oracle.embedding(b1.input_tokens.astype(np.int32), w["embedding"])
            l = shape.layers - 1
            mm8 = lambda x, key, C=None, beta=0.0: oracle.gemm_f8f8(*oracle.quantize_rows_e4m3(x), *wq[key][l], C, 1.0, beta)
            mm16 = lambda x, key, C=None, beta=0.0: oracle.gemm_f8w(x, np.ascontiguousarray(wq[key][l][0].T), wq[key][l][1], C, 1.0, beta)
            for mm, tol in ((mm8, 2e-3), (mm16, 3e-2)):
                checks = {
                    "kqv": mm(inter["ln_attn"], "w_kqv"),
                    "o_out": mm(inter["attn_out"], "w_o", x_in if shape.layers == 1 else None, 1.0 if shape.layers == 1 else 0.0),
                    "act": oracle.silu_mul(mm(inter["ln_ffn"], "w_gate"), mm(inter["ln_ffn"], "w_up")),
                    "hidden": mm(inter["act"], "w_down", inter["o_out"], 1.0),
                }
                for name, ref in checks.items():
                    if name == "o_out" and shape.layers != 1:
                        continue                       # the residual operand of a deeper model is gone by now
                    got = hid if name == "hidden" else inter[name]
                    err = _max_rel(got, ref)
                    # the gate/up pair's output is the product of two GEMM outputs (silu(g) * u), each
                    # within the fp8 bound of its definition: the bound of the product is twice that
                    bound = 2 * tol if name == "act" and tol > 2e-3 else tol
                    print(f"  teacher-forced {name}: max-norm relative error {err:.2e} (bound {bound:.0e})", flush=True)
                    assert err < bound, (pt, name, err, bound)
            # (2) free-running: the same arithmetic in the oracle end to end (rows re-quantised per
            # GEMM).  Re-quantisation makes the layer discontinuous, so two correct implementations
            # agree statistically here, not to fp16 rounding: nudging the oracle's norm weights by
            # one fp16 ulp moves its output by 5.3 % rms at this width; the bound is 8 % rms
            hid_ref, _, _ = oracle.decoder_forward_f8(shape.as_dict(), w, wq, pools_ref, b1.as_dict(), "e4m3")
            d = hid.astype(np.float64) - hid_ref.astype(np.float64)
            rms = np.sqrt((d ** 2).mean() / (hid_ref.astype(np.float64) ** 2).mean())
            print(f"  residual stream rms relative error {rms:.2e}, max-norm {_max_rel(hid, hid_ref):.2e}", flush=True)
            assert rms < 8e-2 and _max_rel(hid, hid_ref) < 2.5e-1, (pt, rms)
            kv_tol = 8e-2
        else:
            hid_ref, _, _ = oracle.decoder_forward(shape.as_dict(), w, pools_ref, b1.as_dict(), want_logits=False)
            err = _max_rel(hid, hid_ref)
            print(f"  residual stream max-norm relative error {err:.2e}", flush=True)
            assert err < LAYER_RTOL, (pt, err)
            kv_tol = 2e-3
            if inter and shape.layers == 1:
                # operator by operator at the per-operator bound: the oracle's operator on the rows
                # the device operator read
                x_in = oracle.embedding(b1.input_tokens.astype(np.int32), w["embedding"])
                checks = {
                    "ln_attn": (inter["ln_attn"], oracle.rmsnorm(x_in, w["ln_attn"][0], 1e-5)),
                    "kqv": (inter["kqv"], oracle.gemm(inter["ln_attn"], w["w_kqv"][0])),
                    "o_out": (inter["o_out"], oracle.gemm(inter["attn_out"], w["w_o"][0], x_in, 1.0, 1.0)),
                    "ln_ffn": (inter["ln_ffn"], oracle.rmsnorm(inter["o_out"], w["ln_ffn"][0], 1e-5)),
                    "act": (inter["act"], oracle.dual_swiglu(inter["ln_ffn"], w["w_gate"][0], w["w_up"][0])),
                    "hidden": (hid, oracle.gemm(inter["act"], w["w_down"][0], inter["o_out"], 1.0, 1.0)),
                }
                for name, (got, ref) in checks.items():
                    e1 = _max_rel(got, ref)
                    print(f"  teacher-forced {name}: max-norm relative error {e1:.2e}", flush=True)
                    assert e1 < 2e-3, (pt, name, e1)
        assert len(set(s0.tolist())) > n // 2          # the decode rows really were fed distinct tokens
        for l in range(shape.layers):
            wrote_ref = (pools_ref[l] != kv_after0[l]).any(axis=(3, 4))       # [page, k/v, entry]
            wrote_got = (kv[l] != kv_after0[l]).any(axis=(3, 4))
            assert np.array_equal(wrote_ref, wrote_got), (pt, l, "KV slots written")
            assert wrote_got.sum() == 2 * n
            assert _max_rel(kv[l][wrote_got], pools_ref[l][wrote_ref]) < kv_tol, (pt, l, "appended K/V rows")


@pytest.mark.parametrize("weight_layout", ["row", "col"])
def test_llama3_8b_layer_64_decode_tokens(oracle, weight_layout):
    from nanoflow_amd import pllm_python as P
    shape = synth.ModelShape(layers=1, vocab=4096)                      # 8B layer dimensions
    kv_lens = np.random.default_rng(2).integers(512, 1025, size=64)
    _decode_layer_case(oracle, shape, kv_lens, seed=0, weight_layout=weight_layout,
                       pipelines=(P.PipelineType.NON_OVERLAP_LOCAL, P.PipelineType.LOCAL))


@pytest.mark.parametrize("weight_layout", ["row", "col"])
def test_llama3_70b_shaped_layer(oracle, weight_layout):
    from nanoflow_amd import pllm_python as P
    shape = synth.ModelShape(hidden=8192, Hq=64, Hkv=8, ffn=28672, vocab=2048, layers=1)
    kv_lens = np.random.default_rng(3).integers(200, 400, size=16)
    _decode_layer_case(oracle, shape, kv_lens, seed=1, pipelines=(P.PipelineType.NON_OVERLAP_LOCAL,),
                       weight_layout=weight_layout)


def test_llama3_70b_shaped_layer_with_e4m3_weights(oracle):
    from nanoflow_amd import pllm_python as P
    shape = synth.ModelShape(hidden=8192, Hq=64, Hkv=8, ffn=28672, vocab=2048, layers=1)
    kv_lens = np.random.default_rng(4).integers(200, 400, size=16)
    try:
        _decode_layer_case(oracle, shape, kv_lens, seed=2, pipelines=(P.PipelineType.NON_OVERLAP_LOCAL,),
                           weight_format="e4m3")
    finally:
        P.setWeightFormat(P.WeightFormat.F16)


def _sample_rows_cols(M, N):
    """Rows and columns a slow oracle GEMM is evaluated on: every 8th row and the last (every tile
    row of every tile height), 24 bands of 16 columns that start 8 columns before a multiple of
    256 (they straddle the tile borders of every tile width), the first and the last band."""
    rows = np.unique(np.concatenate([np.arange(0, M, 8), [M - 1]]))
    starts = [0, N - 16] + [max(((i * N // 23) // 256) * 256 - 8, 0) for i in range(1, 23)]
    cols = np.unique(np.concatenate([np.arange(c, c + 16) for c in starts]))
    return rows, cols[cols < N]


def _teacher_forced_f16(oracle, w, inter, hid, x_in):
    return {
        "ln_attn": (inter["ln_attn"], oracle.rmsnorm(x_in, w["ln_attn"][0], 1e-5)),
        "kqv": (inter["kqv"], oracle.gemm(inter["ln_attn"], w["w_kqv"][0])),
        "o_out": (inter["o_out"], oracle.gemm(inter["attn_out"], w["w_o"][0], x_in, 1.0, 1.0)),
        "ln_ffn": (inter["ln_ffn"], oracle.rmsnorm(inter["o_out"], w["ln_ffn"][0], 1e-5)),
        "act": (inter["act"], oracle.dual_swiglu(inter["ln_ffn"], w["w_gate"][0], w["w_up"][0])),
        "hidden": (hid, oracle.gemm(inter["act"], w["w_down"][0], inter["o_out"], 1.0, 1.0)),
    }


def _teacher_forced_e4m3(oracle, w, wq, inter, hid, x_in, tag):
    """Every fp8 GEMM of the layer on the rows the device operator read.  The oracle's fp8 GEMMs are
    scalar loops, so they are evaluated on sampled rows and columns (_sample_rows_cols): fp8 x fp8
    on identical quantised rows within 2e-3, fp16 activations x dequantised weights (the definition
    the fp8 tolerance is stated for) within 3e-2, the fused pair (a product of two such outputs)
    within twice that.  The WHOLE output is compared with fp32 matrix products of the dequantised
    operands computed by torch on the device (the products of two e4m3 values are exact in fp32)."""
    lut = torch.tensor([oracle.e4m3_to_float(v) for v in range(256)], dtype=torch.float32, device="cuda")
    dq = lambda q: lut[torch.from_numpy(q).cuda().long()] if q.size < (1 << 27) else torch.cat(
        [lut[torch.from_numpy(q[i:i + 2048]).cuda().long()] for i in range(0, q.shape[0], 2048)])
    t32 = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda().float()
    plain = (("kqv", "ln_attn", "w_kqv", None), ("o_out", "attn_out", "w_o", x_in), ("hidden", "act", "w_down", inter["o_out"]))
    for name, src, key, Cm in plain:
        x, got = inter[src], (hid if name == "hidden" else inter[name])
        Wq, sb = wq[key][0]
        rows, cols = _sample_rows_cols(x.shape[0], Wq.shape[0])
        Aq, sa = oracle.quantize_rows_e4m3(x)
        Cs = None if Cm is None else np.ascontiguousarray(Cm[rows][:, cols])
        beta = 0.0 if Cm is None else 1.0
        Ws, ss = np.ascontiguousarray(Wq[cols]), np.ascontiguousarray(sb[cols])
        ref8 = oracle.gemm_f8f8(np.ascontiguousarray(Aq[rows]), np.ascontiguousarray(sa[rows]), Ws, ss, Cs, 1.0, beta)
        ref16 = oracle.gemm_f8w(np.ascontiguousarray(x[rows]), np.ascontiguousarray(Ws.T), ss, Cs, 1.0, beta)
        full = (dq(Aq) @ dq(Wq).T) * t32(sa)[:, None] * t32(sb)[None, :]
        if Cm is not None:
            full += t32(Cm)
        full = full.half().cpu().numpy()
        e8, e16, ef = _max_rel(got[rows][:, cols], ref8), _max_rel(got[rows][:, cols], ref16), _max_rel(got, full)
        print(f"  {tag} teacher-forced {name}: oracle fp8 x fp8 {e8:.2e} (2e-3), oracle dequantised weights {e16:.2e} (3e-2) "
              f"on {len(rows)} x {len(cols)} samples; whole output vs fp32 products {ef:.2e} (2e-3)", flush=True)
        assert e8 < 2e-3 and e16 < 3e-2 and ef < 2e-3, (tag, name, e8, e16, ef)
    # the fused gate/up pair
    x, got = inter["ln_ffn"], inter["act"]
    (Gq, sg), (Uq, su) = wq["w_gate"][0], wq["w_up"][0]
    rows, cols = _sample_rows_cols(x.shape[0], Gq.shape[0])
    Aq, sa = oracle.quantize_rows_e4m3(x)
    As, sas, xs = np.ascontiguousarray(Aq[rows]), np.ascontiguousarray(sa[rows]), np.ascontiguousarray(x[rows])
    cut = lambda W, sc: (np.ascontiguousarray(W[cols]), np.ascontiguousarray(sc[cols]))
    (Gs, sgs), (Us, sus) = cut(Gq, sg), cut(Uq, su)
    ref8 = oracle.silu_mul(oracle.gemm_f8f8(As, sas, Gs, sgs), oracle.gemm_f8f8(As, sas, Us, sus))
    ref16 = oracle.silu_mul(oracle.gemm_f8w(xs, np.ascontiguousarray(Gs.T), sgs), oracle.gemm_f8w(xs, np.ascontiguousarray(Us.T), sus))
    A32, s_a = dq(Aq), t32(sa)[:, None]
    g = ((A32 @ dq(Gq).T) * s_a * t32(sg)[None, :]).half().float()
    u = ((A32 @ dq(Uq).T) * s_a * t32(su)[None, :]).half().float()
    full = (g * torch.sigmoid(g) * u).half().cpu().numpy()
    e8, e16, ef = _max_rel(got[rows][:, cols], ref8), _max_rel(got[rows][:, cols], ref16), _max_rel(got, full)
    print(f"  {tag} teacher-forced act: oracle fp8 x fp8 {e8:.2e} (2e-3), oracle dequantised weights {e16:.2e} (6e-2); "
          f"whole output vs fp32 products {ef:.2e} (2e-3)", flush=True)
    assert e8 < 2e-3 and e16 < 6e-2 and ef < 2e-3, (tag, "act", e8, e16, ef)
    for name, src, key in (("ln_attn", None, "ln_attn"), ("ln_ffn", "o_out", "ln_ffn")):
        ref = oracle.rmsnorm(x_in if src is None else inter[src], w[key][0], 1e-5)
        assert _max_rel(inter[name], ref) < 2e-3, (tag, name)


def _full_width_iteration(oracle, shape, batch, schedules, weight_format="f16", seed=11):
    """One iteration of `batch` through ONE full-width decoder layer on each schedule of
    `schedules` = ((pipeline type, (nano1, kqv1, kqv3)[, weight layout "row" | "col"]), ...), against
    the oracle (one oracle forward serves them all: the layouts hold the same matrices).

    fp16 weights: the residual stream end to end and the appended K / V rows within 2e-3 on every
    schedule, sampled ids; on the schedules that expose their whole-iteration buffers (the sequential
    one and the four-way one) every operator against the oracle's operator on the rows the device
    operator read, 2e-3 each.  e4m3 weights: the operators teacher-forced the same way
    (_teacher_forced_e4m3); the schedules must agree with each other."""
    from nanoflow_amd import engine, pllm_python as P
    nd, T = batch.decodePrefillBorder, batch.tokens
    w = synth.make_weights(shape, seed=0)
    w["embedding"] = synth.normal_f16(np.random.default_rng(1), (shape.vocab, shape.hidden), 1.0)
    tok = batch.input_tokens.copy()
    tok[:nd] = 1                                   # first iteration: decode rows are fed token id 1
    d = batch.as_dict()
    d["input_tokens"] = tok
    x_in = oracle.embedding(tok.astype(np.int32), w["embedding"])
    e4m3 = weight_format == "e4m3"
    wq = oracle.quantize_model_weights(w) if e4m3 else None
    ref = None
    first_hid = None
    # where each token's K / V row lands: (page, entry)
    page_of = batch.kv_indices[batch.kv_indptr[batch.rev_input_indptr] + batch.per_token_offset // 16]
    entry_of = batch.per_token_offset % 16
    gidx = lambda a: torch.from_numpy(a.astype(np.int64)).cuda()
    names = ("ln_attn", "kqv", "attn_out", "o_out", "ln_ffn", "act")
    try:
        for pt, split, *rest in schedules:
            layout = rest[0] if rest else "row"
            masks = rest[1] if len(rest) > 1 else {}          # CU partition of the two streams (environment of the pipeline)
            tag = f"{pt.name} {weight_format} {layout}" + (f" CUs {masks}" if masks else "")
            saved_env = {k: os.environ.get(k) for k in ("NANOFLOW_GEMM_CUS", "NANOFLOW_GEMV_CUS")}
            for k in saved_env:
                os.environ.pop(k, None)
            os.environ.update({k: str(v) for k, v in masks.items()})
            print(f"full-width iteration against the oracle: hidden={shape.hidden} rows={T} ({nd} decode) {tag}", flush=True)
            G = (T + 63) // 64 * 64
            with engine.Engine(shape, pt, global_batch=G, nano1=split[0], kqv1=split[1], kqv3=split[2],
                               kv_pages=batch.num_pages, weights=w, seed=seed, weight_format=weight_format,
                               weight_layout=layout) as e:  # KV pool: N(0, 1) drawn on the device
                if ref is None:
                    kv0 = e.kv[0][:batch.num_pages].cpu().numpy()
                e.update(batch, keep_token_list=np.ones(nd, np.int32))
                ids = e.run().copy()
                hid = e.buffer("hidden").cpu().numpy()[:T]
                inter = {k: e.buffer(k).cpu().numpy()[:T] for k in names} if (pt.is_sequential or pt.is_four_way) else {}
                k_rows = e.kv[0][gidx(page_of), 0, gidx(entry_of)].cpu().numpy()
                v_rows = e.kv[0][gidx(page_of), 1, gidx(entry_of)].cpu().numpy()
            for k, v in saved_env.items():
                os.environ.pop(k, None)
                if v is not None:
                    os.environ[k] = v
            if ref is None:
                if e4m3:
                    ref = (None, None, None, None)
                else:
                    print(f"  oracle forward (one layer, {T} rows)", flush=True)
                    pool_ref = kv0                               # appended in place
                    hid_ref, _, samp_ref = oracle.decoder_forward(shape.as_dict(), w, [pool_ref], d, want_logits=False)
                    ref = (hid_ref, samp_ref, pool_ref[page_of, 0, entry_of], pool_ref[page_of, 1, entry_of])
            if not e4m3:
                err = _max_rel(hid, ref[0])
                print(f"  {tag} residual stream max-norm relative error {err:.2e}", flush=True)
                assert err < LAYER_RTOL, (pt, err)
                assert _max_rel(k_rows, ref[2]) < 2e-3 and _max_rel(v_rows, ref[3]) < 2e-3, pt
                assert (ids == ref[1]).mean() > 0.97, (pt, (ids == ref[1]).mean())      # argmax near-ties may flip
                if inter:
                    for name, (got, want) in _teacher_forced_f16(oracle, w, inter, hid, x_in).items():
                        e1 = _max_rel(got, want)
                        print(f"  {tag} teacher-forced {name}: max-norm relative error {e1:.2e}", flush=True)
                        assert e1 < 2e-3, (pt, name, e1)
            else:
                assert inter, "e4m3 parity is teacher-forced: use schedules that expose their buffers"
                _teacher_forced_e4m3(oracle, w, wq, inter, hid, x_in, tag)
                # appended rows: K / V of the QKV output the device computed, rotated / copied by the oracle
                kdim = shape.Hkv * shape.d
                assert np.array_equal(v_rows.reshape(T, -1), inter["kqv"][:, kdim:2 * kdim]), (pt, "V rows are copies")
                if first_hid is None:
                    first_hid = hid
                else:
                    dd = hid.astype(np.float64) - first_hid.astype(np.float64)
                    rms = np.sqrt((dd ** 2).mean() / (first_hid.astype(np.float64) ** 2).mean())
                    print(f"  {tag} residual stream vs the first schedule: rms {rms:.2e}, identical {np.array_equal(hid, first_hid)}", flush=True)
                    assert rms < 8e-2, (pt, rms)      # re-quantisation makes the layer discontinuous: statistical agreement
    finally:
        P.setWeightFormat(P.WeightFormat.F16)


def test_one_iteration_workload_matches_oracle_at_full_width(oracle):
    """The one-iteration workload itself -- 2048 tokens = 1792 decode rows (KV 1024-1536, permuted page
    table, 9.4 GB of KV in the layer) + one 256-token prefill chunk -- through ONE full-width 8B layer,
    against the oracle: the sequential schedule and the reference's main schedule with its default
    split for this batch (nano-batches 640 + 1408, QKV / attention cuts 256 | 384 | 768 | 640:
    pipeline/include/vortexData.cuh:129-132), operator by operator on the rows the device operator
    read (2e-3 each) and end to end.  The appended K and V rows are compared too."""
    from nanoflow_amd import pllm_python as P
    shape = synth.ModelShape(layers=1, vocab=4096)
    batch = synth.config2_batch(seed=0, vocab=shape.vocab)
    assert batch.tokens == 2048 and batch.decodePrefillBorder == 1792
    _full_width_iteration(oracle, shape, batch, ((P.PipelineType.NON_OVERLAP_LOCAL, (1024, 512, 512), "row"),
                                                 (P.PipelineType.NON_OVERLAP_LOCAL, (1024, 512, 512), "col"),
                                                 (P.PipelineType.PLLM, (640, 256, 768), "row"),
                                                 (P.PipelineType.PLLM, (640, 256, 768), "col")))


LLAMA3_70B_LAYER = dict(hidden=8192, Hq=64, Hkv=8, ffn=28672, vocab=2048, layers=1)


@pytest.mark.parametrize("weight_format", ["f16", "e4m3"])
def test_llama3_70b_layer_on_the_dense_iteration_mix(oracle, weight_format):
    """The 70B configurations at their own row counts: 2048 tokens = 1792 decode rows (KV 1024-1536)
    + one 256-token prefill chunk through one full-width 70B layer (QKV 2048 x 10240 x 8192, gate/up
    2048 x 28672 x 8192, down 2048 x 8192 x 28672), fp16 and e4m3 weights, on the sequential schedule
    and on the reference's main schedule with the split its 70B pipeline files use
    (pipeline/config_all/llama3-70B/2048.json:50-53: nano-batch 1 = 640, QKV cuts 256 and 768)."""
    from nanoflow_amd import pllm_python as P
    shape = synth.ModelShape(**LLAMA3_70B_LAYER)
    batch = synth.config2_batch(seed=3, vocab=shape.vocab)
    assert batch.tokens == 2048 and batch.decodePrefillBorder == 1792
    layouts = ("row", "col") if weight_format == "f16" else ("col",)     # e4m3: only the LM head follows the layout
    _full_width_iteration(oracle, shape, batch,
                          [(P.PipelineType.NON_OVERLAP_LOCAL, (1024, 512, 512), lay) for lay in layouts] +
                          [(P.PipelineType.PLLM, (640, 256, 768), layouts[-1])], weight_format=weight_format)


def _offline_steady_state_batch(vocab, kv_pages=98304, T=2048, cycles=1300):
    """The batch the C++ former forms in the steady state of the offline workload (requests of 1024
    prompt tokens / 512 outputs, at most 2048 tokens per iteration): the scheduler is advanced
    without GPU work, as the reference's evaluation does with --skip_cycles (placeholder outputs),
    then one batch is taken: about 684 decode rows and prefill chunks that continue earlier ones."""
    from nanoflow_amd import pllm_python as P
    former = P.BatchFormer(kv_pages, 16, T, 1024, 512, 512, 1024, 512)
    rng = np.random.default_rng(5)
    for i in range(4096):
        former.add_request(i, rng.integers(0, vocab, size=1024), 512)
    for _ in range(cycles):
        former.schedule()
        former.form()
        former.advance(0.0, placeholder_zero=True)
    former.schedule()
    b = former.form()
    former.close()
    nd = b["decodePrefillBorder"]
    pages_per = np.diff(b["kv_indptr"])
    tokens = np.concatenate([np.ones(nd, np.int32), b["input_tokens"]]).astype(np.int32)
    return synth.Batch(decodePrefillBorder=nd, prefillNum=b["prefillNum"], prefillTokensNum=b["prefillTokensNum"],
                       input_tokens=tokens, input_indptr=b["input_indptr"], rev_input_indptr=b["rev_input_indptr"],
                       per_token_offset=b["per_token_offset"], kv_indptr=b["kv_indptr"], kv_indices=b["kv_indices"],
                       kv_last_page_len=b["kv_last_page_len"],
                       kv_len=((pages_per - 1) * 16 + b["kv_last_page_len"]).astype(np.int32), num_pages=kv_pages)


def test_overlapped_schedules_on_cu_masked_streams_at_full_width(oracle):
    """The two overlapped schedules -- LocalPipeline (two nano-batches) and the reference's main schedule
    (four QKV / attention nano-batches, 640 | 256 | 768) -- with their dense and attention streams on
    disjoint CU sets (20 + 12 and 16 + 16 CUs of every XCD, hipExtStreamCreateWithCUMask), on the dense
    2048-token iteration through one full-width 8B layer: against the oracle end to end, and (four-way
    schedule) operator by operator.  Where a workgroup runs must not change the result."""
    from nanoflow_amd import pllm_python as P
    shape = synth.ModelShape(layers=1, vocab=4096)
    batch = synth.config2_batch(seed=0, vocab=shape.vocab)
    _full_width_iteration(oracle, shape, batch, (
        (P.PipelineType.LOCAL, (1024, 512, 512), "col", {"NANOFLOW_GEMM_CUS": 160, "NANOFLOW_GEMV_CUS": 96}),
        (P.PipelineType.PLLM, (640, 256, 768), "col", {"NANOFLOW_GEMM_CUS": 160, "NANOFLOW_GEMV_CUS": 96}),
        (P.PipelineType.PLLM, (640, 256, 768), "col", {"NANOFLOW_GEMM_CUS": 128, "NANOFLOW_GEMV_CUS": 128})))


def test_llama3_8b_layer_on_the_offline_steady_state_batch(oracle):
    """The headline workload's own mix: the batch the C++ former forms in the steady state of the
    offline run (about 684 decode rows with KV 1024-1535 and prefill chunks, the first of which
    continues a prompt whose earlier chunks are already in the KV pool) through one full-width 8B
    layer, on the sequential schedule (the benchmark's default; operator by operator) and on
    LocalPipeline (the nano-batch border cuts a prefill request)."""
    from nanoflow_amd import pllm_python as P
    shape = synth.ModelShape(layers=1, vocab=4096)
    batch = _offline_steady_state_batch(shape.vocab)
    nd, pre = batch.decodePrefillBorder, batch.prefillNum
    prev = batch.per_token_offset[batch.input_indptr[nd:nd + pre]]     # KV already present per prefill request
    print(f"steady-state batch: {nd} decode rows, {pre} prefill requests of {np.diff(batch.input_indptr[nd:]).tolist()} tokens "
          f"continuing at {prev.tolist()}", flush=True)
    assert 600 < nd < 760 and batch.tokens > 1900 and pre >= 2 and prev.max() > 0
    _full_width_iteration(oracle, shape, batch, ((P.PipelineType.NON_OVERLAP_LOCAL, (1024, 512, 512), "col"),
                                                 (P.PipelineType.NON_OVERLAP_LOCAL, (1024, 512, 512), "row"),
                                                 (P.PipelineType.LOCAL, (1024, 512, 512), "col")))


def test_one_iteration_workload_is_schedule_independent_at_full_width():
    """2048 tokens = 1792 decode (KV 1024-1536) + one 256-token prefill chunk, 8B layer width,
    2 layers: the three schedules must sample the same ids and agree on the residual stream."""
    from nanoflow_amd import engine, pllm_python as P
    shape = synth.ModelShape(layers=2, vocab=8192)
    batch = synth.config2_batch(seed=0, vocab=shape.vocab)
    assert batch.tokens == 2048 and batch.decodePrefillBorder == 1792
    results = {}
    for pt in (P.PipelineType.NON_OVERLAP_LOCAL, P.PipelineType.NANOBATCH_LOCAL, P.PipelineType.LOCAL):
        print(f"full-width iteration pipeline={pt.name}", flush=True)
        with engine.Engine(shape, pt, global_batch=2048, nano1=1024, kqv1=512, kqv3=512,
                           kv_pages=batch.num_pages, seed=7) as e:      # device-generated weights / KV, same seed
            e.update(batch)
            ids = e.run()
            hid = e.buffer("hidden").cpu().numpy()[:batch.tokens]
        results[pt] = (ids.copy(), hid)
        assert ids.shape == (1793,) and (ids >= 0).all() and (ids < shape.vocab).all()
        assert np.isfinite(hid).all()
    base = results[P.PipelineType.NON_OVERLAP_LOCAL]
    for pt, (ids, hid) in results.items():
        assert _max_rel(hid, base[1]) < 2e-3, pt
        agree = (ids == base[0]).mean()
        assert agree > 0.995, (pt, agree)       # argmax near-ties may flip under a different row partition


def test_decode_attention_page_permutation_invariance_at_full_size():
    from nanoflow_amd import kernels as K
    K.lib()
    shape = synth.LLAMA3_8B
    b = synth.config2_batch(seed=0)
    nd = b.decodePrefillBorder
    g = torch.Generator(device="cuda").manual_seed(1)
    pool = torch.empty((b.num_pages, 2, 16, shape.Hkv, shape.d), dtype=torch.float16, device="cuda").normal_(0, 1, generator=g)
    q = torch.empty((nd, shape.Hq * shape.d), dtype=torch.float16, device="cuda").normal_(0, 1, generator=g)
    t = lambda x: torch.from_numpy(np.ascontiguousarray(x)).cuda()
    ws = torch.empty(1 << 20, dtype=torch.uint8, device="cuda")
    qi = t(np.arange(nd + 1, dtype=np.int32))

    def run(pool_, indices):
        o = torch.zeros_like(q)
        K.attention_paged(q, qi, pool_, t(b.kv_indptr[:nd + 1]), t(indices), t(b.kv_last_page_len[:nd]),
                          shape.Hq, shape.Hkv, causal=False, out=o, batch=nd, max_qo_rows=nd, workspace=ws)
        torch.cuda.synchronize()
        return o
    o1 = run(pool, b.kv_indices)
    perm = torch.randperm(b.num_pages, generator=torch.Generator().manual_seed(5))
    pool2 = torch.empty_like(pool)
    pool2[perm.cuda()] = pool                              # page p moves to perm[p]
    o2 = run(pool2, perm.numpy()[b.kv_indices].astype(np.int32))
    assert torch.equal(o1, o2)
    assert torch.isfinite(o1).all() and o1.abs().max() > 0
    # a sample of requests (the pool spans more than 4 GiB; the highest page ids included) against
    # fp32 softmax attention in plain PyTorch on the gathered pages
    assert pool.numel() * 2 > (4 << 30)
    top = int(np.argmax([b.kv_indices[b.kv_indptr[r]:b.kv_indptr[r + 1]].max() for r in range(nd)]))
    group = shape.Hq // shape.Hkv
    for r in sorted({0, nd // 3, nd - 1, top}):
        pages = t(b.kv_indices[b.kv_indptr[r]:b.kv_indptr[r + 1]].astype(np.int64))
        kv_len = (len(pages) - 1) * 16 + int(b.kv_last_page_len[r])
        k = pool[pages, 0].reshape(-1, shape.Hkv, shape.d)[:kv_len].float()          # [keys, Hkv, d]
        v = pool[pages, 1].reshape(-1, shape.Hkv, shape.d)[:kv_len].float()
        qr = q[r].view(shape.Hkv, group, shape.d).float()                               # q head = kv head * group + g
        p_ = torch.softmax(torch.einsum("hgd,khd->hgk", qr, k) / np.sqrt(shape.d), dim=-1)
        ref = torch.einsum("hgk,khd->hgd", p_, v).reshape(-1)
        err = (o1[r].float() - ref).abs().max().item()
        assert err <= 2e-3 * ref.abs().max().item() + 1e-6, (r, err)


def test_fp8_gemm_at_70b_ffn_shape(oracle):
    from nanoflow_amd import kernels as K
    K.lib()
    rng = np.random.default_rng(11)
    M, N, Kd = 16, 8192, 28672                                 # down projection of the 70B shape
    A = rng.normal(0, 1, (M, Kd)).astype(np.float16)
    W = rng.normal(0, 0.02, (N, Kd)).astype(np.float32)
    sc = (np.abs(W).max(axis=1) / 448.0).astype(np.float32)
    Wq = torch.from_numpy(W / sc[:, None]).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    q, s = K.quantize_rows_e4m3(dev(A))
    q_ref, s_ref = oracle.quantize_rows_e4m3(A)
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy(), q_ref) and np.array_equal(s.cpu().numpy(), s_ref)
    got = K.gemm_f8(q, s, dev(Wq), dev(sc)).cpu().numpy()
    ref = oracle.gemm_f8f8(q_ref, s_ref, Wq, sc)
    assert _max_rel(got, ref) < 2e-3
    full = oracle.gemm_f8w(A, np.ascontiguousarray(Wq.T), sc)   # fp16 activations, dequantised weights
    assert _max_rel(got, full) < 3e-2


def _e4m3_lut(oracle):
    return torch.tensor([oracle.e4m3_to_float(v) for v in range(256)], dtype=torch.float32, device="cuda")


@pytest.mark.parametrize("M,N,Kd,beta", [(2048, 10240, 8192, 0.0), (2048, 8192, 8192, 1.0), (2048, 8192, 28672, 1.0)])
def test_gemm_kernels_at_the_70b_layer_shapes(oracle, M, N, Kd, beta):
    """nf_gemm_f16 and nf_gemm_f8_f16 at the 70B layer's QKV, O and down-projection shapes with all
    2048 rows (the 256 x 256 tiles, K = 8192 and 28672): fp16 against the oracle on the whole output;
    fp8 x fp8 against the oracle on sampled rows and columns and against fp32 products of the
    dequantised operands on the whole output."""
    from nanoflow_amd import kernels as K
    K.lib()
    g = torch.Generator(device="cuda").manual_seed(M + N + Kd)
    A = torch.empty((M, Kd), dtype=torch.float16, device="cuda").normal_(0, 1, generator=g)
    W = torch.empty((Kd, N), dtype=torch.float16, device="cuda").normal_(0, 0.02, generator=g)
    Cm = torch.empty((M, N), dtype=torch.float16, device="cuda").normal_(0, 1, generator=g) if beta else None
    print(f"fp16 GEMM {M} x {N} x {Kd} beta={beta}", flush=True)
    got = K.gemm(A, W, Cm, 1.0, beta).cpu().numpy()
    ref = oracle.gemm(A.cpu().numpy(), W.cpu().numpy(), None if Cm is None else Cm.cpu().numpy(), 1.0, beta)
    err = _max_rel(got, ref)
    print(f"  fp16 vs oracle {err:.2e}", flush=True)
    assert err < 2e-3
    print(f"fp8 GEMM {M} x {N} x {Kd} beta={beta}", flush=True)
    Aq, sa = K.quantize_rows_e4m3(A)
    Wq, sb = K.quantize_weight_e4m3(W)                     # [N, K] e4m3 + per-output-channel scales
    got = K.gemm_f8(Aq, sa, Wq, sb, Cm, 1.0, beta)
    lut = _e4m3_lut(oracle)
    full = (lut[Aq.long()] @ lut[Wq.long()].T) * sa[:, None] * sb[None, :]
    if Cm is not None:
        full += Cm.float()
    ef = _max_rel(got.cpu().numpy(), full.half().cpu().numpy())
    rows, cols = _sample_rows_cols(M, N)
    r_t, c_t = torch.from_numpy(rows).cuda(), torch.from_numpy(cols).cuda()
    cpu = lambda t: np.ascontiguousarray(t.cpu().numpy())
    ref8 = oracle.gemm_f8f8(cpu(Aq[r_t]), cpu(sa[r_t]), cpu(Wq[c_t]), cpu(sb[c_t]),
                            None if Cm is None else cpu(Cm[r_t][:, c_t]), 1.0, beta)
    e8 = _max_rel(cpu(got[r_t][:, c_t]), ref8)
    print(f"  fp8 x fp8 vs oracle on {len(rows)} x {len(cols)} samples {e8:.2e}, whole output vs fp32 products {ef:.2e}", flush=True)
    assert e8 < 2e-3 and ef < 2e-3


def test_gate_up_pair_at_the_70b_shape(oracle):
    """The fused gate/up launch at 2048 x 28672 x 8192, fp16 (whole output against the oracle) and
    fp8 x fp8 (sampled against the oracle, whole output against fp32 products)."""
    from nanoflow_amd import kernels as K
    K.lib()
    M, N, Kd = 2048, 28672, 8192
    g = torch.Generator(device="cuda").manual_seed(9)
    A = torch.empty((M, Kd), dtype=torch.float16, device="cuda").normal_(0, 1, generator=g)
    G = torch.empty((Kd, N), dtype=torch.float16, device="cuda").normal_(0, 0.02, generator=g)
    U = torch.empty((Kd, N), dtype=torch.float16, device="cuda").normal_(0, 0.02, generator=g)
    print("fp16 gate/up pair 2048 x 28672 x 8192", flush=True)
    got = K.dual_swiglu(A, G, U).cpu().numpy()
    ref = oracle.dual_swiglu(A.cpu().numpy(), G.cpu().numpy(), U.cpu().numpy())
    err = _max_rel(got, ref)
    print(f"  fp16 vs oracle {err:.2e}", flush=True)
    assert err < 2e-3
    print("fp8 gate/up pair 2048 x 28672 x 8192", flush=True)
    Aq, sa = K.quantize_rows_e4m3(A)
    (Gq, sg), (Uq, su) = K.quantize_weight_e4m3(G), K.quantize_weight_e4m3(U)
    del G, U
    got = K.dual_swiglu_f8(Aq, sa, Gq, sg, Uq, su)
    lut = _e4m3_lut(oracle)
    A32 = lut[Aq.long()]
    gg = ((A32 @ lut[Gq.long()].T) * sa[:, None] * sg[None, :]).half().float()
    uu = ((A32 @ lut[Uq.long()].T) * sa[:, None] * su[None, :]).half().float()
    full = (gg * torch.sigmoid(gg) * uu).half().cpu().numpy()
    ef = _max_rel(got.cpu().numpy(), full)
    rows, cols = _sample_rows_cols(M, N)
    r_t, c_t = torch.from_numpy(rows).cuda(), torch.from_numpy(cols).cuda()
    cpu = lambda t: np.ascontiguousarray(t.cpu().numpy())
    As, sas = cpu(Aq[r_t]), cpu(sa[r_t])
    ref8 = oracle.silu_mul(oracle.gemm_f8f8(As, sas, cpu(Gq[c_t]), cpu(sg[c_t])), oracle.gemm_f8f8(As, sas, cpu(Uq[c_t]), cpu(su[c_t])))
    e8 = _max_rel(cpu(got[r_t][:, c_t]), ref8)
    print(f"  fp8 x fp8 vs oracle on {len(rows)} x {len(cols)} samples {e8:.2e}, whole output vs fp32 products {ef:.2e}", flush=True)
    assert e8 < 2e-3 and ef < 2e-3
