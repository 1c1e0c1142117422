"""The extension module `pllm_python` (nanoflow_amd/ext) driven the way the reference's Python
drives its own: the call sequence of pipeline/utils/serve_8B.py:124-146 (init_pipe) and :452-500
(update / run_async / run_async_wait / getPipelineOutput) with the helpers of
pipeline/utils/pybindUtil.py:40-112 and weightLoader.py:13-24 restated here, on HOST weights that
init() uploads.  Two chained iterations against the oracle."""
import os
import sys

import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

from nanoflow_amd import synth  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
E2E_RTOL = 1e-2


@pytest.fixture(scope="module")
def pllm_python():
    ext = os.path.join(ROOT, "nanoflow_amd", "ext")
    assert any(f.startswith("pllm_python.") for f in os.listdir(ext)), "build the extension: make -C nanoflow_amd/csrc"
    sys.path.insert(0, ext)
    try:
        import pllm_python as mod
    finally:
        sys.path.remove(ext)
    return mod


def to_vortex_weight(P, tensor):
    w = P.VortexWeight()
    if tensor.dim() == 2:
        w.N, w.K = tensor.size(0), tensor.size(1)
    else:
        w.N, w.K = 1, tensor.size(0)
    w.setPtr(tensor.data_ptr())
    return w


def test_module_has_exactly_the_reference_surface(pllm_python):
    names = {n for n in dir(pllm_python) if not n.startswith("_")}
    assert names == {"PipelineType", "VortexConfigData", "VortexInitData", "VortexLayerWeight", "VortexModelWeight",
                     "VortexOutputData", "VortexUpdateData", "VortexWeight", "config", "createInitData",
                     "createModelWeight", "finalize", "getPipelineOutput", "init", "run", "run_async",
                     "run_async_wait", "setModelConfig", "setRank", "update"}
    assert {m for m in pllm_python.PipelineType.__members__} == {
        "PLLM", "NONOVERLAP", "NANOBATCH", "PLLMOFFLOAD", "LOCAL", "NON_OVERLAP_LOCAL", "NANOBATCH_LOCAL",
        "NONOVERLAP_KQVBIAS", "NANOBATCH_KQVBIAS", "KQVBIAS"}


def test_empty_weight_flow_runs_on_the_host_memory_createModelWeight_hands_out(pllm_python, tmp_path):
    """serve_8B.py --empty_weight True (:629-634): createModelWeight allocates the weights (host memory,
    zero-filled here), init uploads them, an iteration runs and samples one id per request."""
    from nanoflow_amd import engine, pllm_python as face
    P = pllm_python
    shape = synth.tiny_shape(layers=2, vocab=1024, Hq=8, Hkv=2, ffn=512)
    b = synth.make_batch([5, 9, 17], [(0, 20)], vocab=shape.vocab, seed=3, extra_pages=8)
    cfg = str(tmp_path / "pipe.json")
    engine.write_config(cfg, shape, global_batch=64, nano1=32, kqv1=16, kqv3=16,
                        pipeline_type=face.PipelineType.LOCAL, kv_pages=b.num_pages)
    P.setModelConfig(cfg)
    P.setRank(1, 1)
    mw = P.VortexModelWeight()
    P.createModelWeight(mw, 0)
    assert len(mw.layer_weight) == shape.layers
    assert mw.embedding.N * mw.embedding.K == shape.vocab * shape.hidden
    assert mw.layer_weight[1].W_D.N * mw.layer_weight[1].W_D.K == shape.ffn * shape.hidden
    data = P.VortexInitData()
    P.createInitData(data, mw, 0)
    assert data.tmp_buffer_size > 0
    print("pybind module, empty-weight flow", flush=True)
    P.init([data], P.PipelineType.LOCAL)
    try:
        c = P.VortexConfigData()
        c.setGemmOpTag([engine.DEFAULT_TAG] * 7)
        c.globalBatchSize, c.nanobatch1Size, c.kqv1Size, c.kqv3Size = 64, 32, 16, 16
        P.config([c])
        pin = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.int32)).pin_memory()
        nd = b.decodePrefillBorder
        t = [pin(b.input_tokens[nd:]), pin(b.input_indptr), pin(b.rev_input_indptr), pin(b.per_token_offset),
             pin(b.kv_indptr), pin(b.kv_indices), pin(b.kv_last_page_len), pin(np.ones(nd))]
        u = P.VortexUpdateData()
        u.setGemvBatchSize(np.array(synth.gemv_batch_split(nd, 16, 32, 16), dtype=np.int32))
        u.setGemvNumBlocks(np.array([108] * 4, dtype=np.int32))
        u.setInputEmbedding(t[0].data_ptr()); u.setInputIndptr(t[1].data_ptr()); u.setRevInputIndptr(t[2].data_ptr())
        u.setPerTokenOffset(t[3].data_ptr()); u.setKVIndptr(t[4].data_ptr()); u.setKVIndices(t[5].data_ptr())
        u.setKVLastPageLen(t[6].data_ptr()); u.setKeepTokenList(t[7].data_ptr())
        u.decodePrefillBorder, u.prefillNum, u.prefillTokensNum, u.keepTokenListLength = nd, b.prefillNum, b.prefillTokensNum, nd
        P.update([u])
        P.run_async()
        P.run_async_wait()
        out = np.array(P.getPipelineOutput())
        assert out.shape == (b.req_num,) and len(set(out.tolist())) == 1     # all-zero logits: one id for every row
    finally:
        P.finalize()


@pytest.mark.parametrize("pt_name", ["LOCAL", "NON_OVERLAP_LOCAL"])
def test_reference_call_sequence_on_host_weights_matches_oracle(pllm_python, oracle, tmp_path, pt_name):
    from nanoflow_amd import engine, pllm_python as face
    P = pllm_python
    shape = synth.tiny_shape(layers=2, vocab=1024, Hq=8, Hkv=2, ffn=512)
    T, nano1 = 96, 40
    b1 = synth.make_batch(list(range(5, 25)), [(7, 30), (0, 46)], vocab=shape.vocab, seed=21, extra_pages=40)
    cfg = str(tmp_path / "pipe.json")
    engine.write_config(cfg, shape, global_batch=T, nano1=nano1, kqv1=20, kqv3=28,
                        pipeline_type=face.PipelineType[pt_name], kv_pages=b1.num_pages,
                        n_tags=7 if pt_name == "LOCAL" else 4)
    print(f"pybind module, pipeline {pt_name}", flush=True)
    P.setModelConfig(cfg)
    P.setRank(1, 1)

    # ---- weights: torch CPU tensors -> VortexModelWeight (weightLoader.py:38-67)
    w = synth.make_weights(shape, seed=0)
    for k in ("w_kqv", "w_o", "w_gate", "w_up", "w_down"):
        w[k] = [(a.astype(np.float32) * 3).astype(np.float16) for a in w[k]]
    w["embedding"] = (w["embedding"].astype(np.float32) * 30).astype(np.float16)
    keep = []

    def tw(a):
        t = torch.from_numpy(np.ascontiguousarray(a))
        keep.append(t)
        return to_vortex_weight(P, t)
    mw = P.VortexModelWeight()
    mw.model_layernorm, mw.embedding, mw.lm_head = tw(w["model_norm"]), tw(w["embedding"]), tw(w["lm_head"])
    layers = []
    for l in range(shape.layers):
        lw = P.VortexLayerWeight()
        lw.W_O1 = tw(w["w_o"][l])
        lw.W_O2 = lw.W_O1
        lw.W_U, lw.W_G, lw.W_D = tw(w["w_up"][l]), tw(w["w_gate"][l]), tw(w["w_down"][l])
        lw.W_KQV = tw(w["w_kqv"][l])
        lw.W_LN_Attention, lw.W_LN_FFN = tw(w["ln_attn"][l]), tw(w["ln_ffn"][l])
        layers.append(lw)
    mw.layer_weight = layers

    # ---- init_pipe (serve_8B.py:131-146; genInitData / load_pipeline_config of pybindUtil.py)
    data = P.VortexInitData()
    P.createInitData(data, mw, 0)
    P.init([data], getattr(P.PipelineType, pt_name))
    c = P.VortexConfigData()
    c.setGemmOpTag([engine.DEFAULT_TAG] * (7 if pt_name == "LOCAL" else 4))
    c.globalBatchSize, c.nanobatch1Size, c.kqv1Size, c.kqv3Size = T, nano1, 20, 28
    P.config([c])
    assert c.globalBatchSize == T

    def update_data(b, keep_list, prefill_tokens):
        pin = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.int32)).pin_memory()
        t = dict(tok=pin(prefill_tokens if len(prefill_tokens) else np.zeros(1)), indptr=pin(b.input_indptr),
                 rev=pin(b.rev_input_indptr), off=pin(b.per_token_offset), kvp=pin(b.kv_indptr),
                 kvi=pin(b.kv_indices), kvl=pin(b.kv_last_page_len), keep=pin(keep_list if len(keep_list) else np.zeros(1)))
        u = P.VortexUpdateData()
        u.setGemvBatchSize(np.array(synth.gemv_batch_split(b.decodePrefillBorder, 20, nano1, 28), dtype=np.int32))
        u.setGemvNumBlocks(np.array([108] * 4, dtype=np.int32))
        u.setInputEmbedding(t["tok"].data_ptr())
        u.setInputIndptr(t["indptr"].data_ptr())
        u.setKVIndices(t["kvi"].data_ptr())
        u.setKVIndptr(t["kvp"].data_ptr())
        u.setKVLastPageLen(t["kvl"].data_ptr())
        u.decodePrefillBorder, u.prefillNum = b.decodePrefillBorder, b.prefillNum
        u.setRevInputIndptr(t["rev"].data_ptr())
        u.setPerTokenOffset(t["off"].data_ptr())
        u.setKeepTokenList(t["keep"].data_ptr())
        u.keepTokenListLength, u.prefillTokensNum = len(keep_list), b.prefillTokensNum
        return u, t

    try:
        # iteration 1: decode rows are fed token id 1 (nothing sampled yet), KV pools start as zeros
        nd = b1.decodePrefillBorder
        u1, hold1 = update_data(b1, np.ones(nd, np.int32), b1.input_tokens[nd:])
        P.update([u1])
        P.run_async()
        P.run_async_wait()
        s1 = np.array(P.getPipelineOutput())
        assert s1.dtype == np.int32 and s1.shape == (b1.req_num,)
        tok1 = b1.input_tokens.copy()
        tok1[:nd] = 1
        d1 = b1.as_dict()
        d1["input_tokens"] = tok1
        pools_ref = [np.zeros((b1.num_pages, 2, 16, shape.Hkv, shape.d), np.float16) for _ in range(shape.layers)]
        _, log1, samp1 = oracle.decoder_forward(shape.as_dict(), w, pools_ref, d1, want_logits=True)
        top2 = np.sort(log1.astype(np.float32), axis=1)[:, -2:]
        clear = (top2[:, 1] - top2[:, 0]) > 2 * E2E_RTOL * np.abs(log1.astype(np.float32)).max()
        assert clear.sum() >= b1.req_num // 2
        assert np.array_equal(s1[clear], samp1[clear])

        # iteration 2: every request decodes its sample (serve_8B.py keeps all slots)
        nreq = b1.req_num
        L = b1.kv_len.astype(np.int64)
        free = [p for p in range(b1.num_pages) if p not in set(b1.kv_indices.tolist())]
        indices, indptr = [], [0]
        for r in range(nreq):
            pg = b1.kv_indices[b1.kv_indptr[r]:b1.kv_indptr[r + 1]].tolist()
            if (L[r] + 1 + 15) // 16 > len(pg):
                pg.append(free.pop())
            indices += pg
            indptr.append(len(indices))
        b2 = synth.Batch(decodePrefillBorder=nreq, prefillNum=0, prefillTokensNum=0, input_tokens=s1.astype(np.int32),
                         input_indptr=np.arange(nreq + 1, dtype=np.int32), rev_input_indptr=np.arange(nreq, dtype=np.int32),
                         per_token_offset=L.astype(np.int32), kv_indptr=np.array(indptr, np.int32),
                         kv_indices=np.array(indices, np.int32), kv_last_page_len=(L % 16 + 1).astype(np.int32),
                         kv_len=(L + 1).astype(np.int32), num_pages=b1.num_pages)
        u2, hold2 = update_data(b2, np.ones(nreq, np.int32), np.zeros(0, np.int32))
        P.update([u2])
        P.run()
        s2 = np.array(P.getPipelineOutput())
        if np.array_equal(s1, samp1):
            _, log2, samp2 = oracle.decoder_forward(shape.as_dict(), w, pools_ref, b2.as_dict(), want_logits=True)
            top2 = np.sort(log2.astype(np.float32), axis=1)[:, -2:]
            clear2 = (top2[:, 1] - top2[:, 0]) > 2 * E2E_RTOL * np.abs(log2.astype(np.float32)).max()
            assert np.array_equal(s2[clear2], samp2[clear2])
        assert s2.shape == (nreq,) and (s2 >= 0).all() and (s2 < shape.vocab).all()
    finally:
        P.finalize()
