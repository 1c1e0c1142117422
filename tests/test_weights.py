"""Weight files in the reference's format (pipeline/utils/weightSaver.py:73-149 and
weightLoader.py:38-67, single rank): Hugging Face checkpoint -> weight_rank_0.pt -> engine dict.
The expected tensors are written out here from the Hugging Face [out, in] convention; nothing
is computed with the converter's own code."""
import json
import os

import numpy as np
import pytest

torch = pytest.importorskip("torch")
safetensors_torch = pytest.importorskip("safetensors.torch")

from nanoflow_amd import weights as W  # noqa: E402

CFG = {"hidden_size": 256, "num_attention_heads": 2, "num_key_value_heads": 1, "intermediate_size": 512,
       "vocab_size": 384, "num_hidden_layers": 2, "rms_norm_eps": 1e-5, "rope_theta": 500000.0}


def _hf_state_dict(seed=0, tied=False, bias=False):
    g = torch.Generator().manual_seed(seed)
    H, F, V, d = CFG["hidden_size"], CFG["intermediate_size"], CFG["vocab_size"], 128
    hq, hkv = CFG["num_attention_heads"], CFG["num_key_value_heads"]
    r = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16)
    sd = {"model.embed_tokens.weight": r(V, H), "model.norm.weight": r(H)}
    if not tied:
        sd["lm_head.weight"] = r(V, H)
    for l in range(CFG["num_hidden_layers"]):
        p = f"model.layers.{l}."
        sd.update({p + "input_layernorm.weight": r(H), p + "post_attention_layernorm.weight": r(H),
                   p + "self_attn.q_proj.weight": r(hq * d, H), p + "self_attn.k_proj.weight": r(hkv * d, H),
                   p + "self_attn.v_proj.weight": r(hkv * d, H), p + "self_attn.o_proj.weight": r(H, hq * d),
                   p + "mlp.gate_proj.weight": r(F, H), p + "mlp.up_proj.weight": r(F, H),
                   p + "mlp.down_proj.weight": r(H, F)})
        if bias:
            sd.update({p + "self_attn.q_proj.bias": r(hq * d), p + "self_attn.k_proj.bias": r(hkv * d),
                       p + "self_attn.v_proj.bias": r(hkv * d)})
    return sd


def _write_checkpoint(tmp_path, sd):
    hf = tmp_path / "hf"
    hf.mkdir()
    keys = sorted(sd)
    half = len(keys) // 2      # two shards, as real checkpoints have
    safetensors_torch.save_file({k: sd[k].contiguous() for k in keys[:half]}, str(hf / "model-00001-of-00002.safetensors"))
    safetensors_torch.save_file({k: sd[k].contiguous() for k in keys[half:]}, str(hf / "model-00002-of-00002.safetensors"))
    json.dump(CFG, open(hf / "config.json", "w"))
    return str(hf)


def _f16(x):
    return x.to(torch.float16).numpy()


def test_convert_and_load_give_the_pipeline_orientation(tmp_path):
    sd = _hf_state_dict()
    out_dir = str(tmp_path / "w")
    path = W.convert_hf_checkpoint(_write_checkpoint(tmp_path, sd), out_dir)
    assert os.path.basename(path) == "weight_rank_0.pt"
    shape = W.shape_from_hf_config(CFG)
    assert (shape.hidden, shape.Hq, shape.Hkv, shape.d, shape.ffn, shape.vocab, shape.layers) == (256, 2, 1, 128, 512, 384, 2)
    w = W.load_weight_file(out_dir, shape)
    assert w["embedding"].dtype == np.float16
    assert np.array_equal(w["embedding"], _f16(sd["model.embed_tokens.weight"]))           # [V, H], as stored
    assert np.array_equal(w["lm_head"], _f16(sd["lm_head.weight"]).T)                       # [H, V]
    assert np.array_equal(w["model_norm"], _f16(sd["model.norm.weight"]))
    for l in range(2):
        p = f"model.layers.{l}."
        kqv = w["w_kqv"][l]
        assert kqv.shape == (256, 128 + 128 + 256)
        # column blocks K | V | Q, each the transposed projection: y = x . W^T
        assert np.array_equal(kqv[:, :128], _f16(sd[p + "self_attn.k_proj.weight"]).T)
        assert np.array_equal(kqv[:, 128:256], _f16(sd[p + "self_attn.v_proj.weight"]).T)
        assert np.array_equal(kqv[:, 256:], _f16(sd[p + "self_attn.q_proj.weight"]).T)
        assert np.array_equal(w["w_o"][l], _f16(sd[p + "self_attn.o_proj.weight"]).T)
        assert np.array_equal(w["w_gate"][l], _f16(sd[p + "mlp.gate_proj.weight"]).T)
        assert np.array_equal(w["w_up"][l], _f16(sd[p + "mlp.up_proj.weight"]).T)
        assert np.array_equal(w["w_down"][l], _f16(sd[p + "mlp.down_proj.weight"]).T)
        assert np.array_equal(w["ln_attn"][l], _f16(sd[p + "input_layernorm.weight"]))
        assert np.array_equal(w["ln_ffn"][l], _f16(sd[p + "post_attention_layernorm.weight"]))
        assert all(a.flags["C_CONTIGUOUS"] for a in (kqv, w["w_o"][l], w["w_down"][l]))


def test_weight_file_has_the_reference_tensor_names(tmp_path):
    out_dir = str(tmp_path / "w")
    W.convert_hf_checkpoint(_write_checkpoint(tmp_path, _hf_state_dict()), out_dir)
    sd = torch.load(os.path.join(out_dir, "weight_rank_0.pt"), weights_only=True)
    want = {"ModelNorm", "Embed", "LmHead"}
    for l in range(2):
        want |= {f"{n}_{l}" for n in ("O1", "O2", "U", "G", "D", "KQV", "BKQV", "LNATT", "LNFFN")}
    assert set(sd) == want
    assert sd["BKQV_0"].shape == (1, 512) and not bool(sd["BKQV_0"].any())
    assert sd["KQV_1"].dtype == torch.float16 and torch.equal(sd["O1_1"], sd["O2_1"])


def test_tied_embeddings_feed_the_lm_head(tmp_path):
    sd = _hf_state_dict(tied=True)
    out_dir = str(tmp_path / "w")
    W.convert_hf_checkpoint(_write_checkpoint(tmp_path, sd), out_dir)
    w = W.load_weight_file(out_dir)
    assert np.array_equal(w["lm_head"], _f16(sd["model.embed_tokens.weight"]).T)


def test_kqv_bias_is_served_by_the_bias_pipelines_and_never_dropped(tmp_path):
    out_dir = str(tmp_path / "w")
    hf = _hf_state_dict(bias=True)
    W.convert_hf_checkpoint(_write_checkpoint(tmp_path, hf), out_dir)
    sd = torch.load(os.path.join(out_dir, "weight_rank_0.pt"), weights_only=True)
    assert sd["BKQV_0"].shape == (1, 512) and bool(sd["BKQV_0"].any())       # written as K | V | Q like the weights
    with pytest.raises(ValueError, match="KQVBIAS"):                          # a plain pipeline type would drop it
        W.load_weight_file(out_dir)
    shape = W.shape_from_hf_config(CFG)
    w = W.load_weight_file(out_dir, shape, kqv_bias=True)
    for l in range(shape.layers):
        p = f"model.layers.{l}.self_attn."
        want = np.concatenate([_f16(hf[p + "k_proj.bias"]), _f16(hf[p + "v_proj.bias"]), _f16(hf[p + "q_proj.bias"])])
        assert w["b_kqv"][l].shape == (shape.kqv_n,) and np.array_equal(w["b_kqv"][l], want)


def test_trace_generator_writes_what_the_serving_command_reads(tmp_path):
    from nanoflow_amd import gen_req, serve
    p = gen_req.write_trace(str(tmp_path / "t.csv"), 50, "200:700", "512", rate=10.0, poisson=True, seed=3)
    reqs = serve.read_trace(p)
    assert len(reqs) == 50 and [r[0] for r in reqs] == list(range(50))
    assert all(200 <= len(r[1]) <= 700 and r[2] == 512 for r in reqs)
    assert all(np.array_equal(r[1], np.arange(len(r[1]))) and r[1].dtype == np.int32 for r in reqs)   # prompt 0, 1, ..., n-1
    arr = [r[3] for r in reqs]
    assert arr == sorted(arr) and 2.0 < arr[-1] < 12.0            # 50 requests at 10 per second
    p = gen_req.write_trace(str(tmp_path / "c.csv"), 8, rate=4.0)
    assert [r[3] for r in serve.read_trace(p)] == [i / 4.0 for i in range(8)]
    p = gen_req.write_trace(str(tmp_path / "o.csv"), 3)
    assert [(r[0], len(r[1]), r[2], r[3]) for r in serve.read_trace(p)] == [(0, 1024, 512, 0.0), (1, 1024, 512, 0.0),
                                                                               (2, 1024, 512, 0.0)]


def write_word_tokenizer(directory, words):
    """A word-level tokenizer directory that transformers' AutoTokenizer loads offline: ids 0.. are
    <unk>, <s>, then the words; every encoded text starts with <s>."""
    import json, os
    from tokenizers import Tokenizer, models, pre_tokenizers, processors
    vocab = {"<unk>": 0, "<s>": 1, **{w: i + 2 for i, w in enumerate(words)}}
    tok = Tokenizer(models.WordLevel(vocab, unk_token="<unk>"))
    tok.pre_tokenizer = pre_tokenizers.Whitespace()
    tok.post_processor = processors.TemplateProcessing(single="<s> $A", special_tokens=[("<s>", 1)])
    os.makedirs(directory, exist_ok=True)
    tok.save(os.path.join(directory, "tokenizer.json"))
    json.dump({"tokenizer_class": "PreTrainedTokenizerFast", "unk_token": "<unk>", "bos_token": "<s>"},
              open(os.path.join(directory, "tokenizer_config.json"), "w"))
    return vocab


def test_prompt_text_rows_are_tokenized_as_the_reference_front_end_does(tmp_path):
    """pipeline/utils/frontend.py:41-47: input_len -1 = the prompt is the text after the fourth comma
    (commas of the text included, the line's newline dropped), tokenized with the model's tokenizer."""
    from nanoflow_amd import serve
    vocab = write_word_tokenizer(str(tmp_path / "tok"), ["the", "quick", "brown", "fox", ",", "jumps", "over", "lazy", "dog"])
    tok = serve.load_tokenizer({"model": str(tmp_path / "tok")})
    assert tok is not None and serve.load_tokenizer({"model": "meta-llama/Meta-Llama-3-8B"}) is None   # a hub name: not fetched
    assert serve.load_tokenizer({"hf_path": str(tmp_path / "tok")}) is not None
    p = tmp_path / "t.csv"
    p.write_text("idx,input_len,output_len,arrival,prompt\n"
                 "0,-1,5,0.0,the quick brown fox, the lazy dog\n"
                 "1,4,6,0.5\n"
                 "2,-1,7,1.0,zebra jumps over\n")
    reqs = serve.read_trace(str(p), tok)
    v = vocab
    assert reqs[0][1].tolist() == [1, v["the"], v["quick"], v["brown"], v["fox"], v[","], v["the"], v["lazy"], v["dog"]]
    assert reqs[1][1].tolist() == [0, 1, 2, 3] and reqs[1][2:] == (6, 0.5)
    assert reqs[2][1].tolist() == [1, 0, v["jumps"], v["over"]] and reqs[2][2:] == (7, 1.0)      # unknown word -> <unk>
    assert tok.decode(reqs[0][1].tolist(), skip_special_tokens=True) == "the quick brown fox , the lazy dog"
    with pytest.raises(SystemExit, match="tokenizer"):
        serve.read_trace(str(p))


def test_shape_mismatch_and_foreign_files_raise(tmp_path):
    out_dir = str(tmp_path / "w")
    W.convert_hf_checkpoint(_write_checkpoint(tmp_path, _hf_state_dict()), out_dir)
    wrong = W.shape_from_hf_config({**CFG, "intermediate_size": 1024})
    with pytest.raises(ValueError, match="w_gate"):
        W.load_weight_file(out_dir, wrong)
    with pytest.raises(ValueError, match="layers"):
        W.load_weight_file(out_dir, W.shape_from_hf_config({**CFG, "num_hidden_layers": 3}))
    torch.save({"something": torch.zeros(3)}, str(tmp_path / "other.pt"))
    with pytest.raises(ValueError, match="not a pipeline weight file"):
        W.load_weight_file(str(tmp_path / "other.pt"))


# ---- against the reference's own converter -------------------------------------------------
# tests/golden/weight_file_checksums.json holds names, shapes, dtypes and SHA-256 of the tensors
# that save_weights of pipeline/utils/weightSaver.py wrote for the synthetic checkpoint built by
# tests/golden/make_weight_fixture.py:build_checkpoint (the script that produced the file).

def _golden():
    import importlib.util
    here = os.path.join(os.path.dirname(__file__), "golden")
    spec = importlib.util.spec_from_file_location("make_weight_fixture", os.path.join(here, "make_weight_fixture.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod, json.load(open(os.path.join(here, "weight_file_checksums.json")))


@pytest.mark.parametrize("case,bias", [("plain", False), ("qkv_bias", True)])
def test_converted_file_is_the_reference_converters_file(tmp_path, case, bias):
    mod, want = _golden()
    hf, out = str(tmp_path / "hf"), str(tmp_path / "w")
    mod.build_checkpoint(hf, bias)
    path = W.convert_hf_checkpoint(hf, out)
    got = mod.describe(path)
    assert sorted(got) == sorted(want[case])
    for name in want[case]:
        assert got[name] == want[case][name], name        # shape, dtype and every byte


def test_shipped_pipeline_files_parse_and_fit_one_mi355x():
    """nanoflow_amd/config_all/*.json: the reference's schema with gpu_num 1, sized so that weights, KV
    pool and scratch stay below 90 % of the 288 GiB of one MI355X."""
    import glob, json, os
    from nanoflow_amd import serve, pllm_python as P
    root = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "nanoflow_amd", "config_all")
    files = sorted(glob.glob(os.path.join(root, "*.json")))
    assert len(files) >= 7
    for f in files:
        cfg = json.load(open(f))
        shape, pt, (T, nano1, kqv1, kqv3), pages = serve.parse_config(cfg)
        assert T == 2048 and 0 < nano1 < T and pages % 64 == 0, f
        assert pt.has_kqv_bias == ("qwen2" in f), f
        kqv_n = shape.hidden + 2 * shape.Hkv * shape.d
        per_layer = shape.hidden * kqv_n + shape.hidden * shape.hidden + 3 * shape.hidden * shape.ffn
        fp8 = cfg["serve_configs"].get("weight_format") == "e4m3"
        weights = shape.layers * per_layer * (1 if fp8 else 2) + 2 * shape.vocab * shape.hidden * 2
        kv = shape.layers * pages * (2 * shape.page_size * shape.Hkv * shape.d * 2)
        scratch = 2 * (T * shape.hidden * 16 + T * shape.vocab * 2 + T * shape.ffn) + (1 << 30)
        assert weights + kv + scratch < 0.90 * (288 << 30), (f, weights / 1e9, kv / 1e9)
        assert kv > 0.25 * (288 << 30), (f, kv / 1e9)                      # and the pool is not a token gesture
        if "3.1" in f:
            assert shape.rope_scaling and shape.rope_scaling["factor"] == 8.0


def test_gemm_tag_layout_fields_decide_the_weight_orientation():
    """engine.layouts_of_tags: the B layout field of the per-layer tags and of the LM head's tag (the last
    one) of a pipeline file; the shipped fp16 files ask for [N][K] weights throughout, the e4m3 ones for
    the fp8 form's own layout (RowMajor tags) with a k-contiguous LM head."""
    import glob, json, os
    from nanoflow_amd import engine
    assert engine.layouts_of_tags([engine.DEFAULT_TAG] * 4) == ("row", "row")
    assert engine.layouts_of_tags([engine.DEFAULT_TAG_NK] * 7) == ("col", "col")
    assert engine.layouts_of_tags([engine.DEFAULT_TAG] * 8 + [engine.DEFAULT_TAG_NK]) == ("row", "col")
    with pytest.raises(ValueError, match="disagree"):
        engine.layouts_of_tags([engine.DEFAULT_TAG, engine.DEFAULT_TAG_NK, engine.DEFAULT_TAG, engine.DEFAULT_TAG])
    with pytest.raises(ValueError, match="malformed"):
        engine.layouts_of_tags(["128_128_32", engine.DEFAULT_TAG])
    root = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "nanoflow_amd", "config_all")
    for f in sorted(glob.glob(os.path.join(root, "*.json"))):
        cfg = json.load(open(f))
        fp8 = cfg["serve_configs"].get("weight_format") == "e4m3"
        assert engine.layouts_of_tags(cfg["pipeline_configs"]["gemm_op_tag"]) == (("row" if fp8 else "col"), "col"), f
