#!/usr/bin/env python3
"""Writes tests/golden/weight_file_checksums.json: the tensors the REFERENCE's own converter
(save_weights of pipeline/utils/weightSaver.py:73-149, one rank) writes for a small synthetic
Hugging Face checkpoint -- names, shapes, dtypes and SHA-256 of the bytes.  The test converts the
same checkpoint with nanoflow_amd.weights and must produce the same file content.

Run in the build container only (imports /root/reference/pipeline/utils/weightSaver.py, which
needs nothing of the compiled extension):

    python tests/golden/make_weight_fixture.py

``build_checkpoint`` is also what the test calls: it only needs numpy, torch and safetensors.
"""
from __future__ import annotations

import hashlib
import json
import os
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
CONFIG = {"hidden_size": 256, "num_attention_heads": 2, "num_key_value_heads": 1, "intermediate_size": 512,
          "vocab_size": 384, "num_hidden_layers": 3, "rms_norm_eps": 1e-5, "rope_theta": 500000.0}


def build_checkpoint(dirpath: str, with_bias: bool) -> None:
    """A 3-layer Llama-shaped checkpoint (two safetensors shards + config.json), bf16 like the real
    ones, from a fixed numpy stream; with_bias adds q/k/v biases (the Qwen2 case)."""
    import torch
    from safetensors.torch import save_file
    rs = np.random.RandomState(20240607)
    H, F, V, d = CONFIG["hidden_size"], CONFIG["intermediate_size"], CONFIG["vocab_size"], 128
    hq, hkv = CONFIG["num_attention_heads"], CONFIG["num_key_value_heads"]
    t = lambda *shape: torch.from_numpy(rs.standard_normal(shape).astype(np.float32)).to(torch.bfloat16)
    sd = {"model.embed_tokens.weight": t(V, H), "model.norm.weight": t(H), "lm_head.weight": t(V, H)}
    for l in range(CONFIG["num_hidden_layers"]):
        p = f"model.layers.{l}."
        sd.update({p + "input_layernorm.weight": t(H), p + "post_attention_layernorm.weight": t(H),
                   p + "self_attn.q_proj.weight": t(hq * d, H), p + "self_attn.k_proj.weight": t(hkv * d, H),
                   p + "self_attn.v_proj.weight": t(hkv * d, H), p + "self_attn.o_proj.weight": t(H, hq * d),
                   p + "mlp.gate_proj.weight": t(F, H), p + "mlp.up_proj.weight": t(F, H),
                   p + "mlp.down_proj.weight": t(H, F)})
        if with_bias:
            sd.update({p + "self_attn.q_proj.bias": t(hq * d), p + "self_attn.k_proj.bias": t(hkv * d),
                       p + "self_attn.v_proj.bias": t(hkv * d)})
    os.makedirs(dirpath, exist_ok=True)
    keys = sorted(sd)
    half = len(keys) // 2
    save_file({k: sd[k].contiguous() for k in keys[:half]}, os.path.join(dirpath, "model-00001-of-00002.safetensors"))
    save_file({k: sd[k].contiguous() for k in keys[half:]}, os.path.join(dirpath, "model-00002-of-00002.safetensors"))
    json.dump(CONFIG, open(os.path.join(dirpath, "config.json"), "w"))


def describe(path: str) -> dict:
    """name -> [shape, dtype, sha256 of the contiguous bytes] of a weight_rank_0.pt."""
    import torch
    sd = torch.load(path, map_location="cpu", weights_only=True)
    out = {}
    for k in sorted(sd):
        v = sd[k].contiguous()
        raw = v.view(torch.int16).numpy().tobytes() if v.element_size() == 2 else v.numpy().tobytes()
        out[k] = [list(v.shape), str(v.dtype), hashlib.sha256(raw).hexdigest()]
    return out


def main():
    sys.path.insert(0, "/root/reference/pipeline/utils")
    work = tempfile.mkdtemp(prefix="nf_weight_fixture_")
    os.chdir(work)
    import io
    real = sys.stdout
    sys.stdout = io.StringIO()            # the converter prints every tensor
    try:
        import weightSaver
        rec = {}
        for name, bias in (("plain", False), ("qkv_bias", True)):
            hf, out = os.path.join(work, name, "hf"), os.path.join(work, name, "w")
            build_checkpoint(hf, bias)
            weightSaver.save_weights(1, 1, out, model_path=hf)
            rec[name] = describe(os.path.join(out, "weight_rank_0.pt"))
    finally:
        sys.stdout = real
    path = os.path.join(HERE, "weight_file_checksums.json")
    json.dump(rec, open(path, "w"), indent=0)
    print(path, os.path.getsize(path), "bytes;", {k: len(v) for k, v in rec.items()}, "tensors")


if __name__ == "__main__":
    main()
