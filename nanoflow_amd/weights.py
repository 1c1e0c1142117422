#!/usr/bin/env python3
"""Weight files of the reference, single-device case (nranks = vnranks = 1).

Two steps, as in the reference:

* ``convert_hf_checkpoint(hf_dir, weight_dir)`` -- pipeline/utils/weightSaver.py:73-149: reads the
  ``*.safetensors`` shards and ``config.json`` of a Hugging Face Llama checkpoint directory and writes
  ``weight_dir/weight_rank_0.pt``, a ``torch.save``d dict of tensors in the pipeline's orientation:

      Embed      [V, H]        model.embed_tokens.weight as stored ('Col', weightSaver.py:91)
      LmHead     [H, V]        lm_head.weight transposed (K x N row-major, weightSaver.py:90)
      ModelNorm  [H]
      KQV_l      [H, (Hkv + Hkv + Hq) * d]   k_proj^T | v_proj^T | q_proj^T   (weightSaver.py:113-121)
      BKQV_l     [1, (Hkv + Hkv + Hq) * d]   k | v | q biases, zeros when the checkpoint has none
      O1_l, O2_l [Hq * d, H]   o_proj^T (the two differ only in how they are split over ranks)
      G_l, U_l   [H, F]        gate_proj^T, up_proj^T
      D_l        [F, H]        down_proj^T
      LNATT_l, LNFFN_l [H]

  Layer tensors are fp16; Embed, LmHead and ModelNorm keep the checkpoint's dtype, as in the
  reference, and become fp16 on load.  A checkpoint with tied embeddings (no lm_head.weight) uses the
  embedding for the LM head.

* ``load_weight_file(weight_dir)`` -- pipeline/utils/weightLoader.py:38-67: reads ``weight_rank_0.pt``
  (with the loader that executes nothing from the file) and returns the dict ``engine.Engine`` takes
  as ``weights=``: fp16 numpy arrays, per-layer entries as lists.

BKQV_l is read only for the *_KQVBIAS pipeline types (the reference's LocalPipeline never reads
B_KQV: pipeline/src/pipeline_local.cu:862-867; its bias pipelines do, pipeline.cu:1048-1058); for
the other types a file with a non-zero BKQV_l is rejected instead of being served wrongly.

    python -m nanoflow_amd.weights --hf_path HF_SNAPSHOT_DIR --weight_path OUT_DIR
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from nanoflow_amd import synth  # noqa: E402

FILE_NAME = "weight_rank_0.pt"

_HF = {
    "ln_attention": "model.layers.{i}.input_layernorm.weight",
    "ln_ffn": "model.layers.{i}.post_attention_layernorm.weight",
    "w_q": "model.layers.{i}.self_attn.q_proj.weight",
    "w_k": "model.layers.{i}.self_attn.k_proj.weight",
    "w_v": "model.layers.{i}.self_attn.v_proj.weight",
    "w_o": "model.layers.{i}.self_attn.o_proj.weight",
    "w_g": "model.layers.{i}.mlp.gate_proj.weight",
    "w_u": "model.layers.{i}.mlp.up_proj.weight",
    "w_d": "model.layers.{i}.mlp.down_proj.weight",
    "b_q": "model.layers.{i}.self_attn.q_proj.bias",
    "b_k": "model.layers.{i}.self_attn.k_proj.bias",
    "b_v": "model.layers.{i}.self_attn.v_proj.bias",
}


def shape_from_hf_config(cfg: dict, page_size: int = 16) -> synth.ModelShape:
    """Model shape from a Hugging Face ``config.json`` dict (the ``model`` block of the reference's
    pipeline configs has the same keys: pipeline/config_all/llama3-8B/1024.json)."""
    hq = cfg["num_attention_heads"]
    return synth.ModelShape(hidden=cfg["hidden_size"], Hq=hq, Hkv=cfg.get("num_key_value_heads", hq),
                            d=cfg.get("head_dim") or cfg["hidden_size"] // hq, ffn=cfg["intermediate_size"],
                            vocab=cfg["vocab_size"], layers=cfg["num_hidden_layers"], page_size=page_size,
                            eps=cfg.get("rms_norm_eps", 1e-5), rope_theta=cfg.get("rope_theta", 1e4),
                            rope_scaling=cfg.get("rope_scaling") or None)


def _read_safetensors_dir(hf_dir: str) -> dict:
    from safetensors import safe_open
    out = {}
    files = sorted(f for f in os.listdir(hf_dir) if f.endswith(".safetensors"))
    if not files:
        raise FileNotFoundError(f"{hf_dir}: no .safetensors files")
    for name in files:
        with safe_open(os.path.join(hf_dir, name), "pt") as f:
            for key in f.keys():
                out[key] = f.get_tensor(key)
    return out


def convert_state_dict(sd: dict, num_layers: int) -> dict:
    """Hugging Face tensor names and [out, in] orientation -> the reference's weight-file dict."""
    t = lambda x: x.t().contiguous()
    embed = sd["model.embed_tokens.weight"]
    head = sd["lm_head.weight"] if "lm_head.weight" in sd else embed
    out = {"ModelNorm": sd["model.norm.weight"], "Embed": embed, "LmHead": t(head)}
    for l in range(num_layers):
        g = lambda k: sd[_HF[k].format(i=l)]
        k_t, v_t, q_t = t(g("w_k")), t(g("w_v")), t(g("w_q"))
        kqv = torch.cat([k_t, v_t, q_t], 1)
        if _HF["b_k"].format(i=l) in sd:
            bias = torch.cat([g("b_k").unsqueeze(0), g("b_v").unsqueeze(0), g("b_q").unsqueeze(0)], 1)
        else:
            bias = torch.zeros(1, kqv.shape[1])
        o_t = t(g("w_o"))
        f16 = lambda x: x.to(torch.float16)
        out.update({f"O1_{l}": f16(o_t), f"O2_{l}": f16(o_t), f"U_{l}": f16(t(g("w_u"))),
                    f"G_{l}": f16(t(g("w_g"))), f"D_{l}": f16(t(g("w_d"))), f"KQV_{l}": f16(kqv),
                    f"BKQV_{l}": f16(bias), f"LNATT_{l}": f16(g("ln_attention")),
                    f"LNFFN_{l}": f16(g("ln_ffn"))})
    return out


def convert_hf_checkpoint(hf_dir: str, weight_dir: str) -> str:
    cfg = json.load(open(os.path.join(hf_dir, "config.json")))
    out = convert_state_dict(_read_safetensors_dir(hf_dir), cfg["num_hidden_layers"])
    os.makedirs(weight_dir, exist_ok=True)
    path = os.path.join(weight_dir, FILE_NAME)
    torch.save(out, path)
    return path


def load_weight_file(weight_dir: str, shape: synth.ModelShape | None = None, kqv_bias: bool = False) -> dict:
    """``weight_dir/weight_rank_0.pt`` -> the ``weights=`` dict of engine.Engine.  With ``shape`` given,
    every tensor's shape is checked against it and a mismatch raises ValueError.  ``kqv_bias``: the
    pipeline type adds BKQV_l (one of the *_KQVBIAS types); without it a file whose biases are not
    all zero is refused, since serving it would silently drop them."""
    path = weight_dir if weight_dir.endswith(".pt") else os.path.join(weight_dir, FILE_NAME)
    sd = torch.load(path, map_location="cpu", weights_only=True)
    layer_ids = [int(m.group(1)) for m in (re.match(r"^D_(\d+)$", k) for k in sd) if m]
    if not layer_ids:
        raise ValueError(f"{path}: no D_<layer> tensors: not a pipeline weight file")
    L = max(layer_ids) + 1
    np16 = lambda x: np.ascontiguousarray(x.to(torch.float16).numpy())
    w = {"embedding": np16(sd["Embed"]), "lm_head": np16(sd["LmHead"]), "model_norm": np16(sd["ModelNorm"]).reshape(-1),
         "w_kqv": [], "w_o": [], "w_gate": [], "w_up": [], "w_down": [], "ln_attn": [], "ln_ffn": []}
    for l in range(L):
        if kqv_bias:
            if f"BKQV_{l}" not in sd:
                raise ValueError(f"{path}: no BKQV_{l}: the pipeline type adds a KQV bias")
            w.setdefault("b_kqv", []).append(np16(sd[f"BKQV_{l}"]).reshape(-1))
        elif f"BKQV_{l}" in sd and bool(torch.any(sd[f"BKQV_{l}"] != 0)):
            raise ValueError(f"{path}: layer {l} has a non-zero KQV bias; serve this model with KQVBIAS, "
                             "NONOVERLAP_KQVBIAS or NANOBATCH_KQVBIAS as serve_configs.pipeline_type")
        w["w_kqv"].append(np16(sd[f"KQV_{l}"]))
        w["w_o"].append(np16(sd[f"O1_{l}"]))
        w["w_gate"].append(np16(sd[f"G_{l}"]))
        w["w_up"].append(np16(sd[f"U_{l}"]))
        w["w_down"].append(np16(sd[f"D_{l}"]))
        w["ln_attn"].append(np16(sd[f"LNATT_{l}"]).reshape(-1))
        w["ln_ffn"].append(np16(sd[f"LNFFN_{l}"]).reshape(-1))
    if shape is not None:
        want = {"embedding": (shape.vocab, shape.hidden), "lm_head": (shape.hidden, shape.vocab),
                "model_norm": (shape.hidden,)}
        per_layer = {"w_kqv": (shape.hidden, shape.kqv_n), "w_o": (shape.Hq * shape.d, shape.hidden),
                     "w_gate": (shape.hidden, shape.ffn), "w_up": (shape.hidden, shape.ffn),
                     "w_down": (shape.ffn, shape.hidden), "ln_attn": (shape.hidden,), "ln_ffn": (shape.hidden,)}
        if kqv_bias:
            per_layer["b_kqv"] = (shape.kqv_n,)
        if L < shape.layers:
            raise ValueError(f"{path}: {L} layers, the model configuration asks for {shape.layers}")
        for k, s in want.items():
            if w[k].shape != s:
                raise ValueError(f"{path}: {k} has shape {w[k].shape}, expected {s}")
        for k, s in per_layer.items():
            for l in range(shape.layers):
                if w[k][l].shape != s:
                    raise ValueError(f"{path}: {k} of layer {l} has shape {w[k][l].shape}, expected {s}")
    return w


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--hf_path", required=True, help="Hugging Face checkpoint directory (config.json + *.safetensors)")
    ap.add_argument("--weight_path", required=True, help="directory that receives weight_rank_0.pt")
    a = ap.parse_args()
    print(convert_hf_checkpoint(a.hf_path, a.weight_path))


if __name__ == "__main__":
    main()
