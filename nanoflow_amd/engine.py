"""Harness around the pipeline control plane: builds the config file, device-resident
weights / KV pools / tmp buffer, and turns a synthetic batch into update data.

Plays the part of the reference's Python glue (pipeline/utils/pybindUtil.py:63-112
``genInitData`` / ``load_pipeline_config`` / ``initUpdateData`` and the set-up half of
pipeline/utils/serve_8B.py:124-146).  torch is used only to own device memory.
"""
from __future__ import annotations

import json
import os
import tempfile

import numpy as np
import torch

from . import pllm_python as P
from . import synth

# The tag grammar of the reference's pipeline files (pipeline/include/gemmShape.cuh:5-6).  The second
# layout field is B's: RowMajor = [K][N] weights as the reference's weight files hold them,
# ColumnMajor = [N][K] (k contiguous, a Hugging Face checkpoint's own orientation).
# cta_m = cta_n = 0 leaves tile and split over K to the kernel layer's cost model; a tag that names a
# tile (and a split_k) selects the closest tile of the kernel layer's menu for launches of more than
# 512 live rows.
DEFAULT_TAG = "0_0_0_0_0_0_1_0_RowMajor_RowMajor_RowMajor"
DEFAULT_TAG_NK = "0_0_0_0_0_0_1_0_RowMajor_ColumnMajor_RowMajor"


def make_tag(tile_m=0, tile_n=0, split_k=1, layout="row") -> str:
    """A GEMM tag that names a tile and a split over K (0 x 0: the library's choice) for weights in the
    given layout; the warp and stage fields, which select nothing in this build, are filled with the
    values the reference's generator would pair with the tile (pipeline/src/generate-gemm/genGEMM.py:57-65)."""
    b = "ColumnMajor" if layout == "col" else "RowMajor"
    if not tile_m:
        return f"0_0_0_0_0_0_{max(split_k, 1)}_0_RowMajor_{b}_RowMajor"
    return f"{tile_m}_{tile_n}_64_{max(tile_m // 2, 16)}_{max(tile_n // 2, 16)}_64_{max(split_k, 1)}_3_RowMajor_{b}_RowMajor"


def tag_weight_layout(tag: str) -> str:
    """"row" ([K][N]) or "col" ([N][K]): the layout a GEMM tag gives its weight."""
    parts = tag.split("_")
    if len(parts) != 11 or parts[9] not in ("RowMajor", "ColumnMajor"):
        raise ValueError(f"malformed GEMM tag {tag!r}")
    return "col" if parts[9] == "ColumnMajor" else "row"


def layouts_of_tags(tags):
    """(layout of the per-layer GEMM weights, layout of the LM head) of a pipeline file's tag list
    (the LM head's tag is the last one in every schedule).  The per-layer tags must agree: one weight
    serves every nano-batch's GEMM of its role, and the gate/up pair, which has no tag, follows them."""
    per_layer = {tag_weight_layout(t) for t in tags[:-1]}
    if len(per_layer) != 1:
        raise ValueError("the per-layer GEMM tags disagree on B's layout (RowMajor / ColumnMajor): "
                         "a weight is stored in one orientation")
    return per_layer.pop(), tag_weight_layout(tags[-1])


def write_config(path, shape: synth.ModelShape, *, global_batch, nano1, kqv1, kqv3, pipeline_type,
                 kv_pages, run_layer=None, distinct_layers=None, max_batch=None, n_tags=7, tags=None):
    """Writes a pipeline JSON in the reference's schema (pipeline/config_all/llama3-8B/1024.json)."""
    layers = shape.layers if distinct_layers is None else distinct_layers
    cfg = {
        "model": {
            "hidden_size": shape.hidden, "intermediate_size": shape.ffn,
            "num_attention_heads": shape.Hq, "num_key_value_heads": shape.Hkv,
            "num_hidden_layers": layers, "rms_norm_eps": shape.eps, "rope_theta": shape.rope_theta,
            "rope_scaling": shape.rope_scaling, "vocab_size": shape.vocab,
        },
        "model_configs": {
            "gpu_num": 1, "run_layer": shape.layers if run_layer is None else run_layer,
            "allocate_kv_data_batch": (kv_pages + 63) // 64, "frame_page_size": shape.page_size,
            "max_batch_size": global_batch if max_batch is None else max_batch,
        },
        "pipeline_configs": {
            "gemm_op_tag": list(tags) if tags else [DEFAULT_TAG] * n_tags, "global_batch_size": global_batch,
            "nanobatch_1_size": nano1, "kqv1_size": kqv1, "kqv3_size": kqv3,
        },
        "serve_configs": {"actual_gpu_num": 1, "pipeline_type": {v: k for k, v in P.pipeline_map.items()}[pipeline_type]},
    }
    with open(path, "w") as f:
        json.dump(cfg, f, indent=1)
    return cfg


def _weight(t: torch.Tensor, N: int, K: int) -> P.VortexWeight:
    assert t.is_cuda and t.dtype == torch.float16 and t.is_contiguous() and t.numel() == N * K
    w = P.VortexWeight()
    w.setPtr(t.data_ptr())
    w.N, w.K = N, K
    return w


class Engine:
    """One pipeline on cuda:0.  ``weights`` is a dict of numpy fp16 arrays (see
    synth.make_weights) or None for N(0, 0.02) weights generated on the device."""

    def __init__(self, shape: synth.ModelShape, pipeline_type=P.PipelineType.LOCAL, *, global_batch,
                 nano1, kqv1=None, kqv3=None, kv_pages, weights=None, kv_pools=None, run_layer=None,
                 distinct_layers=None, seed=0, profiling=False, kv_fill="randn", weight_format="f16",
                 weight_layout="row", gemm_tags=None):
        """weight_layout: "row" = [K][N] weights (the reference's orientation), "col" = [N][K]
        (k contiguous): the five per-layer GEMM weights and the LM head are handed over in that
        orientation and every GEMM tag says so.  With e4m3 weights only the LM head follows it (the
        fp8 form has one layout).  gemm_tags: the tag list of a pipeline file instead; its layout
        fields then decide (layouts_of_tags).  ``weights`` is always given in the [K][N] orientation
        and turned around on the device when the layout asks for it."""
        self.shape = shape
        self.pipeline_type = pipeline_type
        # "e4m3": the five GEMM weights of every layer are quantised on the device as they are
        # made (per-output-channel scales) and only the fp8 form is kept
        self.weight_format = P.WeightFormat[weight_format.upper()]
        P.setWeightFormat(self.weight_format)
        self.T = global_batch
        self.nano1 = nano1
        self.kqv1 = nano1 if kqv1 is None else kqv1
        self.kqv3 = (global_batch - nano1) if kqv3 is None else kqv3
        self.layers = shape.layers if distinct_layers is None else distinct_layers
        self.dev = torch.device("cuda:0")
        fd, self.cfg_path = tempfile.mkstemp(suffix=".json", prefix="nanoflow_cfg_")
        os.close(fd)
        n_tags = pipeline_type.gemm_tags
        e4m3 = self.weight_format == P.WeightFormat.E4M3
        if gemm_tags is not None:
            if len(gemm_tags) != n_tags:
                raise ValueError(f"{pipeline_type.name} takes {n_tags} GEMM tags, the list has {len(gemm_tags)}")
            self.tags = list(gemm_tags)
            layer_layout, head_layout = layouts_of_tags(self.tags)
            if e4m3 and layer_layout != "row":
                raise ValueError("e4m3 weights have one layout: the per-layer GEMM tags must say RowMajor for B")
        else:
            assert weight_layout in ("row", "col"), weight_layout
            layer_layout, head_layout = ("row" if e4m3 else weight_layout), weight_layout
            tag_of = {"row": DEFAULT_TAG, "col": DEFAULT_TAG_NK}
            self.tags = [tag_of[layer_layout]] * (n_tags - 1) + [tag_of[head_layout]]
        self.weight_layout, self.lm_head_layout = layer_layout, head_layout
        write_config(self.cfg_path, shape, global_batch=global_batch, nano1=nano1, kqv1=self.kqv1,
                     kqv3=self.kqv3, pipeline_type=pipeline_type, kv_pages=kv_pages,
                     run_layer=run_layer, distinct_layers=distinct_layers, n_tags=n_tags, tags=self.tags)
        P.setRank(1, 1)
        P.setModelConfig(self.cfg_path)
        self.max_pages = P.maxPageNum()
        gen = torch.Generator(device=self.dev).manual_seed(seed)
        H, V, F, d = shape.hidden, shape.vocab, shape.ffn, shape.d
        kqv_n = shape.kqv_n

        def mk(key, layer, rows, cols, std=0.02, mean=0.0, layout="row"):
            """A [rows, cols] tensor; layout "col" stores its transpose [cols, rows] (for a GEMM
            weight [K, N]: [N][K])."""
            if weights is not None:
                a = weights[key] if layer is None else weights[key][layer]
                t = torch.from_numpy(np.ascontiguousarray(a)).to(self.dev)
                return t.t().contiguous() if layout == "col" else t
            t = torch.empty((cols, rows) if layout == "col" else (rows, cols), dtype=torch.float16, device=self.dev)
            t.normal_(mean, std, generator=gen)
            return t

        self.t = {"embedding": mk("embedding", None, V, H), "lm_head": mk("lm_head", None, H, V, layout=head_layout),
                  "model_norm": mk("model_norm", None, 1, H, 0.02, 1.0), "layers": []}
        mw = P.VortexModelWeight()
        mw.lm_head = _weight(self.t["lm_head"], H, V)
        mw.embedding = _weight(self.t["embedding"], V, H)
        mw.model_layernorm = _weight(self.t["model_norm"], H, 1)

        def gemm_weight(key, layer, rows, cols):
            """(tensor to keep alive, VortexWeight) of a [rows = K, cols = N] GEMM weight."""
            t = mk(key, layer, rows, cols, layout=layer_layout)
            if not e4m3:
                return t, _weight(t, cols, rows)
            blob = torch.empty((P.e4m3WeightBytes(cols, rows),), dtype=torch.uint8, device=self.dev)
            P.quantizeWeightE4M3(t.data_ptr(), blob.data_ptr(), cols, rows, torch.cuda.current_stream().cuda_stream)
            torch.cuda.synchronize()              # t is dropped on return
            w = P.VortexWeight()
            w.setPtr(blob.data_ptr())
            w.N, w.K = cols, rows
            return blob, w

        for l in range(self.layers):
            lt, lw = {}, P.VortexLayerWeight()
            lt["w_kqv"], lw.W_KQV = gemm_weight("w_kqv", l, H, kqv_n)
            lt["w_o"], lw.W_O1 = gemm_weight("w_o", l, shape.Hq * d, H)
            lw.W_O2 = lw.W_O1
            lt["w_gate"], lw.W_G = gemm_weight("w_gate", l, H, F)
            lt["w_up"], lw.W_U = gemm_weight("w_up", l, H, F)
            lt["w_down"], lw.W_D = gemm_weight("w_down", l, F, H)
            lt["ln_attn"] = mk("ln_attn", l, 1, H, 0.02, 1.0)
            lt["ln_ffn"] = mk("ln_ffn", l, 1, H, 0.02, 1.0)
            self.t["layers"].append(lt)
            if pipeline_type.has_kqv_bias:
                # biases of real checkpoints (Qwen2) reach tens in a few channels; N(0, 0.5) here
                lt["b_kqv"] = mk("b_kqv", l, 1, kqv_n, 0.5)
                lw.B_KQV = _weight(lt["b_kqv"], kqv_n, 1)
            lw.W_LN_Attention = _weight(lt["ln_attn"], H, 1)
            lw.W_LN_FFN = _weight(lt["ln_ffn"], H, 1)
            mw.layer_weight.append(lw)
        # KV pools [pages, 2, page, Hkv, d] per distinct layer
        self.kv = []
        for l in range(self.layers):
            if kv_pools is not None:
                pool = torch.zeros((self.max_pages, 2, shape.page_size, shape.Hkv, d),
                                   dtype=torch.float16, device=self.dev)
                src = torch.from_numpy(np.ascontiguousarray(kv_pools[l])).to(self.dev)
                pool[:src.shape[0]] = src
            else:
                pool = torch.empty((self.max_pages, 2, shape.page_size, shape.Hkv, d),
                                   dtype=torch.float16, device=self.dev)
                if kv_fill == "randn":
                    pool.normal_(0.0, 1.0, generator=gen)
                else:
                    pool.zero_()
            self.kv.append(pool)
        self.tmp = torch.empty((P.tmpBufferHalves(),), dtype=torch.float16, device=self.dev)
        init = P.VortexInitData()
        init.setKVdata([p.data_ptr() for p in self.kv])
        init.setWeight(mw, H * H * 3)
        init.setTmpBuffer(self.tmp.data_ptr(), self.tmp.numel())
        torch.cuda.synchronize()
        P.setProfiling(int(profiling))
        self._open = False
        self._hold = None
        P.init([init], pipeline_type)
        self._open = True
        try:
            cfg = P.VortexConfigData()
            cfg.setGemmOpTag(self.tags)
            cfg.globalBatchSize, cfg.nanobatch1Size = global_batch, nano1
            cfg.kqv1Size, cfg.kqv3Size = self.kqv1, self.kqv3
            P.config([cfg])
        except Exception:
            self.close()        # never leave the worker thread waiting behind a failed set-up
            raise

    # ------------------------------------------------------------------ per iteration
    def update(self, b: synth.Batch, keep_token_list=None, num_blocks=(0, 0, 0, 0)):
        """Stages one iteration.  keep_token_list marks, per slot of the PREVIOUS iteration's
        output, the requests that decode again (default: all of them, first iteration: the
        decode rows are fed token id 1 by the control plane)."""
        nd = b.decodePrefillBorder
        keep = np.ones(nd, np.int32) if keep_token_list is None else \
            np.ascontiguousarray(keep_token_list, dtype=np.int32)
        arrs = {
            "prefill_tokens": np.ascontiguousarray(b.input_tokens[nd:], dtype=np.int32),
            "input_indptr": b.input_indptr, "rev": b.rev_input_indptr, "off": b.per_token_offset,
            "kv_indptr": b.kv_indptr, "kv_indices": b.kv_indices, "kv_last": b.kv_last_page_len,
            "keep": keep,
        }
        arrs = {k: np.ascontiguousarray(v, dtype=np.int32) for k, v in arrs.items()}
        u = P.VortexUpdateData()
        u.decodePrefillBorder, u.prefillNum = nd, b.prefillNum
        u.prefillTokensNum, u.keepTokenListLength = b.prefillTokensNum, len(keep)
        u.setInputEmbedding(arrs["prefill_tokens"].ctypes.data)
        u.setInputIndptr(arrs["input_indptr"].ctypes.data)
        u.setRevInputIndptr(arrs["rev"].ctypes.data)
        u.setPerTokenOffset(arrs["off"].ctypes.data)
        u.setKVIndptr(arrs["kv_indptr"].ctypes.data)
        u.setKVIndices(arrs["kv_indices"].ctypes.data)
        u.setKVLastPageLen(arrs["kv_last"].ctypes.data)
        u.setKeepTokenList(arrs["keep"].ctypes.data)
        u.setGemvBatchSize(synth.gemv_batch_split(nd, self.kqv1, self.nano1, self.kqv3)
                           if not self.pipeline_type.is_sequential else [nd, 0, 0, 0])
        u.setGemvNumBlocks(list(num_blocks))
        self._hold = (arrs, u)
        P.update([u])

    def run(self) -> np.ndarray:
        P.run()
        return P.getPipelineOutput()

    def buffer(self, name: str) -> torch.Tensor:
        """Copy of an intermediate ("hidden" or "logits") as a torch tensor."""
        ptr, rows, cols = P.debugBuffer(name)
        out = torch.empty((rows, cols), dtype=torch.float16, device=self.dev)
        torch.cuda.synchronize()
        import ctypes as C
        hip = C.CDLL("libamdhip64.so")
        rc = hip.hipMemcpy(C.c_void_p(out.data_ptr()), C.c_void_p(ptr), C.c_size_t(rows * cols * 2),
                           C.c_int(4))  # hipMemcpyDefault: the source may be device or pinned host memory
        if rc != 0:
            raise RuntimeError(f"hipMemcpy failed: {rc}")
        return out

    def close(self):
        if self._open:
            P.finalize()
            self._open = False
            try:
                os.unlink(self.cfg_path)
            except OSError:
                pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
