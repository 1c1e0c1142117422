#!/usr/bin/env python3
"""Search over the schedule and the nano-batch split for one model shape and batch mix on this GPU.

The reference ships only the RESULT of its parameter search, as the ``pipeline_configs`` block of
each pipeline JSON (pipeline/config_all/llama3-8B/1024.json:41-55: global_batch_size,
nanobatch_1_size, kqv1_size, kqv3_size) plus ``serve_configs.pipeline_type``.  This tool measures
the candidates on the device and writes that block:

    python -m nanoflow_amd.autosearch -c config_all/llama3-8B/1024.json -o tuned.json \\
           [--decode 681 --kv-lo 1024 --kv-hi 1536 --prefill 755:269,0:1024,0:74] [--layers 8]

Candidates: NON_OVERLAP_LOCAL (one stream, no split), NANOBATCH_LOCAL / LOCAL (two nano-batches,
LOCAL on two streams) and PLLM (four QKV / attention nano-batches, two streams) over a grid of
nano-batch-1 sizes and QKV sub-splits, all multiples of ``--step`` rows.  Optional ``--cu-masks`` adds, for LOCAL, static compute-unit splits
between the GEMM and the attention stream (NANOFLOW_GEMM_CUS / NANOFLOW_GEMV_CUS: CU counts, given
here in eighths of the chip: 32 CUs, which a CU mask spreads as 4 CUs over each of the 8 XCDs).
Each candidate runs the same iteration (the decode requests and prefill chunks given, on
``--layers`` layers of random-init weights: the per-layer schedule is what is being compared) and is
timed over ``--iters`` runs after ``--warm``; one further run with HIP events around every attention and dense
GEMM launch records what justifies the choice: the TFLOP/s of the GEMM launches and the GB/s of decode attention
while they ran, and the share of the iteration each kind was running (shares that add up to more than 1 overlap).
The output JSON is the input config with the winning
``pipeline_configs`` / ``pipeline_type`` and a ``search`` block holding every measurement.
"""
from __future__ import annotations

import argparse
import copy
import json
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def candidates(T: int, step: int, types, fine: bool):
    """(pipeline type name, nano1, kqv1, kqv3) tuples; sizes are multiples of step with
    0 < kqv1 <= nano1 < T and 0 < kqv3 <= T - nano1 (pipeline_local.cu:198-217 splits the QKV
    GEMM of nano-batch 1 into kqv1 + rest and that of nano-batch 2 into kqv3 + rest)."""
    out = []
    if "NON_OVERLAP_LOCAL" in types:
        out.append(("NON_OVERLAP_LOCAL", T // 2, T // 4, T // 4))
    split_types = [t for t in types if t != "NON_OVERLAP_LOCAL"]
    if not split_types:
        return out
    n1s = [n for n in range(step, T, step) if T // 4 <= n <= 3 * T // 4]
    for t in split_types:
        for n1 in n1s:
            halves = {(max(step, n1 // 2 // step * step), max(step, (T - n1) // 2 // step * step))}
            if fine:
                halves |= {(max(step, n1 // 4 // step * step), max(step, (T - n1) // 4 // step * step)),
                           (max(step, 3 * n1 // 4 // step * step), max(step, 3 * (T - n1) // 4 // step * step))}
            for k1, k3 in sorted(halves):
                if 0 < k1 <= n1 and 0 < k3 <= T - n1:
                    out.append((t, n1, k1, k3))
    return out


ROLE_TAGS = {   # tag positions of the GEMM roles in gemm_op_tag, per schedule (the LM head's tag is the last one)
    4: {"O": [0], "D": [1], "KQV": [2], "LOGITS": [3]},
    7: {"O": [0, 1], "D": [2, 3], "KQV": [4, 5], "LOGITS": [6]},
    9: {"O": [0, 1], "D": [2, 3], "KQV": [4, 5, 6, 7], "LOGITS": [8]},
}


def measure(shape, batch, T, cand, layers, iters, warm, env=None, tags=None, layout="row"):
    """(milliseconds per iteration of one candidate: median of iters runs; utilisation record of one
    further run with HIP events around every attention and dense GEMM launch: the rate each kind of
    launch reached while it ran, and the share of the iteration each kind was running)."""
    import torch
    from nanoflow_amd import engine, pllm_python as P
    name, n1, k1, k3 = cand
    saved = {k: os.environ.get(k) for k in (env or {})}
    os.environ.update(env or {})
    try:
        eng = engine.Engine(shape, P.PipelineType[name], global_batch=T, nano1=n1, kqv1=k1, kqv3=k3,
                            kv_pages=batch.num_pages, run_layer=layers, distinct_layers=layers, gemm_tags=tags,
                            weight_layout=layout)
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    try:
        eng.update(batch)
        for _ in range(warm):
            eng.run()
        ts = []
        for _ in range(iters):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            eng.run()
            ts.append((time.perf_counter() - t0) * 1e3)
        util = {}
        try:
            P.setProfilingStride(1)
            P.setProfiling(2)
            eng.run()
            P.resetTimings()
            eng.run()
            torch.cuda.synchronize()
            tm = P.getTimings()
            nd = batch.decodePrefillBorder
            kv = batch.kv_len[:nd].astype(np.int64)
            attn_bytes = float((2 * kv * shape.Hkv * shape.d * 2 + 2 * shape.Hq * shape.d * 2
                                + 4 * ((kv + shape.page_size - 1) // shape.page_size + 2)).sum()) * layers
            if tm.gemm_ms > 0:
                util["gemm_tflops_while_running"] = tm.gemm_flop / (tm.gemm_ms * 1e-3) / 1e12
                util["gemm_share_of_iteration"] = tm.gemm_ms / tm.iter_ms
            if tm.decode_attn_ms > 0:
                util["decode_attention_gbps_while_running"] = attn_bytes / (tm.decode_attn_ms * 1e-3) / 1e9
                util["attention_share_of_iteration"] = (tm.decode_attn_ms + tm.prefill_attn_ms) / tm.iter_ms
        finally:
            P.setProfiling(0)
            P.setProfilingStride(0)
        return float(np.median(ts)), util
    finally:
        eng.close()


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("-c", "--config_path", required=True, help="pipeline JSON in the reference's schema")
    ap.add_argument("-o", "--output", required=True, help="tuned pipeline JSON to write")
    ap.add_argument("--decode", type=int, default=681, help="decode requests in the iteration")
    ap.add_argument("--kv-lo", type=int, default=1024)
    ap.add_argument("--kv-hi", type=int, default=1536)
    ap.add_argument("--prefill", default="755:269,0:1024,0:74", help="prefill chunks prev_len:chunk_len,...")
    ap.add_argument("--layers", type=int, default=8, help="layers executed per measurement")
    ap.add_argument("--step", type=int, default=128, help="granularity of the nano-batch sizes")
    ap.add_argument("--types", default="NON_OVERLAP_LOCAL,NANOBATCH_LOCAL,LOCAL,PLLM")
    ap.add_argument("--fine", action="store_true", help="also try 1/4 and 3/4 QKV sub-splits")
    ap.add_argument("--cu-masks", default="", help="LOCAL only: GEMM:attention shares of the CUs to try, in eighths (4 CUs of every XCD each), e.g. 6:2,5:3,4:4")
    ap.add_argument("--gemm-tiles", action="store_true",
                    help="then search, for the winning schedule, the tile and the split over K of each GEMM role (the\n"
                         "cta_m x cta_n and split_k fields of its tags) over the kernel library's tile menu, one role\n"
                         "at a time, and write the winning tags into pipeline_configs.gemm_op_tag")
    ap.add_argument("--weight-layout", default="", choices=["", "row", "col"],
                    help="orientation the weights are handed over in (default: what the input file's tags say, else col)")
    ap.add_argument("--iters", type=int, default=5)
    ap.add_argument("--warm", type=int, default=2)
    ap.add_argument("--seed", type=int, default=0)
    a = ap.parse_args()

    import torch
    from nanoflow_amd import engine, kernels, synth, weights as W
    assert torch.cuda.is_available(), "needs the MI355X"
    cfg = json.load(open(a.config_path))
    in_tags = cfg.get("pipeline_configs", {}).get("gemm_op_tag") or []
    layout = a.weight_layout
    if not layout:
        try:
            layout = engine.layouts_of_tags(in_tags)[0] if len(in_tags) > 1 else "col"
        except ValueError:
            layout = "col"
    shape = W.shape_from_hf_config(cfg["model"], cfg.get("model_configs", {}).get("frame_page_size", 16))
    chunks = [tuple(int(x) for x in c.split(":")) for c in a.prefill.split(",") if c]
    rng = np.random.default_rng(a.seed + 2)
    dlens = rng.integers(a.kv_lo, a.kv_hi + 1, size=a.decode).tolist() if a.decode else []
    batch = synth.make_batch(dlens, chunks, vocab=shape.vocab, seed=a.seed)
    T = cfg.get("pipeline_configs", {}).get("global_batch_size") or batch.tokens
    if batch.tokens > T:
        raise SystemExit(f"the iteration has {batch.tokens} tokens, global_batch_size is {T}")
    layers = min(a.layers, shape.layers)
    types = [t for t in a.types.split(",") if t]
    cands = candidates(T, a.step, types, a.fine)
    rows = []
    print(f"{len(cands)} candidates, {batch.tokens} tokens ({batch.decodePrefillBorder} decode), {layers} layers each", flush=True)
    for cand in cands:
        ms, util = measure(shape, batch, T, cand, layers, a.iters, a.warm, layout=layout)
        rows.append({"pipeline_type": cand[0], "nanobatch_1_size": cand[1], "kqv1_size": cand[2],
                     "kqv3_size": cand[3], "ms": ms, **util})
        print(f"  {cand[0]:18s} nano1 {cand[1]:5d} kqv1 {cand[2]:5d} kqv3 {cand[3]:5d}: {ms:8.3f} ms   "
              f"GEMM {util.get('gemm_tflops_while_running', 0):6.0f} TFLOP/s over {util.get('gemm_share_of_iteration', 0):4.2f} of the iteration, "
              f"decode attention {util.get('decode_attention_gbps_while_running', 0):6.0f} GB/s, attention over "
              f"{util.get('attention_share_of_iteration', 0):4.2f}", flush=True)
    masks = [tuple(int(x) for x in m.split(":")) for m in a.cu_masks.split(",") if m]
    local = [r for r in rows if r["pipeline_type"] == "LOCAL"]
    if masks and local:
        best_local = min(local, key=lambda r: r["ms"])
        cand = ("LOCAL", best_local["nanobatch_1_size"], best_local["kqv1_size"], best_local["kqv3_size"])
        for g, v in masks:
            if g <= 0 or v <= 0 or g + v > 8:
                raise SystemExit(f"--cu-masks {g}:{v}: the shares (eighths of the CUs) must be positive and sum to at most 8")
            env = {"NANOFLOW_GEMM_CUS": str(32 * g), "NANOFLOW_GEMV_CUS": str(32 * v)}   # 32 CUs per eighth
            ms, util = measure(shape, batch, T, cand, layers, a.iters, a.warm, env, layout=layout)
            rows.append({"pipeline_type": "LOCAL", "nanobatch_1_size": cand[1], "kqv1_size": cand[2],
                         "kqv3_size": cand[3], "gemm_cu_eighths": g, "attention_cu_eighths": v, "ms": ms, **util, **env})
            print(f"  LOCAL with {4 * g} CUs of every XCD for GEMM, {4 * v} for attention: {ms:8.3f} ms", flush=True)
    best = min(rows, key=lambda r: r["ms"])
    out = copy.deepcopy(cfg)
    pc = out.setdefault("pipeline_configs", {})
    pc.update({"global_batch_size": T, "nanobatch_1_size": best["nanobatch_1_size"],
               "kqv1_size": best["kqv1_size"], "kqv3_size": best["kqv3_size"]})
    from nanoflow_amd import pllm_python as P
    n_tags = P.PipelineType[best["pipeline_type"]].gemm_tags
    tags = [engine.make_tag(layout=layout)] * n_tags          # the library's own choice everywhere
    tile_rows = []
    if a.gemm_tiles:
        # one role at a time, the other roles at their best so far; a tag applies to launches of more
        # than 512 live rows, so roles whose pieces are shorter see no difference and keep the default
        cand = (best["pipeline_type"], best["nanobatch_1_size"], best["kqv1_size"], best["kqv3_size"])
        env = {k: best[k] for k in ("NANOFLOW_GEMM_CUS", "NANOFLOW_GEMV_CUS") if k in best}
        base_ms, _ = measure(shape, batch, T, cand, layers, a.iters, a.warm, env, tags=tags, layout=layout)
        print(f"tile search on {cand[0]}: library's choice {base_ms:.3f} ms", flush=True)
        menu = [(m, n) for m, n, col_only in kernels.gemm_tile_menu() if layout == "col" or not col_only]
        for role, pos in ROLE_TAGS[n_tags].items():
            if role == "LOGITS":
                continue                                       # one launch per iteration against 4 per layer
            best_role = (base_ms, tags[pos[0]])
            for (tm_, tn_) in menu:
                for split in (1, 2):
                    trial = list(tags)
                    tag = engine.make_tag(tm_, tn_, split, layout)
                    for i in pos:
                        trial[i] = tag
                    ms, _ = measure(shape, batch, T, cand, layers, a.iters, a.warm, env, tags=trial, layout=layout)
                    tile_rows.append({"role": role, "tile_m": tm_, "tile_n": tn_, "split_k": split, "ms": ms})
                    print(f"  {role:4s} tile {tm_:3d} x {tn_:3d} split {split}: {ms:8.3f} ms", flush=True)
                    if ms < best_role[0]:
                        best_role = (ms, tag)
            for i in pos:
                tags[i] = best_role[1]
            base_ms = best_role[0]
        print(f"tile search: {base_ms:.3f} ms with {tags}", flush=True)
    pc["gemm_op_tag"] = tags
    out.setdefault("serve_configs", {})["pipeline_type"] = best["pipeline_type"]
    out["search"] = {"iteration": {"decode_requests": a.decode, "kv_len": [a.kv_lo, a.kv_hi], "prefill_chunks": chunks,
                                   "tokens": batch.tokens}, "layers_per_measurement": layers,
                     "best": best, "measurements": rows, "weight_layout": layout, "gemm_tile_measurements": tile_rows}
    with open(a.output, "w") as f:
        json.dump(out, f, indent=1)
    print(f"best: {best['pipeline_type']} nano1 {best['nanobatch_1_size']} kqv1 {best['kqv1_size']} "
          f"kqv3 {best['kqv3_size']}: {best['ms']:.3f} ms -> {a.output}", flush=True)


if __name__ == "__main__":
    main()
