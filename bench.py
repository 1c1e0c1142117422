#!/usr/bin/env python3
"""Benchmark of the single-GPU nano-batch pipeline on one MI355X.

A step is ONE dense iteration of the Llama-3-8B-shaped model (32 layers executed, vocab
128256, fp16 random-init weights): 2048 tokens = 1792 decode tokens (KV length uniform in
[1024, 1536], paged KV, page 16, permuted page table) + one 256-token prefill chunk, run by
the overlapped LocalPipeline through the control-plane C ABI.  The iteration's update data is
staged once before the timed region (inputs resident in HBM); each timed step is one
``run()`` = embedding ... sampler, ending with the sampled ids on the host.

Prints one JSON line: tokens/s (2048 tokens / step time), the roofline record of the
dominant kernel (paged decode attention, HBM-bound; durations from HIP events recorded on the
attention stream inside the timed region) and a CPU baseline (the oracle, a port of the
reference math, timed on the host cores on a bounded sample of the same workload).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = 2500.0       # dense fp16
# HBM bytes per decode-attention launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE,
# as a ratio to the algorithmic bytes of the same launch; None until measured
# (see profiles/decode_attention_config2_pmc.txt when present).
DECODE_ATTN_TRAFFIC_RATIO = None


def decode_attention_bytes(kv_len: np.ndarray, Hq=32, Hkv=8, d=128, page=16) -> int:
    """Algorithmic bytes of one decode-attention launch over requests with these KV lengths:
    K and V once (2*L*Hkv*d*2 B) + q and o (2*Hq*d*2 B) + page indices / indptr / last-page
    length (4*(ceil(L/page)+2) B) per request (accounting of the reference's
    gemv/src/bench_batch_decode.cu:77-81)."""
    L = kv_len.astype(np.int64)
    return int((2 * L * Hkv * d * 2 + 2 * Hq * d * 2 + 4 * ((L + page - 1) // page + 2)).sum())


def gemm_flops_per_iteration(shape, T, logits_rows, layers) -> float:
    per_tok = 2.0 * shape.hidden * (shape.kqv_n + shape.Hq * shape.d + 2 * shape.ffn) \
        + 2.0 * shape.ffn * shape.hidden
    return per_tok * T * layers + 2.0 * logits_rows * shape.hidden * shape.vocab


def cpu_baseline(shape, batch, n_sample: int, seed: int):
    """Times the oracle on a bounded sample of the same iteration: ONE decoder layer plus the
    LM head over the first n_sample decode requests of the batch (their real KV lengths),
    and scales to the 32-layer model: tokens/s = n / (layers * t_layer + t_head)."""
    from nanoflow_amd import synth
    from oracle import nf_oracle as O
    nd = n_sample
    lens_after = batch.kv_len[:nd]
    b = synth.make_batch(lens_after - 1, [], vocab=shape.vocab, seed=seed)
    rng = np.random.default_rng(seed + 1)
    one = synth.ModelShape(**{**shape.as_dict(), "layers": 1})
    w = synth.make_weights(one, seed=seed)
    pool = [synth.make_kv_pool(b.num_pages, one, rng)]
    x = synth.normal_f16(rng, (nd, shape.hidden))
    O.lib()
    t0 = time.perf_counter()
    hid, _, _ = O.decoder_forward(one.as_dict(), w, pool, b.as_dict(), hidden_in=x,
                                  want_sampled=False)
    t_layer = time.perf_counter() - t0
    t0 = time.perf_counter()
    kept = O.keep_token(hid, b.input_indptr, nd)
    logits = O.gemm(O.rmsnorm(kept, w["model_norm"]), w["lm_head"])
    O.argmax(logits)
    t_head = time.perf_counter() - t0
    total = shape.layers * t_layer + t_head
    return {
        "value": nd / total, "unit": "tokens/s", "cores": O.num_threads(), "kind": "port",
        "sample": (f"oracle (C + OpenMP restatement of the reference math): 1 of {shape.layers} layers "
                   f"+ LM head + sampler on {nd} of the {batch.decodePrefillBorder} decode requests "
                   f"(KV {int(lens_after.min())}-{int(lens_after.max())}); layer {t_layer:.2f} s, head "
                   f"{t_head:.2f} s, scaled to {shape.layers} layers"),
    }


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--pipeline", default="LOCAL", choices=["LOCAL", "NON_OVERLAP_LOCAL", "NANOBATCH_LOCAL"])
    ap.add_argument("--nano1", type=int, default=640, help="rows of nano-batch 1")
    ap.add_argument("--kqv1", type=int, default=256)
    ap.add_argument("--kqv3", type=int, default=768)
    ap.add_argument("--distinct-layers", type=int, default=0,
                    help="distinct weight/KV layers held in HBM (0 = as many of the 32 as fit)")
    ap.add_argument("--cpu-sample", type=int, default=128, help="decode requests in the CPU baseline (0 = skip)")
    ap.add_argument("--seed", type=int, default=0)
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the single-device pipeline on ONE GPU; --gpus N>1 is not "
              "supported (no collectives are part of this path).", file=sys.stderr)
        sys.exit(2)

    import torch
    from nanoflow_amd import engine, synth, pllm_python as P
    assert torch.cuda.is_available(), "bench.py needs the MI355X (no CPU path)"
    shape = synth.LLAMA3_8B
    T = 2048
    batch = synth.config2_batch(seed=args.seed)
    assert batch.tokens == T
    pages = batch.num_pages

    # Distinct layers held: 32 layers of this KV (9.5 GB each) exceed 288 GB, so layers alias
    # modulo `distinct` (the reference's own run_layer > model_layer device).
    free_b, total_b = torch.cuda.mem_get_info()
    per_layer = pages * 2 * 16 * shape.Hkv * shape.d * 2 + \
        2 * (shape.hidden * (shape.kqv_n + shape.Hq * shape.d + 2 * shape.ffn) + shape.ffn * shape.hidden)
    fixed = 2 * (2 * shape.vocab * shape.hidden) + 2 * (T * shape.hidden * 16 + T * shape.vocab * 2) + (4 << 30)
    distinct = args.distinct_layers or int(max(1, min(shape.layers, (free_b * 0.92 - fixed) // per_layer)))

    t_setup = time.perf_counter()
    eng = engine.Engine(shape, P.PipelineType[args.pipeline], global_batch=T, nano1=args.nano1,
                        kqv1=args.kqv1, kqv3=args.kqv3, kv_pages=pages, run_layer=shape.layers,
                        distinct_layers=distinct, seed=args.seed, profiling=True)
    eng.update(batch)
    torch.cuda.synchronize()
    t_setup = time.perf_counter() - t_setup

    for _ in range(args.warmup):
        eng.run()
    P.resetTimings()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = eng.run()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    tm = P.getTimings()
    ms_per_step = dt * 1e3 / args.steps

    # per-iteration PCIe-inclusive variant: stage the update data every step
    t0 = time.perf_counter()
    for _ in range(max(1, args.steps // 2)):
        eng.update(batch)
        eng.run()
    torch.cuda.synchronize()
    ms_with_update = (time.perf_counter() - t0) * 1e3 / max(1, args.steps // 2)

    nd = batch.decodePrefillBorder
    groups = synth.gemv_batch_split(nd, args.kqv1, args.nano1, args.kqv3) if args.pipeline != "NON_OVERLAP_LOCAL" else [nd]
    launches_per_layer = sum(1 for g in groups if g > 0)
    bytes_per_layer = decode_attention_bytes(batch.kv_len[:nd])
    n_launch = max(tm.decode_attn_launches, 1)
    avg_launch_ms = tm.decode_attn_ms / n_launch
    bytes_per_launch = bytes_per_layer / launches_per_layer
    achieved = bytes_per_launch / (avg_launch_ms * 1e-3) / 1e9 if avg_launch_ms > 0 else 0.0
    flops = gemm_flops_per_iteration(shape, T, min((batch.req_num + 127) // 128 * 128, T), shape.layers)

    rec = {
        "metric": "tokens/s/GPU", "value": T / (ms_per_step * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": ("Llama-3-8B shape, one dense 2048-token iteration: 1792 decode tokens "
                         "(KV U[1024,1536], page 16, permuted page table) + one 256-token prefill chunk"),
            "pipeline": args.pipeline, "global_batch": T, "nanobatch_1_size": args.nano1,
            "kqv1_size": args.kqv1, "kqv3_size": args.kqv3, "layers_executed": shape.layers,
            "distinct_layers_in_hbm": distinct, "kv_pages_per_layer": int(pages),
            "decode_attention_launches_per_layer": launches_per_layer,
        },
        "roofline": {
            "kernel": "attn_paged_kernel (paged decode attention)", "bound": "hbm",
            "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
            "traffic": (None if DECODE_ATTN_TRAFFIC_RATIO is None
                        else bytes_per_launch * DECODE_ATTN_TRAFFIC_RATIO),
            "algorithmic_bytes_per_launch": bytes_per_launch, "avg_launch_ms": avg_launch_ms,
            "launches_timed": int(tm.decode_attn_launches),
        },
        "iteration": {
            "device_ms_last": tm.iter_ms, "ms_per_step_with_update": ms_with_update,
            "decode_attention_ms_per_step": tm.decode_attn_ms / args.steps,
            "prefill_attention_ms_per_step": tm.prefill_attn_ms / args.steps,
            "gemm_tflop_per_step": flops / 1e12,
            "gemm_mfma_frac_if_serial": (flops / 1e12) / (max(ms_per_step - 0.0, 1e-9) * 1e-3) / MFMA_PEAK_TFLOPS,
            "setup_s": t_setup, "sampled_tokens": int(out.shape[0]),
        },
    }
    eng.close()
    if args.cpu_sample > 0:
        rec["cpu_baseline"] = cpu_baseline(shape, batch, args.cpu_sample, args.seed)
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
