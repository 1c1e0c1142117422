#!/usr/bin/env python3
"""Benchmark of the single-GPU nano-batch pipeline on one MI355X (Llama-3-8B shape: 32
layers, vocab 128256, fp16 random-init weights, paged KV with page 16).

--workload offline (default): the offline-throughput job the headline metric is quoted on --
  4096 requests, constant 1024-token prompts (ids uniform over the vocab) and 512 output
  tokens, greedy, EOS ignored, served by the C++ batch former + asynchronous loop through the
  control-plane C ABI at <= 2048 tokens per iteration (steady state: ~682 decode rows + ~1366
  chunked-prefill rows).  As in the reference's own evaluation the scheduler is first advanced
  to steady state by simulated cycles (no GPU work), then W warm-up cycles run untimed and K
  cycles run timed; a step is one serving cycle (form batch i+1 on the CPU while the GPU runs
  batch i).  tokens/s = retired requests x 1536 / wall time (the reference's definition).
  --full-run times the whole job from the first request to the last instead.
--workload iteration: ONE dense 2048-token iteration = 1792 decode tokens (KV length uniform
  in [1024, 1536], permuted page table) + one 256-token prefill chunk, update data staged once
  before the timed region; a step is one ``run()`` = embedding ... sampler.
  --decode-requests / --prefill-chunk give other mixes, e.g. 64 and 0: the decode-only iteration
  of a lightly loaded server.

Prints one JSON line: tokens/s, the roofline record of the dominant kernel (offline: the dense
MFMA GEMMs; iteration: paged decode attention, HBM-bound -- durations from HIP events recorded
on the kernels' own streams inside the timed region), and a CPU baseline (the oracle, a port
of the reference math, timed on the host cores on a bounded sample of the same workload).
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
MFMA_FP8_PEAK_TFLOPS = 5000.0   # dense fp8
A100_PUBLISHED_TOKENS_PER_S = 12756.0   # reference, 1x A100 80GB, same offline workload
def _profile_figure(name: str, pattern: str):
    """A figure read from a committed rocprofv3 summary under profiles/ (None when the file or the
    line is missing): the traffic ratios below are measurements of the kernels, kept with the
    commands that made them, not constants of this file."""
    import re
    try:
        m = re.search(pattern, open(os.path.join(ROOT, "profiles", name)).read())
        return float(m.group(1)) if m else None
    except OSError:
        return None


def _overlap_note(workload: str = "offline") -> str:
    """What the overlapped nano-batch schedules cost against the single stream, as measured back to
    back on one box: profiles/schedules_offline_cycle.txt, profiles/schedules_dense_iteration.txt."""
    name = "schedules_offline_cycle.txt" if workload == "offline" else "schedules_dense_iteration.txt"
    local = _profile_figure(name, r"LOCAL - NON_OVERLAP_LOCAL\s*=\s*(-?[0-9.]+) ms")
    pllm = _profile_figure(name, r"PLLM - NON_OVERLAP_LOCAL\s*=\s*(-?[0-9.]+) ms")
    if local is None or pllm is None:
        return f"not measured (profiles/{name} is missing)"
    per = "cycle" if workload == "offline" else "iteration"
    return (f"measured, loses by {local:.1f} ms per {per} (LOCAL: two nano-batches on two streams) and by {pllm:.1f} ms "
            f"(PLLM: four QKV / attention nano-batches) against the single stream NON_OVERLAP_LOCAL, which only runs "
            f"chunked-prefill attention beside decode attention; profiles/{name}; --pipeline LOCAL | PLLM re-measure")


# HBM bytes per decode-attention launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (each scaled
# by what the same counter reads for a 1 GiB device copy), as a ratio to the algorithmic bytes of
# the same launch: profiles/decode_attention_config2_pmc.txt.
DECODE_ATTN_TRAFFIC_RATIO = _profile_figure("decode_attention_config2_pmc.txt", r"traffic / algorithmic\s*=\s*([0-9.]+)")


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


def cpu_baseline(shape, decode_lens_after, prefill_chunks, total_decode, seed: int):
    """Times the oracle on a bounded sample of the same iteration: ONE decoder layer plus the
    LM head over a sample of the batch's requests (decode requests with their real KV
    lengths, prefill chunks of the same proportion), and scales to the full depth:
    tokens/s = rows / (layers * t_layer + t_head)."""
    from nanoflow_amd import synth
    from oracle import nf_oracle as O
    decode_lens_after = np.asarray(decode_lens_after)
    b = synth.make_batch(decode_lens_after - 1, prefill_chunks, vocab=shape.vocab, seed=seed)
    rows = b.tokens
    rng = np.random.default_rng(seed + 1)
    one = synth.ModelShape(**{**shape.as_dict(), "layers": 1})
    w = synth.make_weights(one, seed=seed)
    pool = [synth.make_kv_pool(b.num_pages, one, rng)]
    x = synth.normal_f16(rng, (rows, shape.hidden))
    O.lib()
    t0 = time.perf_counter()
    hid, _, _ = O.decoder_forward(one.as_dict(), w, pool, b.as_dict(), hidden_in=x,
                                  want_sampled=False)
    t_layer = time.perf_counter() - t0
    t0 = time.perf_counter()
    kept = O.keep_token(hid, b.input_indptr, b.req_num)
    logits = O.gemm(O.rmsnorm(kept, w["model_norm"]), w["lm_head"])
    O.argmax(logits)
    t_head = time.perf_counter() - t0
    total = shape.layers * t_layer + t_head
    nd = len(decode_lens_after)
    return {
        "value": rows / total, "unit": "tokens/s", "cores": O.num_threads(), "kind": "port",
        "sample": (f"oracle (C + OpenMP restatement of the reference math): 1 of {shape.layers} layers "
                   f"+ LM head + sampler on {nd} of the {total_decode} decode requests "
                   f"(KV {int(decode_lens_after.min())}-{int(decode_lens_after.max())})"
                   + (f" and prefill chunks (prev, len) {list(prefill_chunks)}" if prefill_chunks else "")
                   + f"; layer {t_layer:.2f} s, head {t_head:.2f} s, scaled to {shape.layers} layers"),
    }


def calibrate(fp8: bool):
    """Ceilings measured on this device in this run, before the model is resident: a register-only
    MFMA loop (zero operands: the highest clock the part holds; pseudo-random operands: the
    switching activity a GEMM on N(0,1) data feeds the matrix pipe) and an 8 GiB read stream."""
    from nanoflow_amd import kernels as K
    K.lib()
    K.calibrate_mfma(fp8, True, 4000)                      # power state settles
    tf_rand, mhz_rand = K.calibrate_mfma(fp8, True, 40000)
    tf_zero, mhz_zero = K.calibrate_mfma(fp8, False, 40000)
    tf_lds, mhz_lds = (None, None) if fp8 else K.calibrate_mfma(False, 2, 40000)
    tf_ld, mhz_ld = (None, None) if fp8 else K.calibrate_mfma(False, 3, 40000)
    tf_16, mhz_16 = K.calibrate_mfma(fp8, 4, 40000)        # the 16x16 instruction of the type, same register tile
    hbm = K.calibrate_hbm_read(8.0, 4)
    return {"mfma_tflops_random_operands": tf_rand, "mfma_clock_mhz_random_operands": mhz_rand,
            "mfma_tflops_zero_operands": tf_zero, "mfma_clock_mhz_zero_operands": mhz_zero,
            # the register-only loop on v_mfma_f32_16x16x32_f16 (fp8: 16x16x128), which the four-wavefront
            # fp16 GEMM tiles are computed with: the higher of the two is the measured MFMA-only ceiling
            "mfma_tflops_random_operands_16x16": tf_16, "mfma_clock_mhz_random_operands_16x16": mhz_16,
            # the same loop with its operand fragments re-read from LDS at the GEMM main loop's rate
            "mfma_tflops_random_operands_from_lds": tf_lds, "mfma_clock_mhz_random_operands_from_lds": mhz_lds,
            # ... and with a 256x256 tile's operand loads (L2 -> LDS) beside them: a main loop without barriers
            "mfma_tflops_with_operand_loads": tf_ld, "mfma_clock_mhz_with_operand_loads": mhz_ld,
            "mfma_dtype": "f8e4m3" if fp8 else "f16", "hbm_read_stream_gbps": hbm,
            "how": "nf_calibrate_mfma: 1024 workgroups x 4 wavefronts x 40000 x 16 independent 32x32 MFMAs "
                   "(or 20000 x 64 independent 16x16 ones), registers only; nf_calibrate_hbm_read: 2048 workgroups stream 8 GiB 4 times"}


def _check_single_gpu(args):
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the single-device pipeline on ONE GPU; --gpus N>1 is not "
              "supported (no collectives are part of this path).", file=sys.stderr)
        sys.exit(2)


def _attention_roofline(tm, bytes_per_launch, name="roofline", calib=None):
    n_launch = max(tm.decode_attn_launches, 1)
    avg_launch_ms = tm.decode_attn_ms / n_launch
    achieved = bytes_per_launch / (avg_launch_ms * 1e-3) / 1e9 if avg_launch_ms > 0 else 0.0
    extra = {}
    if calib:
        extra = {"measured_peak": calib["hbm_read_stream_gbps"],
                 "frac_of_measured_peak": achieved / calib["hbm_read_stream_gbps"]}
        if "paged_read_no_arithmetic_gbps" in calib:
            extra["paged_read_no_arithmetic_gbps"] = calib["paged_read_no_arithmetic_gbps"]
    return {
        **extra,
        "kernel": "attn_decode_kernel (paged decode attention)", "bound": "hbm",
        "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
        "traffic": (None if DECODE_ATTN_TRAFFIC_RATIO is None
                    else bytes_per_launch * DECODE_ATTN_TRAFFIC_RATIO),
        "algorithmic_bytes_per_launch": bytes_per_launch, "avg_launch_ms": avg_launch_ms,
        "launches_timed": int(tm.decode_attn_launches),
    }


# Memory-side bytes per dense GEMM launch over algorithmic bytes (operands once + output), measured
# with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on the fp16 kernels as the offline workload launches
# them (Llama-3-8B shape, M = 2048, LM head on 684 rows, [N][K] weights) and scaled by the copy-kernel
# calibration: profiles/gemm_hbm_traffic_pmc.txt.  It holds for that shape, layout and weight type
# only; other runs report no traffic figure.
GEMM_TRAFFIC_PROFILE = "gemm_hbm_traffic_pmc.txt"
GEMM_TRAFFIC_RATIO = _profile_figure(GEMM_TRAFFIC_PROFILE, r"traffic_bytes_per_algorithmic_byte\s*=\s*([0-9.]+)")


def _gemm_algorithmic_bytes_per_launch(shape, rows, sampled_rows, weight_bytes=2):
    """Operands once plus outputs (and the residual operand of O and down) of one cycle's dense
    GEMMs, averaged over its launches (4 per layer + the LM head).  Activations are fp16; the
    per-layer weights take weight_bytes per element (1 for e4m3), the LM head 2."""
    H, F, V = shape.hidden, shape.ffn, shape.vocab
    hq = shape.Hq * shape.d
    act = (rows * H + rows * shape.kqv_n            # QKV
           + rows * hq + 2 * rows * H               # O (+ C)
           + rows * H + rows * F                    # gate/up
           + rows * F + 2 * rows * H)               # down (+ C)
    wts = H * shape.kqv_n + hq * H + 2 * H * F + F * H
    m_lm = (sampled_rows + 127) // 128 * 128
    total = shape.layers * (2 * act + weight_bytes * wts) + 2 * (m_lm * H + H * V + m_lm * V)
    return total / (4 * shape.layers + 1)


def _gemm_roofline(tm, alg_bytes_per_launch=None, fp8_share=0.0, calib=None, traffic_applies=False):
    """fp8_share: the fraction of the timed GEMM flops that runs on the fp8 matrix cores (the
    per-layer GEMMs with e4m3 weights; the LM head stays fp16).  The peak the launches are priced
    against is then the flop-weighted blend of the two published peaks."""
    n = max(tm.gemm_launches, 1)
    avg_ms = tm.gemm_ms / n
    flop_per_launch = tm.gemm_flop / n
    achieved = flop_per_launch / (avg_ms * 1e-3) / 1e12 if avg_ms > 0 else 0.0
    peak = 1.0 / (fp8_share / MFMA_FP8_PEAK_TFLOPS + (1.0 - fp8_share) / MFMA_PEAK_TFLOPS)
    extra = {}
    if calib and not fp8_share:
        # the register-only MFMA loop on pseudo-random operands: what the matrix pipe sustains on
        # this device at the clock it holds under that load
        best = max(calib["mfma_tflops_random_operands"], calib.get("mfma_tflops_random_operands_16x16") or 0.0)
        extra = {"measured_peak": best, "frac_of_measured_peak": achieved / best,
                 "measured_peak_32x32x16": calib["mfma_tflops_random_operands"],
                 "measured_peak_zero_operands": calib["mfma_tflops_zero_operands"]}
    return {
        **extra,
        "kernel": ("gemm_f16_kernel / dual_swiglu_f16_kernel (all dense GEMM launches of the iteration)" if not fp8_share
                   else "gemm_f8_kernel incl. the fused gate/up variant (e4m3 weights, activations quantised per "
                        "launch; the quantiser's time is not in these launches) + the fp16 LM head"),
        "bound": "mfma", "achieved": achieved, "peak": peak, "unit": "TFLOP/s",
        "frac": achieved / peak,
        # the measured ratio belongs to the fp16 kernels at the 8B shape on [N][K] weights (traffic_applies)
        "traffic": (alg_bytes_per_launch * GEMM_TRAFFIC_RATIO
                    if traffic_applies and alg_bytes_per_launch is not None and GEMM_TRAFFIC_RATIO and not fp8_share else None),
        "traffic_measured_by": (f"profiles/{GEMM_TRAFFIC_PROFILE}: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on these kernels, "
                                f"{GEMM_TRAFFIC_RATIO} bytes moved per algorithmic byte" if traffic_applies and GEMM_TRAFFIC_RATIO else None),
        "algorithmic_bytes_per_launch": alg_bytes_per_launch,
        "algorithmic_flop_per_launch": flop_per_launch, "avg_launch_ms": avg_ms,
        "launches_timed": int(tm.gemm_launches),
    }


def run_iteration(args):
    import torch
    from nanoflow_amd import engine, synth, pllm_python as P
    assert torch.cuda.is_available(), "bench.py needs the MI355X (no CPU path)"
    shape = synth.LLAMA3_70B if args.shape == "70b" else synth.LLAMA3_8B
    wb = 1 if args.weights == "e4m3" else 2                    # bytes per element of the per-layer GEMM weights
    shape_name = "Llama-3-70B" if args.shape == "70b" else "Llama-3-8B"
    T = 2048
    steps = args.steps or 5
    warmup = 2 if args.warmup is None else args.warmup
    # the default mix fills the iteration; --decode-requests / --prefill-chunk give others
    # (e.g. 64 and 0: the decode-only iteration of a lightly loaded server)
    n_dec, n_pre = args.decode_requests, args.prefill_chunk
    if n_dec < 1 or n_pre < 0 or n_dec + n_pre > T:
        raise SystemExit(f"--decode-requests must be at least 1 and, with --prefill-chunk, at most {T}")
    if n_pre > 0:
        batch = synth.config2_batch(seed=args.seed, n_decode=n_dec, prefill_chunk=n_pre, vocab=shape.vocab)
    else:
        lens = np.random.default_rng(args.seed + 2).integers(1024, 1537, size=n_dec)
        batch = synth.make_batch(lens, [], shape.vocab, seed=args.seed)
    assert batch.tokens == n_dec + n_pre
    pages = batch.num_pages

    # Distinct layers held: 32 layers of this KV (9.5 GB each) exceed 288 GB, so layers alias
    # modulo `distinct` (the reference's own run_layer > model_layer device).
    free_b, total_b = torch.cuda.mem_get_info()
    per_layer = pages * 2 * 16 * shape.Hkv * shape.d * 2 + \
        wb * (shape.hidden * (shape.kqv_n + shape.Hq * shape.d + 2 * shape.ffn) + shape.ffn * shape.hidden)
    fixed = 2 * (2 * shape.vocab * shape.hidden) + 2 * (T * shape.hidden * 16 + T * shape.vocab * 2) + (4 << 30)
    distinct = args.distinct_layers or int(max(1, min(shape.layers, (free_b * 0.92 - fixed) // per_layer)))

    calib = calibrate(wb == 1) if args.calibrate else None
    t_setup = time.perf_counter()
    eng = engine.Engine(shape, P.PipelineType[args.pipeline], global_batch=T, nano1=args.nano1,
                        kqv1=args.kqv1, kqv3=args.kqv3, kv_pages=pages, run_layer=shape.layers,
                        distinct_layers=distinct, seed=args.seed, profiling=0,
                        weight_format=args.weights, weight_layout=args.weight_layout)
    P.setGraphMode(args.graph)
    eng.update(batch)
    torch.cuda.synchronize()
    t_setup = time.perf_counter() - t_setup

    # pass 1, the one `value` comes from: no per-launch events
    for _ in range(warmup):
        eng.run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        out = eng.run()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt * 1e3 / steps
    # pass 2, the one the roofline records come from: the same iteration, eagerly, with HIP events
    # around every attention and dense GEMM launch of every 4th layer, on the kernels' own streams
    P.setGraphMode(False)
    P.setProfiling(args.profile_level)
    eng.run()
    P.resetTimings()
    for _ in range(steps):
        eng.run()
    torch.cuda.synchronize()
    tm = P.getTimings()
    P.setProfiling(0)
    P.setGraphMode(args.graph)

    # per-iteration PCIe-inclusive variant: stage the update data every step
    t0 = time.perf_counter()
    for _ in range(max(1, steps // 2)):
        eng.update(batch)
        eng.run()
    torch.cuda.synchronize()
    ms_with_update = (time.perf_counter() - t0) * 1e3 / max(1, steps // 2)

    nd = batch.decodePrefillBorder
    groups = synth.gemv_batch_split(nd, args.kqv1, args.nano1, args.kqv3) if args.pipeline != "NON_OVERLAP_LOCAL" else [nd]
    launches_per_layer = sum(1 for g in groups if g > 0)
    bytes_per_layer = decode_attention_bytes(batch.kv_len[:nd], shape.Hq, shape.Hkv, shape.d)
    lm_rows = min((batch.req_num + 127) // 128 * 128, T)
    flops = gemm_flops_per_iteration(shape, batch.tokens, lm_rows, shape.layers)
    fp8_share = 1.0 - 2.0 * lm_rows * shape.hidden * shape.vocab / flops if wb == 1 else 0.0

    rec = {
        "metric": "tokens/s/GPU", "value": batch.tokens / (ms_per_step * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16" if wb == 2 else "f8e4m3 weights and GEMM inputs, f16 activations and KV",
        "data": "synthetic",
        "config": {
            "workload": (f"{shape_name} shape, one " + ("dense 2048-token " if n_dec + n_pre == T else "")
                         + f"iteration: {n_dec} decode tokens (KV U[1024,1536], page 16, permuted page table)"
                         + (f" + one {n_pre}-token prefill chunk" if n_pre else "")),
            "weights": args.weights,
            "weight_layout": ("[N][K] (k contiguous; GEMM tags say ColumnMajor for B)" if eng.weight_layout == "col" else
                              "[K][N] (the reference's weight-file orientation; tags say RowMajor)") if wb == 2 else
                             "e4m3 [N][K] + per-output-channel scales; LM head fp16 " + ("[V][H]" if eng.lm_head_layout == "col" else "[H][V]"),
            "pipeline": args.pipeline,
            "overlap": (_overlap_note("iteration") if args.shape == "8b" and wb == 2 and n_dec == 1792 and n_pre == 256
                        else None),
            "global_batch": T, "nanobatch_1_size": args.nano1,
            "kqv1_size": args.kqv1, "kqv3_size": args.kqv3, "layers_executed": shape.layers,
            "distinct_layers_in_hbm": distinct, "kv_pages_per_layer": int(pages),
            "decode_attention_launches_per_layer": launches_per_layer,
        },
        "roofline": _attention_roofline(tm, bytes_per_layer / launches_per_layer, calib=calib),
        "iteration": {
            "device_ms_last": tm.iter_ms, "ms_per_step_with_update": ms_with_update,
            "decode_attention_ms_per_step": tm.decode_attn_ms * tm.layer_stride / steps,
            "prefill_attention_ms_per_step": tm.prefill_attn_ms * tm.layer_stride / steps,
            "gemm_tflop_per_step": flops / 1e12,
            "gemm_mfma_frac_if_serial": (flops / 1e12) / (max(ms_per_step, 1e-9) * 1e-3) /
            (MFMA_PEAK_TFLOPS if wb == 2 else 1.0 / (fp8_share / MFMA_FP8_PEAK_TFLOPS + (1 - fp8_share) / MFMA_PEAK_TFLOPS)),
            "setup_s": t_setup, "sampled_tokens": int(out.shape[0]),
        },
    }
    if tm.gemm_launches:
        rec["roofline_gemm"] = _gemm_roofline(tm, fp8_share=fp8_share, calib=calib)
        rec["iteration"]["gemm_ms_per_step"] = tm.gemm_ms * tm.layer_stride / steps
    if calib:
        from nanoflow_amd import kernels as K
        dv = lambda a_: torch.from_numpy(np.ascontiguousarray(a_, np.int32)).cuda()
        calib["paged_read_no_arithmetic_gbps"] = K.calibrate_paged_read(
            eng.kv[0], dv(batch.kv_indptr[:nd + 1]), dv(batch.kv_indices), dv(batch.kv_last_page_len[:nd]),
            nd, shape.Hkv, int(2 * batch.kv_len[:nd].astype(np.int64).sum() * shape.Hkv * shape.d * 2), 10)
        rec["roofline"]["paged_read_no_arithmetic_gbps"] = calib["paged_read_no_arithmetic_gbps"]
        rec["calibration"] = calib
    eng.close()
    if args.cpu_sample > 0:
        rec["cpu_baseline"] = cpu_baseline(shape, batch.kv_len[:args.cpu_sample], [], nd, args.seed)
    return rec


def _serve_whole_job(former, chunk=512):
    """The whole job, `chunk` timed cycles per call of the serving loop, with a progress line
    after each (a 70B job runs for minutes).  Each call starts and ends with the GPU idle: one
    cycle in `chunk` loses the overlap of batch formation with the device."""
    import types
    tot = types.SimpleNamespace(cycles=0, retired=0, wall_s=0.0, tokens_processed=0, cycle_ms=0.0, form_ms=0.0,
                                wait_ms=0.0, update_ms=0.0, gpu_iter_ms=0.0)
    while True:
        st = former.serve(0, chunk, warmup_cycles=0)
        for f in ("cycle_ms", "form_ms", "wait_ms", "update_ms", "gpu_iter_ms"):   # means over cycles
            setattr(tot, f, (getattr(tot, f) * tot.cycles + getattr(st, f) * st.cycles) / max(tot.cycles + st.cycles, 1))
        tot.cycles += st.cycles
        tot.retired += st.retired
        tot.wall_s += st.wall_s
        tot.tokens_processed += st.tokens_processed
        state = former.state()
        left = state["queued"] + state["decoding"] + state["prefilling"]
        print(f"[bench] {tot.cycles} cycles, {tot.retired} requests retired, {left} left, {tot.wall_s:.1f} s",
              file=sys.stderr, flush=True)
        if st.cycles < chunk or left == 0:
            return tot


def run_offline(args):
    import torch
    from nanoflow_amd import engine, synth, pllm_python as P
    assert torch.cuda.is_available(), "bench.py needs the MI355X (no CPU path)"
    shape = synth.LLAMA3_70B if args.shape == "70b" else synth.LLAMA3_8B
    wb = 1 if args.weights == "e4m3" else 2                    # bytes per element of the per-layer GEMM weights
    shape_name = "Llama-3-70B" if args.shape == "70b" else "Llama-3-8B"
    T, n_req, in_len, out_len = args.global_batch, args.requests, 1024, 512
    steps = args.steps or 256
    warmup = 8 if args.warmup is None else args.warmup

    # KV pool: every layer distinct; 2 MiB per page over the 32 layers.  The trace peaks near
    # 66k pages in flight; the pool is sized to HBM with headroom, capped at 128 Ki pages.
    free_b, _ = torch.cuda.mem_get_info()
    weight_b = wb * shape.layers * (shape.hidden * (shape.kqv_n + shape.Hq * shape.d + 2 * shape.ffn)
                                    + shape.ffn * shape.hidden) + 2 * 2 * shape.vocab * shape.hidden
    page_b = shape.layers * 2 * 16 * shape.Hkv * shape.d * 2
    pages = args.kv_pages or int(min(131072, (free_b * 0.90 - weight_b - (6 << 30)) // page_b))
    pages = pages // 64 * 64
    assert pages >= 4096, f"not enough free HBM for the KV pool ({free_b / 2**30:.0f} GiB free)"

    calib = calibrate(False) if args.calibrate else None

    t_setup = time.perf_counter()
    # Random KV contents (N(0,1), as the weights and activations are random): the pool the decode
    # rows read must not be a run of zeros.
    eng = engine.Engine(shape, P.PipelineType[args.pipeline], global_batch=T, nano1=args.nano1,
                        kqv1=args.kqv1, kqv3=args.kqv3, kv_pages=pages, seed=args.seed,
                        profiling=0, kv_fill=args.kv_fill, weight_format=args.weights,
                        weight_layout=args.weight_layout)
    former = P.BatchFormer(pages, shape.page_size, T, args.nano1, args.kqv1, args.kqv3, in_len, out_len)
    rng = np.random.default_rng(args.seed)
    for i in range(n_req):
        former.add_request(i, rng.integers(0, shape.vocab, size=in_len, dtype=np.int32), out_len)
    torch.cuda.synchronize()
    t_setup = time.perf_counter() - t_setup

    # ---- pass 1, the one `value` comes from: iterations replayed from captured hipGraphs, no
    # per-launch events.  Part of the set-up (like the simulated cycles): `prime` serving cycles in
    # which the steady state's launch signatures are seen and captured.
    graph = not args.no_graph and not args.full_run
    P.setGraphMode(graph)
    prime = 0
    if args.full_run:
        skip, warmup = 0, 0
    else:
        skip = args.skip_cycles
        prime = args.prime_cycles if graph else 0
        if prime:
            former.serve(skip, prime, warmup_cycles=0)
            skip = 0
    st = _serve_whole_job(former) if args.full_run else former.serve(skip, steps, warmup_cycles=warmup)
    counters = P.getGraphCounters()
    P.setGraphMode(False)

    # ---- pass 2, the one the roofline records come from: the next cycles of the same job run
    # eagerly with HIP events around every launch of every 16th layer (attention and dense GEMMs),
    # on the streams the kernels run on
    tm = P.getTimings()
    prof_cycles = 0
    if args.profile_level and not args.full_run:
        prof_cycles = min(st.cycles, args.profile_cycles)
        P.setProfilingStride(16 if prof_cycles >= 32 else 4)
        P.setProfiling(args.profile_level)
        st_prof = former.serve(0, prof_cycles, warmup_cycles=2)
        tm = P.getTimings()
        prof_cycles = st_prof.cycles
        P.setProfiling(0)
    state = former.state()
    steps = st.cycles
    n_prof = max(prof_cycles if prof_cycles else st.cycles, 1)   # cycles the per-launch timings cover
    rows_per_req = in_len + out_len - 1          # dense-batch rows a request occupies in its life
    by_retired = st.retired * (in_len + out_len) / st.wall_s
    by_rows = st.tokens_processed / rows_per_req * (in_len + out_len) / st.wall_s
    # the reference's definition counts whole retired requests; over a short window that is
    # quantised (about 1.33 requests retire per cycle), so below 200 retirements the same
    # quantity is taken from the rows processed instead
    use_retired = st.retired >= 200
    value = by_retired if use_retired else by_rows

    # steady-state decode set for the byte accounting: the requests now decoding
    former.schedule()
    nxt = former.form()
    nd = nxt["decodePrefillBorder"]
    kv_len = ((np.diff(nxt["kv_indptr"]) - 1) * shape.page_size + nxt["kv_last_page_len"])[:nd]
    groups = [g for g in nxt["gemv_batch_size"].tolist() if g > 0] if args.pipeline != "NON_OVERLAP_LOCAL" else [nd]
    launches_per_layer = max(len(groups), 1)
    bytes_per_layer = decode_attention_bytes(kv_len, shape.Hq, shape.Hkv, shape.d) if nd else 0
    rows_next, reqs_next = nd + int(nxt["prefillTokensNum"]), nd + int(nxt["prefillNum"])
    flops_next = gemm_flops_per_iteration(shape, rows_next, (reqs_next + 127) // 128 * 128, shape.layers)
    fp8_share = (1.0 - 2.0 * ((reqs_next + 127) // 128 * 128) * shape.hidden * shape.vocab / flops_next
                 if wb == 1 and flops_next else 0.0)
    prefill_chunks = [(int(nxt["per_token_offset"][nxt["input_indptr"][nd + j]]),
                       int(nxt["input_indptr"][nd + j + 1] - nxt["input_indptr"][nd + j]))
                      for j in range(nxt["prefillNum"])]

    rec = {
        "metric": "tokens/s/GPU", "value": value, "unit": "tokens/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": st.cycle_ms,
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": value / A100_PUBLISHED_TOKENS_PER_S if args.shape == "8b" and wb == 2 else None,
        "dtype": "f16" if wb == 2 else "f8e4m3 weights and GEMM inputs, f16 activations and KV", "data": "synthetic",
        "config": {
            "weights": args.weights,
            "weight_layout": ("[N][K] (k contiguous; GEMM tags say ColumnMajor for B)" if eng.weight_layout == "col" else
                              "[K][N] (the reference's weight-file orientation; tags say RowMajor)") if wb == 2 else
                             "e4m3 [N][K] + per-output-channel scales; LM head fp16 " + ("[V][H]" if eng.lm_head_layout == "col" else "[H][V]"),
            "workload": (f"{shape_name} shape, offline throughput: {n_req} requests, constant {in_len}-token "
                         f"prompts (ids uniform over the vocab) / {out_len} output tokens, greedy, EOS "
                         f"ignored, <= {T} tokens per iteration with chunked prefill; "
                         + ("whole job timed" if args.full_run else
                            f"{args.skip_cycles} simulated scheduler cycles to steady state, {prime} untimed cycles "
                            f"that capture the hipGraphs, then {warmup} warm-up and {steps} timed serving cycles "
                            f"replayed from hipGraphs; the roofline records come from the {prof_cycles} eager, "
                            f"per-launch-timed cycles that follow")),
            "kv_contents": args.kv_fill,
            "pipeline": args.pipeline, "overlap": _overlap_note() if args.shape == "8b" and wb == 2 else None,
            "global_batch": T, "nanobatch_1_size": args.nano1,
            "kqv1_size": args.kqv1, "kqv3_size": args.kqv3, "layers_executed": shape.layers,
            "distinct_layers_in_hbm": shape.layers, "kv_pages_per_layer": int(pages),
            "kv_pool_gib": pages * page_b / 2**30,
            "value_formula": ("retired_requests * 1536 / wall_s" if use_retired else
                              "dense_rows_processed / 1535 * 1536 / wall_s (fewer than 200 retirements in the window)"),
            "baseline": ("12756 tokens/s/GPU published by the reference for this workload on 1x A100 80GB"
                         if args.shape == "8b" and wb == 2 else
                         "none: the reference publishes no single-GPU figure for this shape / weight format"),
        },
        "roofline": _gemm_roofline(tm, _gemm_algorithmic_bytes_per_launch(shape, rows_next, reqs_next, wb), fp8_share, calib,
                                   traffic_applies=args.shape == "8b" and wb == 2 and eng.weight_layout == "col" and T == 2048
                                   ) if tm.gemm_launches else _attention_roofline(
            tm, bytes_per_layer / launches_per_layer, calib=calib),
        "serving": {
            "cycles": st.cycles, "retired_requests": st.retired, "wall_s": st.wall_s,
            "tokens_per_s_by_retired_requests": by_retired, "tokens_per_s_by_rows": by_rows,
            "dense_rows_processed": int(st.tokens_processed),
            "cycle_ms": st.cycle_ms, "gpu_iteration_ms": st.gpu_iter_ms,
            "cpu_form_ms": st.form_ms, "cpu_wait_for_gpu_ms": st.wait_ms, "cpu_update_ms": st.update_ms,
            # Cycle time not covered by the device's iteration: the update (staging + H2D copies,
            # which need the previous iteration's samples) and the hand-off (the caller's wake-up after the
            # worker's barrier, the worker's wake-up for the next run, the first launch).  Batch formation
            # is not in it: the loop forms batch c while the GPU runs batch c-1 and then WAITS for the GPU
            # (cpu_wait_for_gpu_ms), so as long as that wait is positive formation is wholly hidden.
            "cpu_exposed_ms_per_cycle": max(0.0, st.cycle_ms - st.gpu_iter_ms),
            "cpu_handoff_ms_per_cycle": max(0.0, st.cycle_ms - st.gpu_iter_ms - st.update_ms),
            "cpu_form_hidden_fraction": (None if st.form_ms <= 0 else 1.0 if st.wait_ms > 0.05 * st.gpu_iter_ms else
                                         max(0.0, 1.0 - max(0.0, st.cycle_ms - st.gpu_iter_ms - st.update_ms) / st.form_ms)),
            "steady_state_decode_rows": int(nd), "steady_state_prefill_rows": int(nxt["prefillTokensNum"]),
            "decode_attention_ms_per_cycle": tm.decode_attn_ms * tm.layer_stride / n_prof,
            "prefill_attention_ms_per_cycle": tm.prefill_attn_ms * tm.layer_stride / n_prof,
            "gemm_ms_per_cycle": tm.gemm_ms * tm.layer_stride / n_prof,   # LM head: timed 1 iteration in layer_stride
            "timed_layer_stride": tm.layer_stride, "per_launch_timed_cycles": prof_cycles,
            "per_launch_timed_cycle_ms": st_prof.cycle_ms if prof_cycles else None,
            # the same serving loop over the per-launch-timed cycles that follow the timed window
            # (eager launches with HIP events around every timed launch: a little slower per cycle)
            "profile_pass": ({"cycles": st_prof.cycles, "retired_requests": st_prof.retired, "wall_s": st_prof.wall_s,
                              "dense_rows_processed": int(st_prof.tokens_processed),
                              "tokens_per_s_by_rows": st_prof.tokens_processed / rows_per_req * (in_len + out_len) / st_prof.wall_s,
                              "cycle_ms": st_prof.cycle_ms} if prof_cycles and st_prof.wall_s > 0 else None),
            "graph_counters": counters,
            "requests_left": state["queued"] + state["decoding"] + state["prefilling"],
            "setup_s": t_setup,
        },
    }
    if calib and nd:
        # the decode rows' own page table through the load pattern of the attention kernel with the
        # arithmetic removed: the ceiling of that access pattern on this device
        dv = lambda a_: torch.from_numpy(np.ascontiguousarray(a_, np.int32)).cuda()
        from nanoflow_amd import kernels as K
        calib["paged_read_no_arithmetic_gbps"] = K.calibrate_paged_read(
            eng.kv[0], dv(nxt["kv_indptr"][:nd + 1]), dv(nxt["kv_indices"]), dv(nxt["kv_last_page_len"][:nd]),
            nd, shape.Hkv, int(2 * kv_len.astype(np.int64).sum() * shape.Hkv * shape.d * 2), 10)
        rec["calibration"] = calib
        if rec["roofline"]["bound"] == "hbm":
            rec["roofline"]["paged_read_no_arithmetic_gbps"] = calib["paged_read_no_arithmetic_gbps"]
    if tm.gemm_launches and tm.decode_attn_launches and nd:
        rec["roofline_decode_attention"] = _attention_roofline(tm, bytes_per_layer / launches_per_layer, calib=calib)
    eng.close()
    if args.cpu_sample > 0 and nd:
        n = min(args.cpu_sample, nd)
        sample_chunks = [(p, max(1, l * n // nd)) for p, l in prefill_chunks]
        rec["cpu_baseline"] = cpu_baseline(shape, kv_len[:n], sample_chunks, nd, args.seed)
    return rec


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default: offline 256, iteration 5)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps (default: offline 8, iteration 2)")
    ap.add_argument("--workload", default="offline", choices=["offline", "iteration"])
    ap.add_argument("--shape", default="8b", choices=["8b", "70b"],
                    help="8b: the Llama-3-8B shape the headline metric is quoted on; 70b: the Llama-3-70B shape\n"
                         "(80 layers, hidden 8192, 64 Q / 8 KV heads, FFN 28672) resident on the one GPU")
    ap.add_argument("--weights", default="f16", choices=["f16", "e4m3"],
                    help="e4m3: the five per-layer GEMM weights in fp8 with per-output-channel scales")
    ap.add_argument("--weight-layout", default="col", choices=["col", "row"],
                    help="col: fp16 weights handed over [N][K], k contiguous (every GEMM tag says ColumnMajor for B; a\n"
                         "Hugging Face checkpoint's own orientation); row: [K][N] as the reference's weight files hold them")
    ap.add_argument("--pipeline", default="auto", choices=["auto", "LOCAL", "NON_OVERLAP_LOCAL", "NANOBATCH_LOCAL", "PLLM", "NANOBATCH", "PLLMOFFLOAD"],
                    help="auto = the fastest schedule measured on MI355X for both workloads: NON_OVERLAP_LOCAL\n"
                         "(one stream); LOCAL measures the two-stream overlapped schedule, PLLM the reference's main\n"
                         "schedule (four QKV / attention nano-batches), PLLMOFFLOAD that with the KV offload round trip")
    ap.add_argument("--global-batch", type=int, default=2048,
                    help="offline workload: tokens per iteration the scheduler keeps (the measured configuration is 2048; "
                         "more is a what-if for a part with room for it)")
    ap.add_argument("--nano1", type=int, default=1024, help="rows of nano-batch 1")
    ap.add_argument("--kqv1", type=int, default=512)
    ap.add_argument("--kqv3", type=int, default=512)
    ap.add_argument("--decode-requests", type=int, default=1792, help="iteration workload: decode requests (one token each)")
    ap.add_argument("--prefill-chunk", type=int, default=256, help="iteration workload: tokens of the one prefill chunk (0 = none)")
    ap.add_argument("--distinct-layers", type=int, default=0,
                    help="iteration workload: distinct weight/KV layers held in HBM (0 = as many of the 32 as fit)")
    ap.add_argument("--requests", type=int, default=4096, help="offline workload: requests in the trace")
    ap.add_argument("--skip-cycles", type=int, default=1280,
                    help="offline workload: simulated scheduler cycles before the GPU runs")
    ap.add_argument("--full-run", action="store_true", help="offline workload: time the whole job")
    ap.add_argument("--kv-pages", type=int, default=0, help="offline workload: KV pool pages (0 = sized to HBM)")
    ap.add_argument("--profile-level", type=int, default=2, choices=[0, 1, 2],
                    help="per-launch events: 1 attention, 2 attention and GEMMs")
    ap.add_argument("--graph", action="store_true",
                    help="iteration workload: the timed iterations are replayed from a captured hipGraph")
    ap.add_argument("--no-graph", action="store_true", help="offline workload: run the timed cycles eagerly")
    ap.add_argument("--prime-cycles", type=int, default=48,
                    help="offline workload: untimed serving cycles before the warm-up in which the hipGraphs are captured")
    ap.add_argument("--profile-cycles", type=int, default=64,
                    help="offline workload: eager cycles with per-launch events after the timed ones (roofline records)")
    ap.add_argument("--kv-fill", default="randn", choices=["randn", "zeros"], help="offline workload: KV pool contents")
    ap.add_argument("--no-calibrate", dest="calibrate", action="store_false",
                    help="skip the in-run MFMA / HBM calibration micro-benchmarks")
    ap.add_argument("--cpu-sample", type=int, default=96, help="decode requests in the CPU baseline (0 = skip)")
    ap.add_argument("--seed", type=int, default=0)
    args = ap.parse_args()
    _check_single_gpu(args)
    if args.pipeline == "auto":
        args.pipeline = "NON_OVERLAP_LOCAL"
    rec = run_offline(args) if args.workload == "offline" else run_iteration(args)
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
