#!/usr/bin/env python3
"""Trace-driven serving run on one MI355X with the command line and result files of the
reference's pipeline/utils/serve_8B.py:

    python -m nanoflow_amd.serve -t trace.csv -c config.json -s SKIP -r CYCLES --empty_weight True -o PREFIX

* trace (pipeline/utils/frontend.py:23-58): a header line, then ``idx,input_len,output_len,arrival``
  per request; a request of input_len n gets the prompt 0, 1, ..., n-1 as in the reference.
  A row with input_len -1 carries its prompt as text after the fourth comma and is tokenized with the
  tokenizer found in the directory ``serve_configs.model`` (the reference's key, serve_8B.py:639-640;
  a hub name is not fetched: there is no network) or else ``serve_configs.hf_path``; without a
  tokenizer such rows are rejected.
* config: the reference's pipeline JSON (pipeline/config_all/llama3-8B/1024.json schema);
  ``serve_configs.pipeline_type`` is one of the reference's names (serve_8B.py:48-59): LOCAL,
  NON_OVERLAP_LOCAL, NANOBATCH_LOCAL; PLLM, NANOBATCH, PLLM_OFFLOAD (the reference's main schedule with
  four QKV / attention nano-batches, here without its exchange steps; PLLM_OFFLOAD adds the KV offload
  round trip), NON_OVERLAP (runs as NON_OVERLAP_LOCAL); for models with a bias on the q/k/v
  projections (Qwen2) KQVBIAS, NONOVERLAP_KQVBIAS, NANOBATCH_KQVBIAS.
* ``--empty_weight True``: random-init weights on the device, as the reference's own evaluation
  runs (pipeline/eval/eval-fix-offline/run.py:42-50).  Otherwise the weights come from
  ``serve_configs.weight_path``/weight_rank_0.pt (nanoflow_amd/weights.py; serve_8B.py:611-629);
  when that file is missing it is first converted from the Hugging Face checkpoint directory
  ``serve_configs.hf_path``.  Nothing is downloaded.  (The flag is parsed as a truth value here;
  the reference's ``type=bool`` turns every non-empty string, "False" included, into True.)
* ``serve_configs.weight_format`` (optional, not in the reference's schema): "f16" (default) or "e4m3" --
  the five GEMM weights of every layer are quantised on the device as they are loaded or made
  (per-output-channel scales) and served from the fp8 form.
* KV pool = ``1024 * allocate_kv_data_batch // 16`` pages per layer (serve_8B.py:643).
* writes PREFIX.stat, PREFIX.stat.csv (same columns as serve_8B.py:792-793), PREFIX.req_time,
  PREFIX.req_tokens (prompt + generated ids of every retired request, one Python list per line,
  by request index: serve_8B.py:718-722), PREFIX.req_tokens.uniq (its distinct lines with their
  counts, serve_8B.py:731) and, when a tokenizer was found, PREFIX.req_words (the same sequences
  decoded without special tokens, preceded by ``Req k:`` lines under ``--output_idx``:
  serve_8B.py:723-728).

Skip cycles advance the scheduler without GPU work and release requests by the estimated cycle
time; run cycles form batch i+1 on the CPU while the GPU runs batch i.  When every request has
arrived before the first run cycle the whole loop runs inside the library (pllm_serve); with later
arrivals the loop is driven from here, one library call per phase, releasing requests by wall time.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def load_tokenizer(serve_configs):
    """The tokenizer of the first of serve_configs.model / serve_configs.hf_path that is a local
    directory holding one, or None.  Nothing is fetched."""
    for key in ("model", "hf_path"):
        d = serve_configs.get(key)
        if d and os.path.isdir(d) and any(os.path.isfile(os.path.join(d, f))
                                          for f in ("tokenizer.json", "tokenizer.model", "tokenizer_config.json")):
            os.environ.setdefault("HF_HUB_OFFLINE", "1")
            from transformers import AutoTokenizer
            return AutoTokenizer.from_pretrained(d, local_files_only=True)
    return None


def read_trace(path, tokenizer=None):
    """[(request index, prompt ids as int32 array, output_len, arrival)] (frontend.py:23-58)."""
    reqs = []
    with open(path) as f:
        next(f, None)                                   # header
        for line in f:
            if not line.strip():
                continue
            p = line.split(",")
            n_in, n_out, arrival = int(p[1]), int(p[2]), float(p[3])
            if n_in == -1:
                if tokenizer is None:
                    raise SystemExit(f"{path}: request {p[0]} carries prompt text (input_len -1) and neither "
                                     "serve_configs.model nor serve_configs.hf_path is a directory with a tokenizer")
                text = line.split(",", 4)[4]            # everything after the fourth comma, commas included
                if text.endswith("\n"):
                    text = text[:-1]
                prompt = np.asarray(tokenizer(text)["input_ids"], dtype=np.int32)
            elif n_in < 0:
                raise SystemExit(f"{path}: request {p[0]} has input_len {n_in}")
            else:
                prompt = np.arange(n_in, dtype=np.int32)
            reqs.append((len(reqs), prompt, n_out, arrival))
    if not reqs:
        raise SystemExit(f"{path}: empty trace")
    return reqs


def parse_config(cfg):
    """(model shape, pipeline type, (global batch, nano-batch 1, kqv1, kqv3), KV pages per layer) of a
    pipeline JSON in the reference's schema."""
    from nanoflow_amd import synth, pllm_python as P
    m, mc, pc, sc = cfg["model"], cfg["model_configs"], cfg["pipeline_configs"], cfg["serve_configs"]
    if mc.get("gpu_num", 1) != 1 or sc.get("actual_gpu_num", 1) != 1:
        raise SystemExit("this build serves on one GPU (gpu_num and actual_gpu_num must be 1)")
    shape = synth.ModelShape(hidden=m["hidden_size"], Hq=m["num_attention_heads"], Hkv=m["num_key_value_heads"],
                             d=m["hidden_size"] // m["num_attention_heads"], ffn=m["intermediate_size"],
                             vocab=m["vocab_size"], layers=m["num_hidden_layers"], page_size=mc.get("frame_page_size", 16),
                             eps=m.get("rms_norm_eps", 1e-5), rope_theta=m.get("rope_theta", 1e4),
                             rope_scaling=m.get("rope_scaling") or None)   # Llama-3.1 (config_all/llama3.1-8B)
    if sc["pipeline_type"] not in P.pipeline_map:
        raise SystemExit(f"serve_configs.pipeline_type {sc['pipeline_type']!r}: one of {', '.join(P.pipeline_map)}")
    sizes = (pc["global_batch_size"], pc["nanobatch_1_size"], pc["kqv1_size"], pc["kqv3_size"])
    return shape, P.pipeline_map[sc["pipeline_type"]], sizes, 1024 * mc["allocate_kv_data_batch"] // 16   # serve_8B.py:643


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("-t", "--trace_path", required=True)
    ap.add_argument("-r", "--run_cycles", type=int, default=20)
    ap.add_argument("-c", "--config_path", required=True)
    ap.add_argument("-s", "--skip_cycles", type=int, default=0)
    ap.add_argument("--est_cycle_time", type=float, default=0.175)
    ap.add_argument("-o", "--output_prefix", default="")
    ap.add_argument("--allocate_page_num", type=int, default=740, help="accepted and unused, as in the reference")
    ap.add_argument("--empty_weight", default="False", help="random-init weights on the device instead of weight_path")
    ap.add_argument("--profile_mode", default="False", help="accepted and unused, as in the reference")
    ap.add_argument("--output_idx", default="False", help="precede every line of PREFIX.req_words by 'Req k:'")
    a = ap.parse_args()
    empty_weight = str(a.empty_weight).lower() in ("true", "1", "yes")
    prefix = a.output_prefix or a.trace_path[:-4]

    import torch
    from nanoflow_amd import engine, synth, pllm_python as P
    assert torch.cuda.is_available(), "needs the MI355X"
    cfg = json.load(open(a.config_path))
    mc, sc = cfg["model_configs"], cfg["serve_configs"]
    shape, pt, (T, nano1, kqv1, kqv3), pages = parse_config(cfg)
    # the file's GEMM tags (their B layout decides the orientation the weights are handed over in);
    # a list written for another schedule's GEMM count falls back to the default tags
    tags = cfg["pipeline_configs"].get("gemm_op_tag") or []
    tags = list(tags) if len(tags) == pt.gemm_tags else None

    weights = None
    if not empty_weight:
        from nanoflow_amd import weights as W
        wdir = sc.get("weight_path")
        if not wdir:
            raise SystemExit("serve_configs.weight_path is not set (or pass --empty_weight True)")
        if not os.path.isfile(os.path.join(wdir, W.FILE_NAME)):
            hf = sc.get("hf_path")
            if not hf or not os.path.isdir(hf):
                raise SystemExit(f"{wdir}/{W.FILE_NAME} not found and serve_configs.hf_path is not a checkpoint "
                                 "directory to convert it from")
            print("Saving weights")
            W.convert_hf_checkpoint(hf, wdir)
        print("Loading weights")
        t0 = time.perf_counter()
        weights = W.load_weight_file(wdir, shape, kqv_bias=pt.has_kqv_bias)
        print("Time taken to load weights: ", time.perf_counter() - t0)

    tokenizer = load_tokenizer(sc)
    reqs = read_trace(a.trace_path, tokenizer)
    too_big = [r[0] for r in reqs if len(r[1]) and int(r[1].max()) >= shape.vocab]
    if too_big:
        raise SystemExit(f"{a.trace_path}: request {too_big[0]} has a token id beyond the model's vocabulary of {shape.vocab}")
    avg_in = sum(len(r[1]) for r in reqs) // len(reqs)
    avg_out = sum(r[2] for r in reqs) // len(reqs)
    eng = engine.Engine(shape, pt, global_batch=T, nano1=nano1, kqv1=kqv1, kqv3=kqv3, kv_pages=pages,
                        run_layer=mc.get("run_layer", shape.layers), kv_fill="zeros", weights=weights,
                        weight_format=sc.get("weight_format", "f16"), gemm_tags=tags)
    former = P.BatchFormer(pages, shape.page_size, T, nano1, kqv1, kqv3, avg_in, avg_out)

    pending = list(reqs)                  # not yet released, in arrival order
    passed = 0.0

    def release(now_clock):
        while pending and pending[0][3] < passed:
            idx, prompt, n_out, _ = pending.pop(0)
            former.add_request(idx, prompt, n_out, now_clock)

    def busy():
        st = former.state()
        return st["queued"] + st["decoding"] + st["prefilling"]

    # ---- skip cycles: scheduler only, requests released by the estimated cycle time
    skipped = 0
    while skipped < a.skip_cycles and (pending or busy()):
        passed += a.est_cycle_time
        release(time.monotonic())
        if busy():
            former.schedule()
            former.form()
            former.advance(time.monotonic(), placeholder_zero=True)
        skipped += 1
    retired_before = former.state()["retired"]
    # first request that had not been admitted when the timed cycles start (frontend.py:67-74)
    queued = former.state()["queued"]
    start_idx = (len(reqs) - len(pending) - queued) if queued else (pending[0][0] if pending else -1)

    t1 = time.perf_counter()
    cycles = 0
    if not pending or pending[-1][3] < passed:
        # everything has arrived: the whole loop runs in the library
        release(time.monotonic())
        st = former.serve(0, a.run_cycles)
        cycles = st.cycles
    else:
        last = time.perf_counter()
        prev_ids, in_flight = None, False
        while cycles < a.run_cycles and (pending or busy()):
            now = time.perf_counter()
            passed += now - last
            last = now
            release(time.monotonic())
            if not busy():
                time.sleep(0.001)
                continue
            former.schedule()
            b = former.form()
            if b["decodePrefillBorder"] + b["prefillTokensNum"] == 0:
                continue
            if in_flight:
                P.run_async_wait()
                prev_ids = P.getPipelineOutput().copy()
            nd = b["decodePrefillBorder"]
            batch = synth.Batch(decodePrefillBorder=nd, prefillNum=b["prefillNum"], prefillTokensNum=b["prefillTokensNum"],
                                input_tokens=np.concatenate([np.zeros(nd, np.int32), b["input_tokens"]]),
                                input_indptr=b["input_indptr"], rev_input_indptr=b["rev_input_indptr"],
                                per_token_offset=b["per_token_offset"], kv_indptr=b["kv_indptr"],
                                kv_indices=b["kv_indices"], kv_last_page_len=b["kv_last_page_len"],
                                kv_len=np.zeros(0, np.int32), num_pages=pages)
            eng.update(batch, keep_token_list=b["keep_token_list"])
            P.run_async()
            in_flight = True
            if prev_ids is not None:
                former.harvest(prev_ids)
            former.advance(time.monotonic())
            cycles += 1
        if in_flight:
            P.run_async_wait()
    t2 = time.perf_counter()

    n_retired = former.state()["retired"]
    done = n_retired - retired_before
    infos = [former.retired_info(k) for k in range(n_retired)]
    outputs = dict(former.retired_output(k) for k in range(n_retired))
    eng.close()
    prompts = {r[0]: r[1] for r in reqs}
    lines = []
    for idx in sorted(outputs):
        gen = [int(t) for t in outputs[idx]]
        if gen and gen[-1] == -1:           # the placeholder of a sample that was never harvested
            gen.pop()
        lines.append([int(t) for t in prompts[idx]] + gen)
    with open(prefix + ".req_tokens", "w") as fq:
        for l in lines:
            fq.write(f"{l}\n")
    with open(prefix + ".req_tokens.uniq", "w") as fu:      # what `sort | uniq -c` prints
        import collections
        for text, n in sorted(collections.Counter(str(l) for l in lines).items()):
            fu.write(f"{n:7d} {text}\n")
    if tokenizer is not None:
        with open(prefix + ".req_words", "w") as fw:
            for k, l in enumerate(lines):
                if str(a.output_idx).lower() in ("true", "1", "yes"):
                    fw.write(f"Req {k}:\n")
                fw.write(f"{tokenizer.decode(l, skip_special_tokens=True)}\n")
    with open(prefix + ".stat", "w") as fs, open(prefix + ".stat.csv", "w") as fc, open(prefix + ".req_time", "w") as ft:
        def out(s):
            print(s)
            fs.write(s + "\n")
        if done == 0 or cycles == 0:
            print("No new request processed")
            return
        total = t2 - t1
        tps = done * (avg_in + avg_out) / total
        out(f"TOTAL Time taken: {total}")
        out(f"Token per second: {tps}")
        out(f"per GPU: {tps}")
        out(f"Total Cycle: {cycles}")
        out(f"Cycle time taken: {total / cycles}")
        out(f"start_idx: {start_idx}")
        kept = [r for r in infos if r["req_idx"] >= start_idx]
        if not kept:
            print("No fully processed request")
            return
        out(f"Actual Retired request size: {len(kept)}")
        ttft = sum(r["encode_latency"] for r in kept) / len(kept)
        tpot = sum(r["decode_latency"] / max(1, r["output_len"] - 1) for r in kept) / len(kept)
        norm = sum((r["decode_start_at"] + r["decode_latency"] - r["request_comein_time"]) / r["output_len"]
                   for r in kept) / len(kept)
        out(f"Average TTFT: {ttft}")
        out(f"Average TPOT: {tpot}")
        out(f"Average Normalize Latency: {norm}")
        fc.write("total_time,token_per_second,token_per_second_per_gpu,total_cycle,cycle_time,average_ttft,"
                 "average_tpot,average_normalize_latency\n")
        fc.write(f"{total},{tps},{tps},{cycles},{total / cycles},{ttft},{tpot},{norm}\n")
        ft.write("req_idx,input_len,output_len,req_comein_time,encode_latency,decode_start_at,decode_latency\n")
        for r in kept:
            ft.write(f"{r['req_idx']},{r['input_len']},{r['output_len']},{r['request_comein_time']},"
                     f"{r['encode_latency']},{r['decode_start_at']},{r['decode_latency']}\n")


if __name__ == "__main__":
    main()
