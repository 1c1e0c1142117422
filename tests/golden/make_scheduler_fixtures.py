#!/usr/bin/env python3
"""Writes tests/golden/scheduler_trace_*.json: what the REFERENCE's own scheduler does, cycle by
cycle, on constant-length and mixed-length traces -- the one part of the path that nothing else
pins (admission order over long traces: Scheduler.schedule_req / bench_text_gen of
pipeline/utils/serve_8B.py:212-569 with pipeline/utils/kv_cache.py and request_info.py).

Run in the build container only (it imports the reference from /root/reference; the GPU box has
neither the reference nor a use for this script):

    python tests/golden/make_scheduler_fixtures.py

The reference's scheduler is driven exactly as its evaluation drives it before the timed cycles:
``bench_text_gen(retired, actualRun=False)`` (serve_8B.py:657-663, the --skip_cycles loop), the mode
in which it calls nothing of the compiled extension.  Three accommodations, none of which touches
the scheduling logic:
  * the modules import the compiled extension ``pllm_python`` at top level; an empty stand-in
    module with the names evaluated at import time (the PipelineType members, the class named in
    an annotation) is put in sys.modules -- no function of it is ever called;
  * DistKVPool.__init__ probes ``torch.zeros(1, device="cuda:0")``; the pool object is created
    with __new__ and given the same fields (kv_cache.py:43-51);
  * Tensor.pin_memory needs an accelerator; it is replaced by the identity for this process.
Page ids are left out of the fixtures: the reference pops them from a Python set, an order its
own code does not define.  Everything else the scheduler decides is recorded per cycle.
"""
from __future__ import annotations

import enum
import io
import json
import os
import sys
import tempfile
import types
import zlib

REF = "/root/reference/pipeline/utils"
HERE = os.path.dirname(os.path.abspath(__file__))


def import_reference():
    stub = types.ModuleType("pllm_python")
    stub.PipelineType = enum.Enum("PipelineType", ["LOCAL", "PLLM", "NONOVERLAP", "NANOBATCH", "PLLMOFFLOAD",
                                                   "NON_OVERLAP_LOCAL", "NANOBATCH_LOCAL", "KQVBIAS",
                                                   "NANOBATCH_KQVBIAS", "NONOVERLAP_KQVBIAS"])
    for name in ("VortexModelWeight", "VortexLayerWeight", "VortexWeight", "VortexInitData", "VortexUpdateData",
                 "VortexConfigData"):
        setattr(stub, name, type(name, (), {}))
    sys.modules["pllm_python"] = stub
    import torch
    torch.Tensor.pin_memory = lambda self, *a, **k: self
    sys.path.insert(0, REF)
    os.chdir(tempfile.mkdtemp(prefix="nf_fixture_"))     # the module opens serve.log in the cwd
    import serve_8B
    import kv_cache
    import request_info
    return serve_8B, kv_cache, request_info


def run_trace(mods, name, requests, capacity, T, nano1, kqv1, kqv3, cycles):
    serve_8B, kv_cache, request_info = mods
    pool = kv_cache.DistKVPool.__new__(kv_cache.DistKVPool)
    pool._free = set(range(capacity))
    pool.num_layers, pool.num_kv_heads, pool.head_dim = 1, 8, 128
    pool.capacity, pool.page_size, pool.num_devices = capacity, 16, 1
    queue = request_info.NewRequestQueue()
    for i, (n_in, n_out) in enumerate(requests):
        r = request_info.NewRequestInfo()
        r.req_idx, r.prompt, r.output_len, r.start_time = i, list(range(n_in)), n_out, 0.0
        queue.put(r)
    avg_in = sum(r[0] for r in requests) // len(requests)
    avg_out = sum(r[1] for r in requests) // len(requests)
    serve_8B.file_schedule = io.StringIO()
    sch = serve_8B.Scheduler(pool, queue, [], avg_out, avg_in)
    # what init_pipe (serve_8B.py:131-147) derives from the pipeline config
    sch.config_data = types.SimpleNamespace(globalBatchSize=T, nanobatch1Size=nano1, kqv1Size=kqv1, kqv3Size=kqv3)
    sch._global_bsz = T
    sch._decode_bsz = T * avg_out // (avg_out + avg_in)
    sch._prefill_bsz = T * avg_in // (avg_out + avg_in)
    retired = []
    out = []
    real_stdout = sys.stdout
    sys.stdout = io.StringIO()                            # the loop prints per cycle
    try:
        for _ in range(cycles):
            if queue.size + sch._decode_workset.size + sch._prefill_workset.size == 0:
                break
            n_ret = len(retired)
            sch.bench_text_gen(retired, actualRun=False)
            dec, pre = sch._old_decode, sch._old_prefill   # the iteration that was just formed
            indptr = list(sch._old_input_indptr)
            nd = len(dec._set)
            # chunk lengths come from input_indptr: a request whose prefill completed has had its
            # .input replaced by the placeholder of its first decode step by now (serve_8B.py:555)
            chunk = [indptr[nd + j + 1] - indptr[nd + j] for j in range(len(pre._set))]
            dec_ids = [r.req_idx for r in dec._set]
            assert indptr[:nd + 1] == list(range(nd + 1))           # one row per decode request
            rec = {
                # decode requests in batch order: count and CRC-32 of the comma-joined ids (the
                # full list every 16th cycle), to keep the fixture small
                "nd": nd, "dcrc": zlib.crc32(",".join(map(str, dec_ids)).encode()),
                # [request, chunk length, tokens already in its KV before this chunk]
                "prefill": [[r.req_idx, chunk[j], r.kv_cache.seqlen - chunk[j]] for j, r in enumerate(pre._set)],
                "gemv": list(sch._gemv_batch_size),
                "free": pool.num_free_pages,
                "retired": [r.req_idx for r in retired[n_ret:]],
                # the keep list this cycle leaves for the next update (serve_8B.py:527-560): how many
                # slots of this iteration's output it covers, and which of them decode again
                "ktl": sch._old_token_length,
                "kcrc": zlib.crc32(",".join(str(i) for i, v in enumerate(sch.pinned_keep_token_list.tolist()) if v).encode()),
            }
            if len(out) % 16 == 0:
                rec["decode"] = dec_ids
            out.append(rec)
    finally:
        sys.stdout = real_stdout
    return {"name": name, "requests": requests, "capacity": capacity, "global_batch_size": T,
            "nanobatch_1_size": nano1, "kqv1_size": kqv1, "kqv3_size": kqv3, "avg_prefill": avg_in,
            "avg_decode": avg_out, "cycles": out}


def main():
    mods = import_reference()
    import random
    rnd = random.Random(7)
    traces = {
        # the benchmark's shape, scaled down 8x: constant lengths, pool sized so that the page
        # forecast (not the batch size) limits admission
        "const": ([(128, 64)] * 160, 300, 256, 128, 64, 64, 300),
        # mixed lengths, tight pool
        "mixed": ([(rnd.randint(5, 300), rnd.randint(2, 90)) for _ in range(120)], 420, 256, 96, 32, 96, 500),
        # prompts longer than an iteration: chunked prefill over several cycles
        "long_prompts": ([(rnd.randint(200, 700), rnd.randint(2, 40)) for _ in range(40)], 700, 256, 128, 64, 64, 400),
    }
    for name, (reqs, cap, T, n1, k1, k3, cycles) in traces.items():
        rec = run_trace(mods, name, [list(r) for r in reqs], cap, T, n1, k1, k3, cycles)
        path = os.path.join(HERE, f"scheduler_trace_{name}.json")
        with open(path, "w") as f:
            json.dump(rec, f, separators=(",", ":"))
        print(name, len(rec["cycles"]), "cycles ->", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
