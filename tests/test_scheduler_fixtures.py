"""The C++ batch former and its Python restatement against what the REFERENCE's own scheduler does
(tests/golden/scheduler_trace_*.json, written by tests/golden/make_scheduler_fixtures.py from
pipeline/utils/serve_8B.py's Scheduler in its skip-cycle mode): admission order, chunked prefill,
decode order, the attention group split, free pages and retirements, cycle by cycle over whole
traces.  Page ids are not part of the fixtures (the reference pops them from a Python set)."""
import glob
import json
import os
import zlib

import numpy as np
import pytest

from oracle import scheduler_oracle as SO

FIXTURES = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "scheduler_trace_*.json")))


def _crc(ids):
    return zlib.crc32(",".join(map(str, ids)).encode())


def _check_keep(c, prev, keep_len, keep_list):
    """The keep list handed to update c is what cycle c-1 of the reference left behind."""
    if prev is None:
        return
    assert keep_len == prev["ktl"], (c, "keepTokenListLength", keep_len, prev["ktl"])
    ones = [i for i, v in enumerate(list(keep_list)[:keep_len]) if v]
    assert _crc(ones) == prev["kcrc"], (c, "keep list", ones[:8])


def _check_cycle(c, want, nd, dec_ids, prefill, gemv, free, retired):
    assert nd == want["nd"], (c, "decode rows", nd, want["nd"])
    assert _crc(dec_ids) == want["dcrc"], (c, "decode order", dec_ids[:8])
    if "decode" in want:
        assert dec_ids == want["decode"], (c, "decode order")
    assert prefill == want["prefill"], (c, "prefill chunks", prefill, want["prefill"])
    assert list(gemv) == want["gemv"], (c, "attention groups", list(gemv), want["gemv"])
    assert free == want["free"], (c, "free pages", free, want["free"])
    assert retired == want["retired"], (c, "retired", retired, want["retired"])


def test_fixtures_are_present():
    assert len(FIXTURES) >= 3


@pytest.mark.parametrize("path", FIXTURES, ids=lambda p: os.path.basename(p)[len("scheduler_trace_"):-5])
def test_python_restatement_follows_the_reference_scheduler(path):
    t = json.load(open(path))
    s = SO.Scheduler(t["capacity"], 16, t["global_batch_size"], t["nanobatch_1_size"], t["kqv1_size"],
                     t["kqv3_size"], t["avg_prefill"], t["avg_decode"])
    for i, (n_in, n_out) in enumerate(t["requests"]):
        s.add_request(i, [i] * n_in, n_out)
    prev = None
    for c, want in enumerate(t["cycles"]):
        s.schedule()
        b = s.form()
        _check_keep(c, prev, b["keepTokenListLength"], b["keep_token_list"])
        prev = want
        dec_ids = [r.req_idx for r in s.decode]
        nd = b["decodePrefillBorder"]
        ind = b["input_indptr"]
        prefill = [[r.req_idx, ind[nd + j + 1] - ind[nd + j], b["per_token_offset"][ind[nd + j]]]
                   for j, r in enumerate(s.prefill)]
        n_ret = len(s.retired)
        s.advance(placeholder_zero=True)
        _check_cycle(c, want, nd, dec_ids, prefill, b["gemv_batch_size"], len(s.pool._free),
                     [r.req_idx for r in s.retired[n_ret:]])
    assert len(s.queue) + len(s.decode) + len(s.prefill) == 0 or len(t["cycles"]) >= 100


@pytest.mark.parametrize("path", FIXTURES, ids=lambda p: os.path.basename(p)[len("scheduler_trace_"):-5])
def test_cpp_batch_former_follows_the_reference_scheduler(path):
    from nanoflow_amd import pllm_python as P
    t = json.load(open(path))
    f = P.BatchFormer(t["capacity"], 16, t["global_batch_size"], t["nanobatch_1_size"], t["kqv1_size"],
                      t["kqv3_size"], t["avg_prefill"], t["avg_decode"])
    try:
        for i, (n_in, n_out) in enumerate(t["requests"]):
            f.add_request(i, np.full(n_in, i, np.int32), n_out)      # the prompt's tokens name the request
        owner = {}                                                   # first KV page -> request
        prev = None
        for c, want in enumerate(t["cycles"]):
            f.schedule()
            b = f.form()
            _check_keep(c, prev, b["keepTokenListLength"], b["keep_token_list"])
            prev = want
            nd, ind, kvp, kvi = b["decodePrefillBorder"], b["input_indptr"], b["kv_indptr"], b["kv_indices"]
            prefill = []
            for j in range(b["prefillNum"]):
                lo, hi = int(ind[nd + j]), int(ind[nd + j + 1])
                req = int(b["input_tokens"][lo - nd])
                assert np.all(b["input_tokens"][lo - nd:hi - nd] == req)
                prefill.append([req, hi - lo, int(b["per_token_offset"][lo])])
                owner[int(kvi[kvp[nd + j]])] = req
            dec_ids = [owner[int(kvi[kvp[i]])] for i in range(nd)]
            n_ret = f.state()["retired"]
            f.advance(0.0, placeholder_zero=True)
            st = f.state()
            retired = [f.retired_info(k)["req_idx"] for k in range(n_ret, st["retired"])]
            _check_cycle(c, want, nd, dec_ids, prefill, b["gemv_batch_size"], st["free_pages"], retired)
    finally:
        f.close()
