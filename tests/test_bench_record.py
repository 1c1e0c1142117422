"""bench.py without a GPU: the figures it quotes from the committed rocprofv3 summaries are there to be
read, the algorithmic work it prices launches with matches the formulas stated for the kernels, and more
than one GPU is refused with a message."""
import importlib.util
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    m = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(m)
    return m


def test_traffic_ratios_and_overlap_note_come_from_the_committed_profiles():
    b = _bench()
    # measured ratios of HBM traffic to algorithmic bytes: a decode-attention launch reads every KV byte
    # once; a GEMM's panels are fetched once per XCD and round
    assert b.DECODE_ATTN_TRAFFIC_RATIO is not None and 1.0 <= b.DECODE_ATTN_TRAFFIC_RATIO < 1.05
    assert b.GEMM_TRAFFIC_RATIO is not None and 1.0 < b.GEMM_TRAFFIC_RATIO < 4.0
    note = b._overlap_note()
    assert note.startswith("measured, loses by ") and "profiles/schedules_offline_cycle.txt" in note
    note = b._overlap_note("iteration")
    assert note.startswith("measured, loses by ") and "per iteration" in note and "schedules_dense_iteration.txt" in note
    assert b._profile_figure("no_such_profile.txt", r"x = ([0-9.]+)") is None
    assert b._profile_figure("schedules_offline_cycle.txt", r"no such line = ([0-9.]+)") is None


def test_algorithmic_bytes_of_a_decode_attention_launch():
    """K and V once, q and o rows, page indices and the two index arrays: the per-request figure of the
    reference's decode benchmark (gemv/src/bench_batch_decode.cu:77-81) summed over the launch."""
    b = _bench()
    kv = np.array([1024, 1536, 17], dtype=np.int64)
    Hq, Hkv, d, page = 32, 8, 128, 16
    want = 0
    for L in kv:
        want += 2 * L * Hkv * d * 2          # K and V, fp16
        want += 2 * Hq * d * 2               # the q row and the o row
        want += 4 * (-(-L // page) + 2)      # page ids, kv_indptr and kv_last_page_len entries
    assert b.decode_attention_bytes(kv, Hq, Hkv, d, page) == want


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0 and "ONE GPU" in (r.stderr + r.stdout) and not r.stdout.strip().startswith("{")
