"""Host-side batch formation (C++, through the C ABI) against the Python restatement of the
reference scheduler and against hand-derived cases.  No GPU."""
import numpy as np
import pytest

from nanoflow_amd import pllm_python as P
from oracle import scheduler_oracle as SO

ARRS = ("input_tokens", "input_indptr", "rev_input_indptr", "per_token_offset", "kv_indptr",
        "kv_indices", "kv_last_page_len", "keep_token_list", "gemv_batch_size")
SCAL = ("decodePrefillBorder", "prefillNum", "prefillTokensNum", "keepTokenListLength")


def make_pair(kv_pages, gb, nano1, kqv1, kqv3, ap, ad, page=16):
    return (P.BatchFormer(kv_pages, page, gb, nano1, kqv1, kqv3, ap, ad),
            SO.Scheduler(kv_pages, page, gb, nano1, kqv1, kqv3, ap, ad))


def assert_same(b_cpp, b_py, cycle):
    for k in SCAL:
        assert b_cpp[k] == b_py[k], (cycle, k, b_cpp[k], b_py[k])
    for k in ARRS:
        want = np.asarray(b_py[k], dtype=np.int64)
        if k == "keep_token_list":      # the reference ships a global-batch-long list; only the
            want = want[:b_py["keepTokenListLength"]]   # first keepTokenListLength entries are read
        assert np.array_equal(np.asarray(b_cpp[k]), want), (cycle, k)


def fake_model(batch, vocab=1000):
    """Deterministic 'sampled ids' for an iteration: a hash of each request's last row."""
    ip = np.asarray(batch["input_indptr"])
    off = np.asarray(batch["per_token_offset"])
    last = ip[1:] - 1
    return ((off[last] * 7919 + np.arange(len(last)) * 104729) % vocab).astype(np.int32)


def run_both(cpp, py, cycles, check_invariants=True, gb=None):
    """Drives both formers through the asynchronous loop order of the reference
    (form i+1, then harvest outputs of i, then advance)."""
    prev_out = None
    running = 0
    stats = []
    for c in range(cycles):
        st = cpp.state()
        if st["queued"] + st["decoding"] + st["prefilling"] == 0:
            break
        cpp.schedule(); py.schedule()
        b1, b2 = cpp.form(), py.form()
        assert_same(b1, b2, c)
        if check_invariants:
            tok = b1["decodePrefillBorder"] + b1["prefillTokensNum"]
            assert tok <= gb
            # every page is owned by exactly one request
            assert len(set(b1["kv_indices"].tolist())) == len(b1["kv_indices"])
            # kv metadata is consistent with the append positions
            pages = np.diff(b1["kv_indptr"])
            kv_len = (pages - 1) * 16 + b1["kv_last_page_len"]
            last_tok = b1["input_indptr"][1:] - 1
            assert np.array_equal(b1["per_token_offset"][last_tok] + 1, kv_len)
            assert int(np.sum(b1["gemv_batch_size"])) == b1["decodePrefillBorder"]
        out = fake_model(b1)
        running += 1
        if running >= 2:                       # outputs of the previous iteration arrive now
            cpp.harvest(prev_out); py.harvest(prev_out)
        r1, r2 = cpp.advance(float(c)), py.advance()
        assert r1 == r2, (c, r1, r2)
        prev_out = out
        stats.append((b1["decodePrefillBorder"], b1["prefillTokensNum"]))
    return stats


def test_page_allocation_formula_hand_derived():
    # allocate_tokens: pages appended = (n + last_page_offset - 1) // 16 with an empty cache
    # counting as a full last page:  n=1 -> 1 page; n=16 -> 1; n=17 -> 2; then +1 token on a
    # 17-token cache (last page holds 1) -> 0 new pages; +15 -> 0; +16 -> 1.
    f = P.BatchFormer(64, 16, 64, 32, 16, 16, 17, 4)
    f.add_request(0, np.arange(17), 4)
    f.schedule()
    b = f.form()
    assert b["prefillNum"] == 1 and b["prefillTokensNum"] == 17
    assert b["kv_indptr"].tolist() == [0, 2] and b["kv_indices"].tolist() == [0, 1]
    assert b["kv_last_page_len"].tolist() == [1]
    assert b["per_token_offset"].tolist() == list(range(17))
    assert b["rev_input_indptr"].tolist() == [0] * 17
    assert b["keepTokenListLength"] == 0
    assert f.advance() == 0
    # iteration 2: the request decodes (1 row at position 17, still 2 pages, last page len 2)
    f.schedule()
    b = f.form()
    assert (b["decodePrefillBorder"], b["prefillNum"]) == (1, 0)
    assert b["per_token_offset"].tolist() == [17] and b["kv_last_page_len"].tolist() == [2]
    assert b["kv_indices"].tolist() == [0, 1]
    assert b["keepTokenListLength"] == 1 and b["keep_token_list"].tolist() == [1]
    assert b["gemv_batch_size"].tolist() == [1, 0, 0, 0]


def test_chunked_prefill_hand_derived():
    # global batch 32; a 50-token prompt is cut 32 | 18; the tail runs next to nothing else
    f = P.BatchFormer(64, 16, 32, 16, 8, 8, 50, 3)
    f.add_request(7, np.arange(100, 150), 3)
    f.schedule()
    b = f.form()
    assert b["prefillTokensNum"] == 32 and b["input_tokens"].tolist() == list(range(100, 132))
    assert b["kv_indptr"].tolist() == [0, 2] and b["kv_last_page_len"].tolist() == [16]
    assert f.advance() == 0
    f.schedule()
    b = f.form()
    assert b["decodePrefillBorder"] == 0 and b["prefillTokensNum"] == 18
    assert b["input_tokens"].tolist() == list(range(132, 150))
    assert b["per_token_offset"].tolist() == list(range(32, 50))      # continues at position 32
    assert b["kv_indptr"].tolist() == [0, 4] and b["kv_last_page_len"].tolist() == [2]
    # the chunk of the previous iteration is not kept (no sample is consumed from it)
    assert b["keepTokenListLength"] == 1 and b["keep_token_list"].tolist() == [0]
    assert f.advance() == 0
    f.schedule()
    b = f.form()                       # now decoding: 1 row, keep list marks the finished prefill
    assert b["decodePrefillBorder"] == 1 and b["keep_token_list"].tolist() == [1]
    assert b["per_token_offset"].tolist() == [50]


def test_gemv_batch_split_formula():
    # min(d, kqv1), min(rest, nano1 - kqv1), min(rest, kqv3), rest
    f = P.BatchFormer(80000, 16, 2048, 640, 256, 768, 8, 600)
    for i in range(1500):
        f.add_request(i, np.arange(8), 600)
    for _ in range(8):
        f.schedule(); b = f.form(); f.advance()
    d = b["decodePrefillBorder"]
    g = b["gemv_batch_size"].tolist()
    assert 640 < d <= 1408
    assert g == [256, 384, d - 640, 0]
    for _ in range(4):
        f.schedule(); b = f.form(); f.advance()
    d = b["decodePrefillBorder"]
    assert d > 1408
    assert b["gemv_batch_size"].tolist() == [256, 384, 768, d - 1408]


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_matches_python_restatement_constant_length(seed):
    # scaled-down constant-length trace (prefill 64 / decode 24), global batch 128
    cpp, py = make_pair(kv_pages=600, gb=128, nano1=48, kqv1=16, kqv3=40, ap=64, ad=24)
    rng = np.random.default_rng(seed)
    for i in range(60):
        prompt = rng.integers(0, 1000, size=64)
        cpp.add_request(i, prompt, 24); py.add_request(i, prompt, 24)
    stats = run_both(cpp, py, 400, gb=128)
    st = cpp.state()
    assert st["retired"] == 60 and st["queued"] == 0 and st["free_pages"] == 600
    assert len(py.retired) == 60
    for k in range(60):
        idx, out = cpp.retired_output(k)
        assert idx == py.retired[k].req_idx
        assert out.tolist() == py.retired[k].output
    # steady state keeps the batch full
    assert max(d + p for d, p in stats) == 128


def test_matches_python_restatement_variable_length_and_tight_pool():
    # variable prompt / output lengths (bounded by the lengths the forecast assumes), pool small
    # enough that the page forecast throttles admission; prompts longer than the batch are chunked
    cpp, py = make_pair(kv_pages=90, gb=96, nano1=40, kqv1=20, kqv3=28, ap=150, ad=30)
    rng = np.random.default_rng(5)
    for i in range(80):
        n, o = int(rng.integers(1, 151)), int(rng.integers(2, 31))
        prompt = rng.integers(0, 500, size=n)
        cpp.add_request(i, prompt, o); py.add_request(i, prompt, o)
    run_both(cpp, py, 3000, gb=96)
    st = cpp.state()
    assert st["retired"] == 80 and st["free_pages"] == 90
    assert np.array_equal(cpp.future_page_usage(), py.future_page_usage())


def test_future_page_usage_matches():
    cpp, py = make_pair(kv_pages=2000, gb=256, nano1=128, kqv1=64, kqv3=64, ap=100, ad=50)
    for i in range(30):
        cpp.add_request(i, np.arange(100), 50); py.add_request(i, np.arange(100), 50)
    for c in range(20):
        cpp.schedule(); py.schedule()
        assert np.array_equal(cpp.future_page_usage(), py.future_page_usage()), c
        cpp.form(); py.form(); cpp.advance(); py.advance()


def test_pool_exhaustion_is_reported_not_fatal():
    # requests far longer than the forecast's assumed lengths overrun the pool: the reference
    # asserts "Out of memory"; the C ABI returns an error and stays usable
    cpp, py = make_pair(kv_pages=12, gb=256, nano1=128, kqv1=64, kqv3=64, ap=8, ad=2)
    for i in range(4):
        cpp.add_request(i, np.arange(100), 4); py.add_request(i, np.arange(100), 4)
    cpp.schedule(); py.schedule()
    with pytest.raises(P.NanoflowPipelineError, match="Out of memory"):
        cpp.form()
    with pytest.raises(AssertionError, match="Out of memory"):
        py.form()
    assert cpp.state()["queued"] == len(py.queue)


def test_offline_trace_at_full_scale():
    # the offline-throughput workload itself: 4096 requests, 1024-token prompts, 512 outputs,
    # 2048 tokens per iteration; scheduler only (no GPU)
    f = P.BatchFormer(120000, 16, 2048, 1024, 512, 512, 1024, 512)
    rng = np.random.default_rng(0)
    for i in range(4096):
        f.add_request(i, rng.integers(0, 128256, 1024), 512)
    cycles, full, steady = 0, 0, []
    while True:
        st = f.state()
        if st["queued"] + st["decoding"] + st["prefilling"] == 0:
            break
        f.schedule()
        b = f.form()
        tok = b["decodePrefillBorder"] + b["prefillTokensNum"]
        assert tok <= 2048
        full += tok == 2048
        if 1300 <= cycles < 2800:
            steady.append(b["decodePrefillBorder"])
        assert int(np.sum(b["gemv_batch_size"])) == b["decodePrefillBorder"]
        f.advance(0.0, True)
        cycles += 1
    st = f.state()
    assert st["retired"] == 4096 and st["free_pages"] == 120000
    # every request occupies 1024 prefill rows + 511 decode rows
    assert cycles >= 4096 * 1535 // 2048
    assert full > 2900                                   # the batch is full until the trace drains
    assert 675 < np.mean(steady) < 690                   # steady state: ~682 decode rows per iteration
