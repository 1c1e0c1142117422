"""Pure-Python restatement of the reference's CPU batch formation and paged-KV bookkeeping.

TEST INFRASTRUCTURE ONLY (the checker for csrc/host/batchFormer.cpp).

Follows, function by function:
  KVPool / KVCache     pipeline/utils/kv_cache.py:20-104 (DistKVPool, DistKVCache)
  batched metadata     pipeline/utils/kv_cache.py:112-135 (BatchedDistKVCache.__init__)
  Scheduler            pipeline/utils/serve_8B.py:104-569 (check_future_page_usage :177-203,
                       schedule_req :212-346, bench_text_gen :348-569), with the GPU calls
                       replaced by a callback that returns the sampled ids of an iteration.
One stated freedom: which free page is handed out.  The reference pops from a Python ``set``
(CPython implementation detail); here the pool is a LIFO stack that first issues 0, 1, 2, ...
and re-issues the most recently freed page first -- the same rule as the C++ former, so the
two can be compared bit for bit.

Parity status: pinned.  The integer formulas by hand-derived cases in tests/test_batch_former.py;
the behaviour over whole traces (admission order, chunked prefill, decode order, group split, free
pages, retirements per cycle) by tests/golden/scheduler_trace_*.json, which
tests/golden/make_scheduler_fixtures.py wrote by running the reference's own Scheduler in its
skip-cycle mode (tests/test_scheduler_fixtures.py).  Page ids are outside the fixtures.
"""
from __future__ import annotations

import numpy as np


class KVPool:
    def __init__(self, capacity: int, page_size: int):
        self.capacity = capacity
        self.page_size = page_size
        self._free = list(range(capacity - 1, -1, -1))   # pop() -> 0, 1, 2, ...

    @property
    def num_free_pages(self) -> int:
        return len(self._free)

    def alloc_page(self) -> int:
        assert len(self._free) > 0, "Out of memory"
        return self._free.pop()

    def free_page(self, idx: int):
        self._free.append(idx)


class KVCache:
    def __init__(self, pool: KVPool):
        self._pool = pool
        self.indices: list[int] = []
        self.seqlen = 0

    @property
    def last_page_offset(self) -> int:
        return (self.seqlen - 1) % self._pool.page_size + 1

    def allocate_tokens(self, num_tokens: int):
        assert 0 < num_tokens <= self._pool.num_free_pages * self._pool.page_size, "Out of memory"
        appended = (num_tokens + self.last_page_offset - 1) // self._pool.page_size
        for _ in range(appended):
            self.indices.append(self._pool.alloc_page())
        self.seqlen += num_tokens

    def release(self):
        self.seqlen = 0
        for idx in self.indices:
            self._pool.free_page(idx)
        self.indices.clear()


class Fly:
    def __init__(self, req_idx, input, output, prompt, chunked_prefill, kv_cache, output_len, input_len):
        self.req_idx = req_idx
        self.input = list(input)
        self.output = list(output)
        self.prompt = prompt
        self.chunked_prefill = chunked_prefill
        self.kv_cache = kv_cache
        self.output_len = output_len
        self.input_len = input_len


class Scheduler:
    def __init__(self, kv_pages, page_size, global_bsz, nano1, kqv1, kqv3, avg_prefill, avg_decode):
        self.pool = KVPool(kv_pages, page_size)
        self.global_bsz, self.nano1, self.kqv1, self.kqv3 = global_bsz, nano1, kqv1, kqv3
        self.avg_prefill, self.avg_decode = avg_prefill, avg_decode
        self.queue: list = []
        self.decode: list[Fly] = []
        self.prefill: list[Fly] = []
        self.new_decode: list[Fly] = []
        self.new_prefill: list[Fly] = []
        self.old_decode: list[Fly] = []
        self.old_prefill: list[Fly] = []
        self.keep_list = np.zeros(0, np.int32)
        self.old_token_length = 0
        self.retired: list[Fly] = []

    def add_request(self, req_idx, prompt, output_len):
        self.queue.append((req_idx, list(prompt), output_len))

    @staticmethod
    def _eff(ws):
        return sum(len(r.input) for r in ws)

    def future_page_usage(self):
        P = self.pool.page_size
        max_seq_len = self.avg_decode + self.avg_prefill + 2
        usage = np.zeros(max_seq_len, dtype=np.int64)
        idx = np.arange(max_seq_len, dtype=np.int64)
        for req in self.decode:
            cur = req.kv_cache.seqlen + 1
            usage[0:max_seq_len - cur] += (idx[:max_seq_len - cur] + cur + P - 1) // P
        for _ in self.prefill:
            cur = self.avg_prefill + 1
            usage[0:max_seq_len - cur] += (idx[:max_seq_len - cur] + cur + P - 1) // P
        return usage

    def schedule(self):
        self.new_decode, self.new_prefill = [], []
        P = self.pool.page_size
        decode_idle = self.global_bsz - self._eff(self.decode)
        prefill_idle = self.global_bsz - self._eff(self.prefill) - self._eff(self.decode)
        future = self.future_page_usage()
        min_avail = self.pool.capacity - np.max(future)
        max_seq_len = self.avg_decode + self.avg_prefill + 2
        idx = np.arange(max_seq_len, dtype=np.int64)
        while prefill_idle > 0 and decode_idle > 0 and len(self.queue) > 0 and \
                min_avail > (self.avg_prefill + self.avg_decode + P) // P:
            req_idx, prompt, output_len = self.queue.pop(0)
            kv = KVCache(self.pool)
            n = len(prompt)
            if n > prefill_idle:
                self.prefill.append(Fly(req_idx, prompt[:prefill_idle], [], prompt, True, kv, output_len, n))
                self.new_prefill.append(Fly(req_idx, prompt[prefill_idle:], [], prompt, False, kv, output_len, n))
                prefill_idle = 0
                decode_idle -= 1
            else:
                self.prefill.append(Fly(req_idx, prompt, [], prompt, False, kv, output_len, n))
                prefill_idle -= n
                decode_idle -= 1
            cur = self.avg_prefill + 1
            future[0:max_seq_len - cur] += (idx[:max_seq_len - cur] + cur + P - 1) // P
            min_avail = self.pool.capacity - np.max(future)
        if prefill_idle < 0:
            assert len(self.prefill) == 1, "At most add one large prefill each iteration."
            over = -prefill_idle
            head = self.prefill[0]
            self.new_prefill.append(Fly(head.req_idx, head.input[-over:], [], head.prompt, False,
                                        head.kv_cache, head.output_len, head.input_len))
            head.input = head.input[:-over]
            head.chunked_prefill = True

    def form(self) -> dict:
        input_ids = []
        for req in self.prefill:
            input_ids.extend(req.input)
        for req in self.prefill:
            req.kv_cache.allocate_tokens(len(req.input))
        for req in self.decode:
            req.kv_cache.allocate_tokens(len(req.input))
        dpb = self._eff(self.decode)
        g = [0, 0, 0, 0]
        g[0] = min(dpb, self.kqv1)
        g[1] = min(dpb - g[0], self.nano1 - self.kqv1)
        g[2] = min(dpb - g[0] - g[1], self.kqv3)
        g[3] = dpb - g[0] - g[1] - g[2]
        input_indptr, prev_len = [0], []
        kv_indptr, kv_indices, kv_last = [0], [], []
        for req in self.decode:
            input_indptr.append(input_indptr[-1] + len(req.input))
            prev_len.append(req.kv_cache.seqlen - 1)
        for req in self.prefill:
            input_indptr.append(input_indptr[-1] + len(req.input))
            prev_len.append(req.kv_cache.seqlen - len(req.input))
        for req in self.decode + self.prefill:
            kv_indices.extend(req.kv_cache.indices)
            kv_last.append(req.kv_cache.last_page_offset)
            kv_indptr.append(kv_indptr[-1] + len(req.kv_cache.indices))
        rev, off = [], []
        for i in range(len(input_indptr) - 1):
            for j in range(input_indptr[i], input_indptr[i + 1]):
                rev.append(i)
                off.append(j - input_indptr[i] + prev_len[i])
        return dict(decodePrefillBorder=dpb, prefillNum=len(self.prefill), prefillTokensNum=len(input_ids),
                    keepTokenListLength=self.old_token_length, input_tokens=input_ids,
                    input_indptr=input_indptr, rev_input_indptr=rev, per_token_offset=off,
                    kv_indptr=kv_indptr, kv_indices=kv_indices, kv_last_page_len=kv_last,
                    keep_token_list=list(self.keep_list), gemv_batch_size=g)

    def harvest(self, output_ids):
        if output_ids is None or len(output_ids) == 0:
            return
        for i, req in enumerate(self.old_prefill):
            if not req.chunked_prefill:
                req.output[-1] = int(output_ids[i + len(self.old_decode)])
                req.input = [req.output[-1]]
        for i, req in enumerate(self.old_decode):
            req.output[-1] = int(output_ids[i])
            req.input = [req.output[-1]]

    def advance(self, placeholder_zero=False):
        self.old_token_length = len(self.decode) + len(self.prefill)
        append_token_id = 0 if placeholder_zero else -1
        keep = np.zeros(self.global_bsz, np.int32)
        n_retired = 0
        for i, req in enumerate(self.decode):
            if len(req.output) >= req.output_len - 1:
                req.kv_cache.release()
                self.retired.append(req)
                n_retired += 1
            else:
                keep[i] = 1
                req.output.append(append_token_id)
                req.input = [0]
                self.new_decode.append(req)
        for i, req in enumerate(self.prefill):
            if not req.chunked_prefill:
                keep[len(self.decode) + i] = 1
                req.input = [0]
                req.output.append(append_token_id)
                self.new_decode.append(req)
        self.keep_list = keep
        self.old_decode, self.old_prefill = self.decode, self.prefill
        self.decode, self.prefill = self.new_decode, self.new_prefill
        self.new_decode, self.new_prefill = [], []
        return n_retired
