#!/usr/bin/env python3
"""Kernel-level throughput of the HIP operators at the pipeline's own shapes (one MI355X).

    python -m nanoflow_amd.kernel_bench --op gemm --m 2048            # KQV, O, down, LM head
    python -m nanoflow_amd.kernel_bench --op dual --m 1024
    python -m nanoflow_amd.kernel_bench --op gemm_f8 --m 2048 --model 70b
    python -m nanoflow_amd.kernel_bench --op dual_f8 --m 2048 --model 70b     # fused fp8 gate/up pair
    python -m nanoflow_amd.kernel_bench --op attn --requests 1792 --kv-lo 1024 --kv-hi 1536
    python -m nanoflow_amd.kernel_bench --op prefill --chunks 755:269,0:1024,0:74
    python -m nanoflow_amd.kernel_bench --op copy                     # counter-calibration kernel
    python -m nanoflow_amd.kernel_bench --op calibrate                # measured MFMA / HBM / paged-read ceilings
    python -m nanoflow_amd.kernel_bench --op blas --m 2048            # the same GEMM shapes through torch.matmul (hipBLASLt / rocBLAS)
    python -m nanoflow_amd.kernel_bench --op corun                    # GEMM and decode attention alone and together: time and board power
    python -m nanoflow_amd.kernel_bench --op cusplit                  # the same pair on CU-masked streams (disjoint CU sets, the same on every XCD)

Each line reports the average launch time over --iters launches (HIP events on the launch
stream) and the algorithmic rate: 2*M*N*K flops (4*M*N*K for the fused gate/up pair), or the
decode-attention bytes of gemv/src/bench_batch_decode.cu:77-81 (K and V once, q and o, page
indices).  --iters 1 --warm 0 gives one launch per shape, for counter collection.
"""
from __future__ import annotations

import argparse
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from nanoflow_amd import kernels as K, synth  # noqa: E402

DEV = "cuda"


WARM_MS = 0.0   # --warm-ms: keep launching for this long before timing (the clocks of a part that sat
                # idle take tens of milliseconds of load to settle; short cold runs read 5-15 % low)


def timeit(fn, iters, warm):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    if WARM_MS > 0:
        import time
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < WARM_MS:
            for _ in range(5):
                fn()
            torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) / iters


def cold_copies(W, cold: bool):
    """An endless iterator over W, or (--cold) over enough copies of it that a launch never finds its
    weights in the 256 MB last-level cache: the way a layer's weights arrive in the pipeline, where
    a model's 15 to 140 GB of weights pass through between two uses of the same matrix."""
    import itertools
    if not cold:
        return itertools.repeat(W)
    n = max(2, -(-(1 << 30) // (W.numel() * W.element_size())))   # at least 1 GiB of distinct weights
    return itertools.cycle([W] + [W.clone() for _ in range(n - 1)])


def layer_shapes(shape: synth.ModelShape, M: int):
    return [("kqv", M, shape.kqv_n, shape.hidden), ("o", M, shape.hidden, shape.Hq * shape.d),
            ("down", M, shape.hidden, shape.ffn), ("lm_head", (M + 127) // 128 * 128, shape.vocab, shape.hidden)]


class PowerSampler:
    """Board power from the amdgpu hwmon file (microwatts), sampled every 50 ms on a thread."""

    def __init__(self):
        import glob, threading
        self.paths = [p for d in glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*")
                      for p in (os.path.join(d, "power1_input"), os.path.join(d, "power1_average")) if os.path.exists(p)]
        self.samples, self.stop = [], False
        self.thread = threading.Thread(target=self._run, daemon=True)
        self.thread.start()

    def _run(self):
        import time
        while not self.stop:
            try:
                w = max(int(open(p).read()) / 1e6 for p in self.paths)
            except (OSError, ValueError):
                w = float("nan")
            self.samples.append((time.perf_counter(), w))
            time.sleep(0.05)

    def mean(self, t0, t1):
        v = [w for t, w in self.samples if t0 <= t <= t1 and w == w]
        return sum(v) / len(v) if v else float("nan")


def masked_stream(first_cu: int, n_cu: int):
    """A stream restricted to CUs first_cu .. first_cu + n_cu - 1 (multiples of 4) of EVERY XCD.  Bit i
    of the CU mask is a CU of XCD i % 8 on this part (a kernel that records its XCC id under a mask
    shows it), so one 32-bit word holds 4 CUs of each of the 8 XCDs."""
    import ctypes as C
    assert first_cu % 4 == 0 and n_cu % 4 == 0 and 0 < n_cu and first_cu + n_cu <= 32
    hip = C.CDLL("libamdhip64.so")
    s = C.c_void_p()
    mask = (C.c_uint32 * 8)(*[0xFFFFFFFF if first_cu // 4 <= i < (first_cu + n_cu) // 4 else 0 for i in range(8)])
    rc = hip.hipExtStreamCreateWithCUMask(C.byref(s), 8, mask)
    assert rc == 0, f"hipExtStreamCreateWithCUMask: {rc}"
    return torch.cuda.ExternalStream(s.value)


def corun(a, shape, rnd):
    """The fused gate/up GEMM (M rows) and decode attention (the offline cycle's request mix), each alone
    and both at once on two streams: time per pair against the serial sum, and board power."""
    import time
    M = a.m
    A, Bg, Bu = rnd(M, shape.hidden), rnd(shape.hidden, shape.ffn, std=0.02), rnd(shape.hidden, shape.ffn, std=0.02)
    out = torch.empty(M, shape.ffn, dtype=torch.float16, device=DEV)
    gemm = lambda: K.dual_swiglu(A, Bg, Bu, out=out)
    fl = 4.0 * M * shape.ffn * shape.hidden
    b = synth.config2_batch(seed=0, n_decode=a.requests, lo=a.kv_lo, hi=a.kv_hi, prefill_chunk=16)
    nd = b.decodePrefillBorder
    pool = rnd(b.num_pages, 2, shape.page_size, shape.Hkv, shape.d)
    q = rnd(b.tokens, shape.Hq * shape.d)
    o = torch.zeros_like(q)
    t = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(DEV)
    qi, kvp, kvi, kvl = t(b.input_indptr[:nd + 1]), t(b.kv_indptr[:nd + 1]), t(b.kv_indices), t(b.kv_last_page_len[:nd])
    ws = torch.empty(1 << 20, dtype=torch.uint8, device=DEV)
    attn = lambda: K.attention_paged(q, qi, pool, kvp, kvi, kvl, shape.Hq, shape.Hkv, causal=False, out=o, batch=nd,
                                     max_qo_rows=nd, workspace=ws)
    L = b.kv_len[:nd].astype(np.int64)
    nb = int((2 * L * shape.Hkv * shape.d * 2).sum())
    power = PowerSampler()

    def phase(name, fn, note=None, secs=2.5):
        torch.cuda.synchronize()
        t0, n = time.perf_counter(), 0
        while time.perf_counter() - t0 < secs:
            for _ in range(5):
                fn()
            torch.cuda.synchronize()
            n += 5
        t1 = time.perf_counter()
        per = (t1 - t0) / n
        print(f"{name:44s} {per * 1e6:9.1f} us  board power {power.mean(t0 + 0.5, t1):7.1f} W"
              + (f"  {note(per)}" if note else ""), flush=True)
        return per

    time.sleep(1.0)
    print(f"idle: board power {power.mean(0, time.perf_counter()):7.1f} W", flush=True)
    tg = phase(f"gate/up GEMM {M}x{shape.ffn}x{shape.hidden} alone", gemm, lambda p: f"{fl / p / 1e12:7.1f} TFLOP/s")
    ta = phase(f"decode attention {nd} requests alone", attn, lambda p: f"{nb / p / 1e9:7.1f} GB/s")
    if a.op == "corun":
        s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
        splits = [("both, two unmasked streams", s1, s2)]
    else:
        splits = [(f"both, GEMM on {gc} + attention on {32 - gc} CUs of every XCD", masked_stream(0, gc),
                   masked_stream(gc, 32 - gc)) for gc in (24, 20, 16, 12)]
    for name, sg, sa in splits:
        def both():
            with torch.cuda.stream(sg):
                gemm()
            with torch.cuda.stream(sa):
                attn()
        if a.op == "cusplit":
            def g_only():
                with torch.cuda.stream(sg):
                    gemm()
            def a_only():
                with torch.cuda.stream(sa):
                    attn()
            phase("  GEMM alone on its CUs", g_only, lambda p: f"{fl / p / 1e12:7.1f} TFLOP/s", secs=1.5)
            phase("  attention alone on its CUs", a_only, lambda p: f"{nb / p / 1e9:7.1f} GB/s", secs=1.5)
        phase(name, both, lambda p: f"serial sum {(tg + ta) * 1e6:7.1f} us -> x{(tg + ta) / p:.3f}")
    if a.op == "corun":
        phase("mfma loop f16, pseudo-random operands", lambda: K.calibrate_mfma(False, True, 2000), secs=2.0)
        phase("mfma loop f16, zero operands", lambda: K.calibrate_mfma(False, False, 2000), secs=2.0)
        phase("mfma loop f16, pseudo-random operands re-read from LDS", lambda: K.calibrate_mfma(False, 2, 2000), secs=2.0)
        phase("   ... with the tile's operand loads (L2 -> LDS) beside them", lambda: K.calibrate_mfma(False, 3, 2000), secs=2.0)
        phase("mfma loop f16 on 16x16x32 instructions, pseudo-random operands", lambda: K.calibrate_mfma(False, 4, 2000), secs=2.0)
        buf = torch.empty(4 << 30, dtype=torch.uint8, device=DEV).random_()
        sc = torch.zeros(8192, dtype=torch.uint8, device=DEV)
        import ctypes as C
        gb = C.c_double()
        phase("hbm read stream 4 GiB x 2", lambda: K.lib().nf_calibrate_hbm_read(buf.data_ptr(), buf.numel(), 2, sc.data_ptr(),
                                                                                 8192, C.byref(gb), None), secs=2.0)
    power.stop = True


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--op", required=True, choices=["gemm", "dual", "gemm_f8", "dual_f8", "attn", "prefill", "copy", "calibrate", "blas",
                                                  "corun", "cusplit"])
    ap.add_argument("--chunks", default="755:269,0:1024,0:74",
                    help="prefill: prev_len:chunk_len per request (default: a steady-state offline iteration)")
    ap.add_argument("--model", default="8b", choices=["8b", "70b"])
    ap.add_argument("--m", type=int, default=2048, help="rows (tokens) of the GEMM operand")
    ap.add_argument("--only", default="", help="gemm: run only this role (kqv, o, down, lm_head)")
    ap.add_argument("--requests", type=int, default=1792)
    ap.add_argument("--kv-lo", type=int, default=1024)
    ap.add_argument("--kv-hi", type=int, default=1536)
    ap.add_argument("--num-blocks", type=int, default=0, help="attn: cap on resident workgroups (0 = none)")
    ap.add_argument("--mib", type=int, default=1024, help="copy: MiB moved")
    ap.add_argument("--dtype", default="f16", choices=["f16", "bf16"], help="gemm, dual: element type")
    ap.add_argument("--b-col-major", action="store_true", help="gemm: weights stored [N][K] (k contiguous)")
    ap.add_argument("--tile", default="", help="gemm: MxN, the tile to run on (the closest of the library's menu) instead of its own choice")
    ap.add_argument("--split-k", type=int, default=1, help="gemm with --tile: shares K is cut into")
    ap.add_argument("--cold", action="store_true",
                    help="gemm, dual, gemm_f8, dual_f8, blas: cycle through 1 GiB of weight copies so that every launch streams its weights from HBM")
    ap.add_argument("--ws", action="store_true", help="gemm: the entry point with a workspace (split over K where it pays)")
    ap.add_argument("--warm-ms", type=float, default=300.0,
                    help="gemm, dual, blas, attn: keep launching this long before timing (0: only --warm launches)")
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--warm", type=int, default=3)
    a = ap.parse_args()
    global WARM_MS
    WARM_MS = a.warm_ms if a.iters > 2 else 0.0      # counter-collection runs (--iters 1 or 2) stay short
    assert torch.cuda.is_available(), "needs the MI355X"
    shape = synth.LLAMA3_8B if a.model == "8b" else synth.LLAMA3_70B
    g = torch.Generator(device=DEV).manual_seed(0)
    rnd = lambda *s, std=1.0: torch.empty(s, dtype=torch.float16, device=DEV).normal_(0, std, generator=g)
    edt = torch.float16 if a.dtype == "f16" else torch.bfloat16   # element type of the gemm / dual operands

    if a.op in ("gemm", "gemm_f8"):
        for name, M, N, Kd in layer_shapes(shape, a.m):
            if a.only and name != a.only:
                continue
            out = torch.empty(M, N, dtype=edt if a.op == "gemm" else torch.float16, device=DEV)
            if a.op == "gemm":
                A = rnd(M, Kd).to(edt)
                B = (rnd(N, Kd, std=0.02) if a.b_col_major else rnd(Kd, N, std=0.02)).to(edt)
                Bs = cold_copies(B, a.cold)
                if a.tile:
                    tm, tn = (int(v) for v in a.tile.lower().split("x"))
                    ws = torch.empty((max(K.lib().nf_gemm_tiled_workspace_bytes(M, N, Kd, a.split_k), 16),), dtype=torch.uint8, device=DEV)
                    fn = lambda: K.gemm_tiled(A, next(Bs), (tm, tn), a.split_k, b_col_major=a.b_col_major, out=out, workspace=ws)
                elif a.ws:
                    ws = torch.empty((max(K.lib().nf_gemm_workspace_bytes(M, N, Kd), 16),), dtype=torch.uint8, device=DEV)
                    fn = lambda: K.gemm_ws(A, next(Bs), out=out, b_col_major=a.b_col_major, workspace=ws)
                else:
                    fn = lambda: K.gemm(A, next(Bs), out=out, b_col_major=a.b_col_major)
            else:
                Aq = torch.randint(0, 120, (M, Kd), dtype=torch.uint8, device=DEV)
                Bq = torch.randint(0, 120, (N, Kd), dtype=torch.uint8, device=DEV)
                sa, sb = torch.ones(M, device=DEV), torch.ones(N, device=DEV)
                Bqs = cold_copies(Bq, a.cold)
                fn = lambda: K.gemm_f8(Aq, sa, next(Bqs), sb, out=out)
            ms = timeit(fn, a.iters, a.warm)
            print(f"{a.op} {name:8s} {M}x{N}x{Kd}: {ms * 1e3:9.1f} us  {2.0 * M * N * Kd / ms / 1e9:8.1f} TFLOP/s", flush=True)
    elif a.op == "dual":
        wshape = (shape.ffn, shape.hidden) if a.b_col_major else (shape.hidden, shape.ffn)
        A, Bg, Bu = (t.to(edt) for t in (rnd(a.m, shape.hidden), rnd(*wshape, std=0.02), rnd(*wshape, std=0.02)))
        out = torch.empty(a.m, shape.ffn, dtype=edt, device=DEV)
        Gs, Us = cold_copies(Bg, a.cold), cold_copies(Bu, a.cold)
        ms = timeit(lambda: K.dual_swiglu(A, next(Gs), next(Us), out=out, b_col_major=a.b_col_major), a.iters, a.warm)
        print(f"dual gate/up {'[N][K] weights ' if a.b_col_major else ''}{a.m}x{shape.ffn}x{shape.hidden}: {ms * 1e3:9.1f} us  "
              f"{4.0 * a.m * shape.ffn * shape.hidden / ms / 1e9:8.1f} TFLOP/s", flush=True)
    elif a.op == "dual_f8":
        M, N, Kd = a.m, shape.ffn, shape.hidden
        Aq = torch.randint(0, 120, (M, Kd), dtype=torch.uint8, device=DEV)
        Gq = torch.randint(0, 120, (N, Kd), dtype=torch.uint8, device=DEV)
        Uq = torch.randint(0, 120, (N, Kd), dtype=torch.uint8, device=DEV)
        sa, sg, su = torch.ones(M, device=DEV), torch.full((N,), 1e-4, device=DEV), torch.full((N,), 1e-4, device=DEV)
        out = torch.empty(M, N, dtype=torch.float16, device=DEV)
        Gqs, Uqs = cold_copies(Gq, a.cold), cold_copies(Uq, a.cold)
        ms = timeit(lambda: K.dual_swiglu_f8(Aq, sa, next(Gqs), sg, next(Uqs), su, out=out), a.iters, a.warm)
        print(f"dual_f8 gate/up {M}x{N}x{Kd}: {ms * 1e3:9.1f} us  {4.0 * M * N * Kd / ms / 1e9:8.1f} TFLOP/s", flush=True)
    elif a.op == "attn":
        b = synth.config2_batch(seed=0, n_decode=a.requests, lo=a.kv_lo, hi=a.kv_hi, prefill_chunk=16)
        nd = b.decodePrefillBorder
        pool = rnd(b.num_pages, 2, shape.page_size, shape.Hkv, shape.d)
        q = rnd(b.tokens, shape.Hq * shape.d)
        o = torch.zeros_like(q)
        t = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(DEV)
        qi, kvp, kvi, kvl = t(b.input_indptr[:nd + 1]), t(b.kv_indptr[:nd + 1]), t(b.kv_indices), t(b.kv_last_page_len[:nd])
        ws = torch.empty(1 << 20, dtype=torch.uint8, device=DEV)
        fn = lambda: K.attention_paged(q, qi, pool, kvp, kvi, kvl, shape.Hq, shape.Hkv, causal=False, out=o,
                                       batch=nd, max_qo_rows=nd, workspace=ws, num_blocks=a.num_blocks)
        ms = timeit(fn, a.iters, a.warm)
        L = b.kv_len[:nd].astype(np.int64)
        nbytes = int((2 * L * shape.Hkv * shape.d * 2 + 2 * shape.Hq * shape.d * 2 + 4 * ((L + 15) // 16 + 2)).sum())
        print(f"decode attention {nd} requests, KV [{a.kv_lo},{a.kv_hi}]: {ms * 1e3:9.1f} us  "
              f"{nbytes / ms / 1e6:8.1f} GB/s  ({nbytes} algorithmic bytes per launch)", flush=True)
    elif a.op == "prefill":
        chunks = [tuple(int(x) for x in c.split(":")) for c in a.chunks.split(",")]
        b = synth.make_batch([], chunks, vocab=shape.vocab, seed=0)
        pool = rnd(b.num_pages, 2, shape.page_size, shape.Hkv, shape.d)
        q = rnd(b.tokens, shape.Hq * shape.d)
        o = torch.zeros_like(q)
        t = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(DEV)
        qi, kvp, kvi, kvl = t(b.input_indptr), t(b.kv_indptr), t(b.kv_indices), t(b.kv_last_page_len)
        ws = torch.empty(1 << 20, dtype=torch.uint8, device=DEV)
        fn = lambda: K.attention_paged(q, qi, pool, kvp, kvi, kvl, shape.Hq, shape.Hkv, causal=True, out=o,
                                       batch=len(chunks), max_qo_rows=b.tokens, workspace=ws)
        ms = timeit(fn, a.iters, a.warm)
        flops = sum(l * (2 * (p + l) - l) * 2 * shape.Hq * shape.d for p, l in chunks)
        print(f"chunked-prefill attention {chunks}: {ms * 1e3:9.1f} us  {flops / ms / 1e9:8.1f} TFLOP/s "
              f"(causal flops of gemv/src/bench_batch_prefill.cu:133-134)", flush=True)
    elif a.op == "calibrate":
        for fp8 in (False, True):
            K.calibrate_mfma(fp8, True, 4000)
            for rand in (True, False):
                tf, mhz = K.calibrate_mfma(fp8, rand, 40000)
                print(f"mfma loop {'fp8 32x32x64' if fp8 else 'f16 32x32x16'} {'pseudo-random' if rand else 'zero':13s} operands: "
                      f"{tf:8.1f} TFLOP/s at {mhz:6.0f} MHz shader clock", flush=True)
            if fp8:
                tf, mhz = K.calibrate_mfma(True, 4, 40000)
                print(f"mfma loop fp8 16x16x128 pseudo-random operands (64 accumulators: the same register tile): "
                      f"{tf:8.1f} TFLOP/s at {mhz:6.0f} MHz shader clock", flush=True)
            if not fp8:
                tf, mhz = K.calibrate_mfma(False, 2, 40000)
                print(f"mfma loop f16 32x32x16 pseudo-random operands re-read from LDS every 16 MFMAs (8 x 16 B per lane): "
                      f"{tf:8.1f} TFLOP/s at {mhz:6.0f} MHz shader clock", flush=True)
                tf, mhz = K.calibrate_mfma(False, 3, 40000)
                print(f"   ... with 64 KB of operand loads per workgroup per 64 MFMAs (L2 -> LDS) beside them: "
                      f"{tf:8.1f} TFLOP/s at {mhz:6.0f} MHz shader clock", flush=True)
                tf, mhz = K.calibrate_mfma(False, 4, 40000)
                print(f"mfma loop f16 16x16x32 pseudo-random operands (64 accumulators: the same register tile): "
                      f"{tf:8.1f} TFLOP/s at {mhz:6.0f} MHz shader clock", flush=True)
        print(f"hbm read stream, 8 GiB x 4: {K.calibrate_hbm_read(8.0, 4):8.1f} GB/s", flush=True)
        b = synth.config2_batch(seed=0, n_decode=a.requests, lo=a.kv_lo, hi=a.kv_hi, prefill_chunk=16)
        nd = b.decodePrefillBorder
        pool = rnd(b.num_pages, 2, shape.page_size, shape.Hkv, shape.d)
        t = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(DEV)
        kvb = int(2 * b.kv_len[:nd].astype(np.int64).sum() * shape.Hkv * shape.d * 2)
        gbps = K.calibrate_paged_read(pool, t(b.kv_indptr[:nd + 1]), t(b.kv_indices), t(b.kv_last_page_len[:nd]), nd,
                                      shape.Hkv, kvb, 10)
        print(f"paged read without arithmetic, {nd} requests KV [{a.kv_lo},{a.kv_hi}]: {gbps:8.1f} GB/s", flush=True)
    elif a.op == "blas":
        shapes = layer_shapes(shape, a.m) + [("gate/up (2 GEMMs)", a.m, shape.ffn, shape.hidden)]
        for name, M, N, Kd in shapes:
            A = rnd(M, Kd)
            Bkn, Bnk = rnd(Kd, N, std=0.02), rnd(N, Kd, std=0.02)
            out = torch.empty(M, N, dtype=torch.float16, device=DEV)
            reps = 2 if name.startswith("gate") else 1
            # every measurement follows --warm-ms of the same launches: all are timed warm; with --cold
            # every launch (each of the two gate/up GEMMs too) takes the next of 1 GiB of weight copies
            kn, nk = cold_copies(Bkn, a.cold), cold_copies(Bnk, a.cold)
            ms_kn = timeit(lambda: [torch.matmul(A, next(kn), out=out) for _ in range(reps)], a.iters, a.warm)
            ms_nk = timeit(lambda: [torch.matmul(A, next(nk).t(), out=out) for _ in range(reps)], a.iters, a.warm)
            # this library as the pipelines call it (workspace entry points: the down projection at 2048
            # rows is split over K), on both weight layouts
            ws = torch.empty(max(K.lib().nf_gemm_workspace_bytes(M, N, Kd), 16), dtype=torch.uint8, device=DEV)
            if name.startswith("gate"):
                kn2, nk2 = cold_copies(rnd(Kd, N, std=0.02), a.cold), cold_copies(rnd(N, Kd, std=0.02), a.cold)
                ms_us = timeit(lambda: K.dual_swiglu(A, next(kn), next(kn2), out=out), a.iters, a.warm)
                ms_us_nk = timeit(lambda: K.dual_swiglu(A, next(nk), next(nk2), out=out, b_col_major=True), a.iters, a.warm)
                ms_same = timeit(lambda: K.dual_swiglu(A, Bnk, Bnk, out=out, b_col_major=True), a.iters, a.warm)
            else:
                ms_us = timeit(lambda: K.gemm_ws(A, next(kn), out=out, workspace=ws), a.iters, a.warm)
                ms_us_nk = timeit(lambda: K.gemm_ws(A, next(nk), out=out, workspace=ws, b_col_major=True), a.iters, a.warm)
            fl = 2.0 * reps * M * N * Kd
            print(f"{name:18s} {M}x{N}x{Kd}: torch.matmul [K,N] weights {fl / ms_kn / 1e9:7.1f}  [N,K] weights "
                  f"{fl / ms_nk / 1e9:7.1f}  this library [K,N] {fl / ms_us / 1e9:7.1f}  [N,K] {fl / ms_us_nk / 1e9:7.1f} TFLOP/s", flush=True)
            if name.startswith("gate"):
                print(f"{'':18s} this library's fused pair, [N,K], with ONE buffer given as both weight matrices (half the weight "
                      f"bytes, same flops): {fl / ms_same / 1e9:7.1f} TFLOP/s", flush=True)
    elif a.op in ("corun", "cusplit"):
        corun(a, shape, rnd)
    else:
        n = a.mib << 20
        src = torch.empty(n, dtype=torch.uint8, device=DEV).random_(generator=g)
        dst = torch.empty_like(src)
        ms = timeit(lambda: dst.copy_(src), a.iters, a.warm)
        print(f"copy {a.mib} MiB: {ms * 1e3:9.1f} us  {2 * n / ms / 1e6:8.1f} GB/s (read + write; "
              f"{n} bytes read, {n} bytes written per launch)", flush=True)


if __name__ == "__main__":
    main()
