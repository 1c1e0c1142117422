#!/usr/bin/env python3
"""Writes a request trace for nanoflow_amd.serve: a header line, then ``idx,input_len,output_len,arrival``.

    python -m nanoflow_amd.gen_req --input_len 1024 --output_len 512 --rate 0 -n 4096 -o offline.csv
    python -m nanoflow_amd.gen_req --input_len 1024 --output_len 512 --rate 15 --poisson -n 700 -o online15.csv

Counterpart of the reference's pipeline/utils/gen_req.py (a fixed prompt repeated at a constant
interval, 1 / request_rate, 0 meaning "all at time 0") and of the constant-length traces of its
offline evaluation (pipeline/eval/eval-fix-offline/gen_const_len_req.py: rows ``i,1024,512,0``).
Here a row carries token counts instead of prompt text (no tokenizer ships with this package), the
lengths may be drawn uniformly from a range (``--input_len 200:700``), and ``--poisson`` draws
exponential gaps with the same mean instead of the constant interval.
"""
from __future__ import annotations

import argparse

import numpy as np


def _length(spec: str, rng, n):
    if ":" in spec:
        lo, hi = (int(x) for x in spec.split(":"))
        return rng.integers(lo, hi + 1, size=n)
    return np.full(n, int(spec))


def write_trace(path, n, input_len="1024", output_len="512", rate=0.0, poisson=False, seed=0):
    rng = np.random.default_rng(seed)
    n_in, n_out = _length(str(input_len), rng, n), _length(str(output_len), rng, n)
    if rate <= 0:
        arrival = np.zeros(n)
    elif poisson:
        arrival = np.cumsum(rng.exponential(1.0 / rate, size=n))
    else:
        arrival = np.arange(n) / rate
    with open(path, "w") as f:
        f.write("idx,input_len,output_len,arrival\n")
        for i in range(n):
            f.write(f"{i},{int(n_in[i])},{int(n_out[i])},{arrival[i]:.6f}\n")
    return path


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("-o", "--output", required=True)
    ap.add_argument("-n", "--requests", type=int, default=4096)
    ap.add_argument("--input_len", default="1024", help="tokens, or lo:hi for a uniform draw")
    ap.add_argument("--output_len", default="512", help="tokens, or lo:hi for a uniform draw")
    ap.add_argument("--rate", type=float, default=0.0, help="requests per second; 0 = all at time 0")
    ap.add_argument("--poisson", action="store_true", help="exponential gaps instead of a constant interval")
    ap.add_argument("--seed", type=int, default=0)
    a = ap.parse_args()
    write_trace(a.output, a.requests, a.input_len, a.output_len, a.rate, a.poisson, a.seed)
    print(f"{a.requests} requests -> {a.output}")


if __name__ == "__main__":
    main()
