"""DynamicQuantize sweep over the shapes of the reference's benchmark/benchmark_dynamic_quant.py:
row lengths of sharded decoder models x 10 row counts, fp16 input from rand, every call timed with
the L2 flushed first (the reference times with triton.testing.do_bench, which does that; :28-38).

    python -m flashnn_amd.benchmarks.dynamic_quant [--m 1 2048] [--json out.json]

Prints median / 20 % / 80 % latency in microseconds and the bytes moved per second at the median
(2 bytes read and 1 written per element)."""
import argparse
import json

import torch

import flashnn_amd
from flashnn_amd import workloads
from flashnn_amd.benchmarks._timing import bench_calls


def run_case(M, K, op):
    g = torch.Generator(device="cuda").manual_seed(M * 1000003 + K)
    x = torch.rand(M, K, device="cuda", generator=g).half()
    med, lo, hi = bench_calls(lambda i: op(x), flush_bytes=256 * 1024 * 1024)
    return {"M": M, "K": K, "us": med * 1e3, "us_q20": lo * 1e3, "us_q80": hi * 1e3,
            "gbps": (3.0 * M * K + 2.0 * M) / med * 1e-6}


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--m", type=int, nargs="*", default=workloads.SWEEP_M)
    ap.add_argument("--json", default=None)
    args = ap.parse_args(argv)
    op = flashnn_amd.DynamicQuantize()
    rows = []
    print(f"{'K':>6} {'M':>5} {'us':>8} {'q20':>8} {'q80':>8} {'GB/s':>8}", flush=True)
    for K in workloads.DYNAMIC_QUANT_SWEEP_K:
        for M in args.m:
            r = run_case(M, K, op)
            rows.append(r)
            print(f"{K:6d} {M:5d} {r['us']:8.1f} {r['us_q20']:8.1f} {r['us_q80']:8.1f} {r['gbps']:8.0f}", flush=True)
    if args.json:
        with open(args.json, "w") as f:
            json.dump(rows, f, indent=1)
    return rows


if __name__ == "__main__":
    main()
