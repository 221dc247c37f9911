"""A8W8 GEMM sweep over the shapes of the reference's benchmark/benchmark_gemm_a8w8_amd.py:
20 (N, K) pairs of sharded decoder models x 10 activation row counts, int8 operands drawn like the
reference draws them (randint(-128, 127), fp16 scales from rand), fp16 output, a rotation of operand
sets adding up to 512 MB so that no call finds its operands in a cache (:12-16, :57-71).

    python -m flashnn_amd.benchmarks.gemm_a8w8_amd [--m 1 2048] [--limit-shapes 4] [--json out.json]
                                                   [--same-operands] [--provider torch]

--same-operands times every call on one operand set, which is what the reference's other sweep,
benchmark/benchmark_gemm_a8w8.py:49-73, does over the same shapes (operands then stay in the caches where
they fit); --provider torch times the operator's torch path (its "torch" line, :66-73).

Prints one line per (N, K, M): median microseconds and TOPS at the median / 20 % / 80 % quantile
(the reference's "TFLOPS" column is 2*M*N*K / time as well)."""
import argparse
import json

import torch

import flashnn_amd
from flashnn_amd import workloads
from flashnn_amd.benchmarks._timing import bench_calls

ROTATION_BYTES = 512 * 1024 * 1024


def num_operand_sets(M, N, K):
    size = M * N + M * K + N * K + M + N
    return -(-ROTATION_BYTES // size)


def run_case(M, N, K, op, max_sets=64):
    n_sets = max(1, min(num_operand_sets(M, N, K), max_sets))
    g = torch.Generator(device="cuda").manual_seed(M * 1000003 + N * 101 + K)
    sets = []
    for _ in range(n_sets):
        sets.append((torch.randint(-128, 127, (M, K), dtype=torch.int8, device="cuda", generator=g),
                     torch.randint(-128, 127, (N, K), dtype=torch.int8, device="cuda", generator=g),
                     torch.rand(M, 1, device="cuda", generator=g).half(),
                     torch.rand(1, N, device="cuda", generator=g).half()))
    med, lo, hi = bench_calls(lambda i: op(*sets[i % n_sets]))
    tops = lambda ms: 2.0 * M * N * K / ms * 1e-9
    return {"M": M, "N": N, "K": K, "sets": n_sets, "us": med * 1e3, "tops": tops(med),
            "tops_q20": tops(lo), "tops_q80": tops(hi)}


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--m", type=int, nargs="*", default=workloads.SWEEP_M)
    ap.add_argument("--limit-shapes", type=int, default=0, help="only the first so many (N, K) pairs")
    ap.add_argument("--json", default=None)
    ap.add_argument("--same-operands", action="store_true", help="one operand set for every call (no rotation)")
    ap.add_argument("--provider", choices=["hip", "torch"], default="hip")
    args = ap.parse_args(argv)
    shapes = workloads.sharded_model_gemm_shapes()
    if args.limit_shapes:
        shapes = shapes[:args.limit_shapes]
    op = flashnn_amd.GemmA8W8(out_ty=torch.half)
    was = flashnn_amd.get_use_triton()
    flashnn_amd.set_use_triton(args.provider == "hip")
    rows = []
    print(f"{'N':>6} {'K':>6} {'M':>5} {'us':>9} {'TOPS':>8} {'q20':>8} {'q80':>8}", flush=True)
    for N, K in shapes:
        for M in args.m:
            r = run_case(M, N, K, op, max_sets=1 if args.same_operands else 64)
            rows.append(r)
            print(f"{N:6d} {K:6d} {M:5d} {r['us']:9.1f} {r['tops']:8.1f} {r['tops_q20']:8.1f} {r['tops_q80']:8.1f}",
                  flush=True)
            torch.cuda.empty_cache()
    flashnn_amd.set_use_triton(was)
    if args.json:
        with open(args.json, "w") as f:
            json.dump(rows, f, indent=1)
    return rows


if __name__ == "__main__":
    main()
