"""Per-call GPU timing in the style of triton.testing.do_bench, which the reference's benchmark
scripts use: warm up, then bracket every call with its own pair of events and report quantiles."""
import torch


def _quantiles(times_ms, qs):
    t = torch.tensor(sorted(times_ms), dtype=torch.float64)
    return [float(torch.quantile(t, q)) for q in qs]


def bench_calls(fn, rep_ms=100.0, warmup_ms=25.0, quantiles=(0.5, 0.2, 0.8), flush_bytes=0, max_reps=2000):
    """Times fn(i) for i = 0, 1, ... and returns the requested quantiles in milliseconds.

    `flush_bytes` > 0 overwrites a buffer of that size before every timed call, outside the timed
    bracket, so that the call starts with none of its operands in the L2 (do_bench does the same
    with 256 MB); callers that rotate through operand sets larger than the caches pass 0."""
    flush = torch.empty(flush_bytes, dtype=torch.int8, device="cuda") if flush_bytes else None
    fn(0)
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for i in range(5):
        fn(i)
    e.record()
    torch.cuda.synchronize()
    est = max(s.elapsed_time(e) / 5, 1e-3)
    n_warm = max(1, min(max_reps, int(warmup_ms / est)))
    n_rep = max(5, min(max_reps, int(rep_ms / est)))
    for i in range(n_warm):
        fn(i)
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_rep)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_rep)]
    for i in range(n_rep):
        if flush is not None:
            flush.zero_()
        starts[i].record()
        fn(i)
        ends[i].record()
    torch.cuda.synchronize()
    return _quantiles([a.elapsed_time(b) for a, b in zip(starts, ends)], quantiles)
