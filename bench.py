#!/usr/bin/env python3
"""Benchmark of the quantized-GEMM hot path on one MI355X.

Primary workload ("step"): per-token dynamic int8 quantisation of fp16 activations
[2048, 4096] followed by the A8W8 GEMM against int8 weights [12288, 4096] with the fused
per-token x per-channel scale epilogue writing bf16 (the Llama-7B QKV prefill shape).
`value` is 2*M*N*K / step time in TOPS with all inputs resident in HBM.

Also measured in the same run and reported in the same JSON line:
  roofline      the A8W8 GEMM kernel alone against the dense int8 MFMA peak, and under "a16w4_decode_m1" the
                second half of the metric: the A16W4 decode at M=1 against the 8 TB/s of HBM, on the
                reference's weight layout and on the packed form of GemmWeightOnly.prepack
  secondary     one entry per point of every configuration the path is quoted on, each against its bound:
                  c1     DynamicQuant + A8W8 at M=16 K=N=4096, fp16 out
                  c2     the four M=2048 prefill shapes (quant + GEMM, and the GEMM alone)
                  c3     A16W8 decode, M in {1, 8, 32} x three (K, N)
                  c4     A16W4 group-128 at K=8192 N=28672, M in {1, 4, 16, 64, 256} (M=1 always runs)
                  c5     RMSNormDquant -> A8W8 at K=N=8192, M in {1, 32, 512, 8192}
                  g64    A16W4 group-64 at the reference test's shape M=3 N=1024 K=4096
                  other  four shapes off the configured list whose kernel choice was settled by timing alternatives
                  splitk A8W8 shapes whose K the library splits, against the unsplit kernel
                  rows   the row kernels on their own;  moe  the fused mixture-of-experts GEMMs
  cpu_baseline  the reference's torch CPU path (oracle/torch_path.py) on the host cores

Inputs come from flashnn_amd/workloads.py (the configured distributions); int8 activations are produced by
the library's own quantisation of them.  Operand sets are rotated so that the working set exceeds the
256 MB Infinity Cache.  Kernel durations are HIP events recorded on the stream the kernels run on; the
kernel named in an entry is the one the library reports having launched (fnn_last_kernel).
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0     # MI355X dense int8 MFMA, published (5.0 POP/s)
PEAK_F16_TFLOPS = 2500.0    # dense bf16 / fp16 MFMA, published (2.5 PFLOP/s)
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E, published (8 TB/s)
ALL_LEGS = ("c1", "c2", "c3", "c4", "c5", "g64", "other", "splitk", "rows", "moe")


def _timed(fn, iters, torch, preroll_s=0.04):
    """(average milliseconds by HIP events on the current stream, average host wall milliseconds) of
    fn(i) over `iters` back-to-back calls.  An untimed pre-roll of the same call comes first and is in
    neither figure (its length in calls is kept in _timed.preroll_calls): host-side input generation between
    the measurements leaves the device idle long enough
    for its clocks to drop, and a hundred launches of a 20 us kernel would be over before they are back."""
    t0 = time.perf_counter()
    k = 0
    while time.perf_counter() - t0 < preroll_s:
        for _ in range(20):
            fn(k)
            k += 1
        torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    w0 = time.perf_counter()
    start.record()
    for i in range(iters):
        fn(i)
    end.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - w0) * 1e3 / iters
    _timed.preroll_calls = k
    return start.elapsed_time(end) / iters, wall


def _traffic(key):
    """HBM bytes per launch measured with rocprofv3 --pmc for the workload `key` (profiles/traffic.json:
    FETCH_SIZE and WRITE_SIZE readings scaled by what a plain copy of known size reads), or None."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        rec = json.load(f).get(key)
    return rec["bytes"] if rec else None


def _entry(workload, ms, bound, amount, kernels, traffic_key=None, **extra):
    """One secondary entry, kept short (the whole line has to fit the tail a harness keeps): w = workload,
    k = kernel as the library names it, us = microseconds per launch, bound = the roofline that applies
    ('hbm': 8000 GB/s; 'mfma': 5000 TOP/s int8; 'mfma16': 2500 TFLOP/s bf16/fp16), ach = achieved GB/s, TOP/s
    or TFLOP/s on the algorithmic bytes or operations of the call, frac = ach / peak, traffic = measured HBM
    bytes per launch where counted."""
    if bound == "hbm":
        achieved, peak = amount / (ms * 1e-3) / 1e9, PEAK_HBM_GBS
    else:
        achieved = amount / (ms * 1e-3) / 1e12
        peak = PEAK_INT8_TOPS if bound == "mfma" else PEAK_F16_TFLOPS
    e = {"w": workload, "k": kernels, "us": round(ms * 1e3, 2), "bound": bound, "ach": round(achieved, 1),
         "frac": round(achieved / peak, 3)}
    t = _traffic(traffic_key) if traffic_key else None
    if t is not None:
        e["traffic"] = t
    e.update(extra)
    return e


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="", help="comma list of secondary legs (%s, calib, none); default: all but calib"
                    % ", ".join(ALL_LEGS))
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (one MI355X per box); run with --gpus 1. "
                 "The configurations are per-GPU shapes: column-parallel layers shard N without any exchange, "
                 "row-parallel layers shard K and all-reduce the [M, N] partial results.")

    import torch

    import flashnn_amd
    from flashnn_amd import _lib, launchers, workloads

    lib = _lib.load()
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = "cuda:0"
    legs = set(args.only.split(",")) if args.only else set(ALL_LEGS)
    props = torch.cuda.get_device_properties(0)
    secondary = []
    iters = max(20, min(args.steps, 100))

    def kernel_of(fn):
        fn(0)
        return _lib.last_kernel()

    def rotating(t, total_bytes=300e6, at_least=2, at_most=64):
        """Copies of a device tensor, enough that one pass over them exceeds the Infinity Cache."""
        n = int(total_bytes // max(1, t.numel() * t.element_size())) + 1
        n = max(at_least, min(at_most, n))
        return [t] + [t.clone() for _ in range(n - 1)]

    if "calib" in legs:
        # a plain copy of known size: the counter readings of FETCH_SIZE / WRITE_SIZE for this
        # kernel give the scale factor that turns the readings of the other kernels into bytes
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    # --------------------------------------------- c2: A8W8 prefill, M = 2048 (qkv is the primary workload)
    M = 2048
    x_cpu = workloads.activations(M, 4096, torch.float16, seed=0, outlier_frac=0.01)
    primary = None
    w_qkv = ws_qkv = None
    for name, (K, N) in workloads.A8W8_PREFILL_SHAPES.items():
        if name != "qkv" and "c2" not in legs:
            continue
        x = x_cpu if K == 4096 else workloads.activations(M, K, torch.float16, seed=0, outlier_frac=0.01)
        w_cpu, wsc_cpu = workloads.int8_weights(N, K, seed=1)
        if name == "qkv":
            w_qkv, ws_qkv = w_cpu, wsc_cpu
        ws = rotating(w_cpu.to(dev), at_least=3)
        n = len(ws)
        xs = [x.to(dev).clone() for _ in range(n)]
        wscale = wsc_cpu.to(dev)
        qs = [torch.empty(M, K, dtype=torch.int8, device=dev) for _ in range(n)]
        ss = [torch.empty(M, dtype=torch.float16, device=dev) for _ in range(n)]
        outs = [torch.empty(M, N, dtype=torch.bfloat16, device=dev) for _ in range(n)]

        def quant_only(i):
            launchers.hip_dynamic_quantize(qs[i % n], xs[i % n], ss[i % n])

        def gemm_only(i):
            launchers.hip_gemm_a8w8_forward(outs[i % n], qs[i % n], ws[i % n], ss[i % n], wscale)

        def step(i):
            quant_only(i)
            gemm_only(i)

        ops = 2.0 * M * N * K
        k_quant, k_gemm = kernel_of(quant_only), kernel_of(gemm_only)
        if name == "qkv":
            # The device leaves its idle clocks only after some tens of milliseconds of work (measured:
            # 113 us per step right after 20 warm-up steps, 102 us from 200 warm-up steps on): whatever
            # --warmup says, the steps are preceded by an untimed pre-roll of the same step.
            for i in range(args.warmup):
                step(i)
            torch.cuda.synchronize()
            ms_step, wall_ms = _timed(step, args.steps, torch, preroll_s=0.06)
            preroll_steps = _timed.preroll_calls
            # the GEMM kernel's duration inside the step: the same steps once more (straight after the timed
            # ones, clocks as they were), with an event on either side of every GEMM launch.  The first event
            # completes when the quantisation kernel has, so the launch gap between the two kernels is inside.
            evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
            for i in range(args.steps):
                quant_only(i)
                evs[i][0].record()
                gemm_only(i)
                evs[i][1].record()
            torch.cuda.synchronize()
            ms_gemm = sum(a.elapsed_time(b) for a, b in evs) / args.steps
            ms_gemm_alone, _ = _timed(gemm_only, args.steps, torch)      # ... and launched back to back on its own
            ms_quant, _ = _timed(quant_only, args.steps, torch)
            primary = dict(M=M, K=K, N=N, ops=ops, ms_step=ms_step, wall_ms=wall_ms, ms_gemm=ms_gemm, nset=n,
                           ms_gemm_alone=ms_gemm_alone, preroll_steps=preroll_steps,
                           k_gemm=k_gemm, k_quant=k_quant)
            if "rows" in legs:
                secondary.append(_entry(f"dynamic_quant fp16 M={M} K={K}", ms_quant, "hbm", 3.0 * M * K + 2.0 * M,
                                        k_quant, "dynamic_quant M=2048 K=4096"))
        else:
            ms_step, _ = _timed(step, iters, torch)
            ms_gemm, _ = _timed(gemm_only, iters, torch)
            secondary.append(_entry(f"c2 a8w8 {name} M={M} K={K} N={N} bf16", ms_gemm, "mfma", ops, k_gemm,
                                    f"a8w8 {name}", us_with_quant=round(ms_step * 1e3, 2)))
        del ws, xs, qs, ss, outs
        torch.cuda.empty_cache()
    gemm_tops = primary["ops"] / (primary["ms_gemm"] * 1e-3) / 1e12
    roofline = {"kernel": primary["k_gemm"], "bound": "mfma", "achieved": round(gemm_tops, 2),
                "peak": PEAK_INT8_TOPS, "unit": "TOP/s", "frac": round(gemm_tops / PEAK_INT8_TOPS, 4),
                "us_per_launch": round(primary["ms_gemm"] * 1e3, 2), "traffic": _traffic("a8w8 qkv"),
                "timed": "events around every GEMM launch of the step loop (launch gap behind the quantisation included)",
                "us_per_launch_back_to_back": round(primary["ms_gemm_alone"] * 1e3, 2)}
    # what this device sustains on int8 MFMAs alone (operands in registers, about 0.1 s each): the
    # clock follows the power drawn, so random operand bytes run well below the datasheet rate
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    sustained = {}
    probe = ctypes.CDLL(os.path.join(ROOT, "flashnn_amd", "benchmarks", "libfnn_probe.so"))
    probe.fnn_probe_mfma_rate.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                          ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]
    for label, rnd in (("random_operand_bytes", 1), ("constant_operands", 0)):
        rate = ctypes.c_double(0.0)
        rc = probe.fnn_probe_mfma_rate(_lib.ptr(sink), rnd, 2000, 40, ctypes.byref(rate),
                                       _lib.current_stream(torch.device(dev)))
        if rc != 0:
            sys.exit(f"bench.py: the MFMA rate probe failed with hipError {rc}")
        sustained[label] = round(rate.value, 1)
    roofline["mfma_only_sustained"] = dict(sustained, unit="TOP/s")
    roofline["frac_of_sustained_random"] = round(gemm_tops / sustained["random_operand_bytes"], 4)
    # for scale: the int8 GEMM of the image's BLAS on the same shape (torch._int_mm: int32 output, no scale
    # epilogue), rotating operand sets like the step above
    try:
        Mq, Kq, Nq = primary["M"], primary["K"], primary["N"]
        gq = torch.Generator(device=dev).manual_seed(5)
        a_sets = [torch.randint(-128, 128, (Mq, Kq), dtype=torch.int8, device=dev, generator=gq) for _ in range(6)]
        b_sets = [torch.randint(-128, 128, (Nq, Kq), dtype=torch.int8, device=dev, generator=gq) for _ in range(6)]
        ms_blas, _ = _timed(lambda i: torch._int_mm(a_sets[i % 6], b_sets[i % 6].t()), args.steps, torch)
        roofline["blas_int8_gemm"] = {"fn": "torch._int_mm(a, b.t()), int32 out, no epilogue", "us": round(ms_blas * 1e3, 2),
                                      "TOPs": round(primary["ops"] / (ms_blas * 1e-3) / 1e12, 1)}
        del a_sets, b_sets
    except Exception as exc:          # (a torch build without the int8 GEMM: the figure is context, not part of the metric)
        roofline["blas_int8_gemm"] = {"fn": "torch._int_mm", "error": str(exc)[:80]}
    torch.cuda.empty_cache()
    # what the memory side delivers without arithmetic: the tile's copy pattern alone (direct-to-LDS copies of
    # 448 rows x 128 bytes per slab, one workgroup per CU, over the QKV operands' row length), and a stream of
    # the decode GEMV's request pattern over the bytes of its weights
    probe.fnn_probe_copy_rate.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                          ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]
    probe.fnn_probe_stream_rate.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p,
                                            ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]
    src = torch.randint(-128, 128, (1 << 29,), dtype=torch.int8, device=dev)     # 512 MiB
    rate = ctypes.c_double(0.0)
    rc = probe.fnn_probe_copy_rate(_lib.ptr(src), 200 << 20, 4096, 32, 2, 50, _lib.ptr(sink), ctypes.byref(rate),
                                   _lib.current_stream(torch.device(dev)))
    if rc != 0:
        sys.exit(f"bench.py: the copy rate probe failed with hipError {rc}")
    tile_bytes = (256 + 192) * 4096
    roofline["copy_only"] = {"GBps_per_cu": round(rate.value, 1), "pattern": "448 rows x 128 B per slab, direct to LDS, one workgroup per CU, rows shared within an XCD as in the kernel",
                             "kernel_GBps_per_cu": round(2 * tile_bytes / (primary["ms_gemm"] * 1e-3) / 1e9, 1)}
    a16w4_bytes = 28672 * 8192 // 2 + 4 * 64 * 28672
    rc = probe.fnn_probe_stream_rate(_lib.ptr(src), a16w4_bytes, 100, _lib.ptr(sink), ctypes.byref(rate),
                                     _lib.current_stream(torch.device(dev)))
    if rc != 0:
        sys.exit(f"bench.py: the stream rate probe failed with hipError {rc}")
    stream_hot = rate.value
    # ... and with the range moving through 500 MB, so that nothing is left in the caches from the launch before
    t_cold = []
    for rep in range(24):
        off = (rep % 4) * a16w4_bytes // 4096 * 4096
        rc = probe.fnn_probe_stream_rate(src.data_ptr() + off, a16w4_bytes, 1, _lib.ptr(sink), ctypes.byref(rate),
                                         _lib.current_stream(torch.device(dev)))
        if rc != 0:
            sys.exit(f"bench.py: the stream rate probe failed with hipError {rc}")
        t_cold.append(rate.value)
    t_cold.sort()
    roofline["stream_only"] = {"bytes": a16w4_bytes, "TBps_rotating": round(t_cold[len(t_cold) // 2], 2),
                               "TBps_same_range": round(stream_hot, 2),
                               "pattern": "9 non-temporal 16-byte loads per lane in flight, 8 waves per CU, launch gap included"}
    del src
    torch.cuda.empty_cache()

    # ------------------------------------------------------- c1: DynamicQuant + A8W8, M = 16, fp16 out
    x1_cpu = workloads.activations(16, 4096, torch.float16, seed=10)
    w1_cpu, ws1_cpu = workloads.int8_weights(4096, 4096, seed=11)
    if "c1" in legs:
        M1, K1, N1 = 16, 4096, 4096
        ws = rotating(w1_cpu.to(dev))
        n = len(ws)
        x1, wsc = x1_cpu.to(dev), ws1_cpu.to(dev)
        q1 = torch.empty(M1, K1, dtype=torch.int8, device=dev)
        s1 = torch.empty(M1, dtype=torch.float16, device=dev)
        o1 = torch.empty(M1, N1, dtype=torch.float16, device=dev)

        def gemm1(i):
            launchers.hip_gemm_a8w8_forward(o1, q1, ws[i % n], s1, wsc)

        def step1(i):
            launchers.hip_dynamic_quantize(q1, x1, s1)
            gemm1(i)

        kq = kernel_of(lambda i: launchers.hip_dynamic_quantize(q1, x1, s1))
        kg = kernel_of(gemm1)
        ms_s, _ = _timed(step1, iters, torch)
        ms_g, _ = _timed(gemm1, iters, torch)
        b1 = float(N1) * K1 + M1 * K1 + 2.0 * M1 * N1 + 2.0 * M1 + 4.0 * N1
        secondary.append(_entry(f"c1 a8w8 M={M1} K={K1} N={N1} fp16: GEMM", ms_g, "hbm", b1, kg,
                                us_quant_plus_gemm=round(ms_s * 1e3, 2), quant_kernel=kq))
        del ws
        torch.cuda.empty_cache()

    # ----------------------------------------------- c5: RMSNormDquant -> A8W8, K = N = 8192, bf16
    if "c5" in legs:
        K5 = N5 = 8192
        w5_cpu, ws5_cpu = workloads.int8_weights(N5, K5, seed=52)
        ws = rotating(w5_cpu.to(dev), at_least=4)
        n = len(ws)
        wsc = ws5_cpu.to(dev)
        norm = flashnn_amd.RMSNormDquant(K5, eps=1e-6).to(dev)
        norm.weight.data = workloads.rmsnorm_gamma(K5).to(dev)
        gemm5 = flashnn_amd.GemmA8W8(torch.bfloat16)
        for M5 in (1, 32, 512, 8192):
            h = workloads.activations(M5, K5, torch.bfloat16, seed=51, outlier_frac=0.01).to(dev)
            hs = rotating(h, total_bytes=300e6 if M5 >= 512 else 0, at_least=1, at_most=3)
            nh = len(hs)
            q5, s5 = norm(h)

            def chain(i):
                q, s = norm(hs[i % nh])
                gemm5(q, ws[i % n], s, wsc)

            def gemm_alone(i):
                gemm5(q5, ws[i % n], s5, wsc)

            kn = kernel_of(lambda i: norm(h))
            kg = kernel_of(gemm_alone)
            ms_c, _ = _timed(chain, iters if M5 < 8192 else 20, torch)
            ms_g, _ = _timed(gemm_alone, iters if M5 < 8192 else 20, torch)
            if M5 <= 32:
                amount, bound = float(N5) * K5 + M5 * K5 + 2.0 * M5 * N5 + 2.0 * M5 + 4.0 * N5, "hbm"
            else:
                amount, bound = 2.0 * M5 * N5 * K5, "mfma"
            secondary.append(_entry(f"c5 rmsnorm_dquant -> a8w8 M={M5} K={K5} N={N5} bf16: GEMM", ms_g, bound, amount,
                                    kg, f"a8w8 c5 M={M5}", us_norm_plus_gemm=round(ms_c * 1e3, 2), norm_kernel=kn))
            del hs
        del ws
        torch.cuda.empty_cache()

    # ------------------------------------------------- c4: A16W4 group 128, K = 8192, N = 28672, bf16
    K4, N4 = workloads.A16W4_SHAPE
    packed, scale4, zp4, _, _ = workloads.int4_group_weights(N4, K4, 128)
    # (M = 1 is the second half of the metric and always runs, on the reference layout and on the packed form)
    pk = rotating(packed.to(dev), total_bytes=500e6)
    n = len(pk)
    sc = [scale4.to(dev).clone() for _ in range(n)]
    zp = [zp4.to(dev).clone() for _ in range(n)]
    wbytes = N4 * K4 / 2 + 2 * (K4 // 128) * N4 * 2
    decode = {}
    for m4 in (1, 4, 16, 64, 256) if "c4" in legs else (1,):
        act = workloads.activations(m4, K4, torch.bfloat16, seed=3).to(dev)
        o4 = torch.empty(m4, N4, dtype=torch.bfloat16, device=dev)
        f = lambda i: launchers.hip_gemm_a16w4_forward(o4, act, pk[i % n], sc[i % n], None, zp[i % n])
        kern = kernel_of(f)
        ms, _ = _timed(f, iters, torch)
        extra = {"weight_GBps": round(wbytes / (ms * 1e-3) / 1e9, 1)}
        if m4 >= 64:      # also as a matrix-core workload
            extra["bf16_TFLOPs"] = round(2.0 * m4 * N4 * K4 / (ms * 1e-3) / 1e12, 1)
            extra["frac_of_bf16_peak"] = round(2.0 * m4 * N4 * K4 / (ms * 1e-3) / 1e12 / PEAK_F16_TFLOPS, 3)
        e = _entry(f"c4 a16w4 g128 M={m4} K={K4} N={N4} bf16", ms, "hbm", wbytes + 2.0 * m4 * K4 + 2.0 * m4 * N4,
                   kern, f"a16w4 g128 M={m4}", **extra)
        secondary.append(e)
        if m4 == 1:
            decode["reference_layout"] = e
    # the same decode on weights repacked once (GemmWeightOnly.prepack): the packed form holds exactly the
    # bytes of the reference layout (nibbles, fp16 scales, fp16 zero points), so the algorithmic bytes are
    # the bytes it reads
    packs = [launchers.hip_a16w4_prepack(pk[i], sc[i], zp[i]) for i in range(n)]
    act = workloads.activations(1, K4, torch.bfloat16, seed=3).to(dev)
    o4 = torch.empty(1, N4, dtype=torch.bfloat16, device=dev)
    f = lambda i: launchers.hip_gemm_a16w4_prepacked_forward(o4, act, packs[i % n])
    kern = kernel_of(f)
    ms, _ = _timed(f, max(iters, 100), torch)
    e = _entry(f"c4 a16w4 g128 M=1 K={K4} N={N4} bf16, weights prepacked", ms, "hbm", wbytes + 2.0 * K4 + 2.0 * N4, kern,
               "a16w4 g128 M=1 prepacked", weight_GBps=round(wbytes / (ms * 1e-3) / 1e9, 1),
               packed_bytes=int(packs[0].buffer.numel()))
    secondary.append(e)
    decode["prepacked"] = e
    if "c4" in legs:      # a few rows on the packed form (its kernel for 16, 32 or 64 rows per pass)
        for m4 in (4, 16, 64):
            act = workloads.activations(m4, K4, torch.bfloat16, seed=3).to(dev)
            o4 = torch.empty(m4, N4, dtype=torch.bfloat16, device=dev)
            f = lambda i: launchers.hip_gemm_a16w4_prepacked_forward(o4, act, packs[i % n])
            kern = kernel_of(f)
            ms, _ = _timed(f, iters, torch)
            secondary.append(_entry(f"c4 a16w4 g128 M={m4} K={K4} N={N4} bf16, weights prepacked", ms, "hbm",
                                    wbytes + 2.0 * m4 * K4 + 2.0 * m4 * N4, kern, f"a16w4 g128 M={m4} prepacked",
                                    weight_GBps=round(wbytes / (ms * 1e-3) / 1e9, 1)))
    del pk, sc, zp, packs
    torch.cuda.empty_cache()

    # ------------------------------------------------------------ c3: A16W8 decode, fp16, per-channel
    if "c3" in legs:
        for (K8, N8) in workloads.A16W8_DECODE_SHAPES:
            w8_cpu, s8_cpu = workloads.int8_weights(N8, K8, seed=40)
            w8 = rotating(w8_cpu.to(dev), total_bytes=600e6, at_least=3)
            n = len(w8)
            s8 = s8_cpu.half().to(dev)
            for m8 in (1, 8, 32):
                act = workloads.activations(m8, K8, torch.float16, seed=4).to(dev)
                o8 = torch.empty(m8, N8, dtype=torch.float16, device=dev)
                f = lambda i: launchers.hip_gemm_a16w8_forward(o8, act, w8[i % n], s8)
                kern = kernel_of(f)
                ms, _ = _timed(f, iters, torch)
                secondary.append(_entry(f"c3 a16w8 decode M={m8} K={K8} N={N8} fp16", ms, "hbm",
                                        N8 * K8 + 2.0 * N8 + 2.0 * m8 * K8 + 2.0 * m8 * N8, kern))
            del w8
        torch.cuda.empty_cache()

    # ----------- g64: the reference test's weight-only shape, M = 3, N = 1024, K = 4096, group 64, fp16, int8 and int4
    if "g64" in legs:
        Mg, Ng, Kg = 3, 1024, 4096
        gg = torch.Generator().manual_seed(64)
        act = workloads.activations(Mg, Kg, torch.float16, seed=65).to(dev)
        og = torch.empty(Mg, Ng, dtype=torch.float16, device=dev)
        for bits in (8, 4):
            if bits == 8:
                qg = torch.randint(-127, 128, (Ng, Kg), generator=gg, dtype=torch.int8)
                sg = torch.empty(Kg // 64, Ng).uniform_(1e-3, 1e-2, generator=gg).half()
                zg = torch.randint(-8, 9, (Kg // 64, Ng), generator=gg).half()
                fwd = launchers.hip_gemm_a16w8_forward
            else:
                qg, sg, zg, _, _ = workloads.int4_group_weights(Ng, Kg, 64, seed=64)
                fwd = launchers.hip_gemm_a16w4_forward
            qgs = rotating(qg.to(dev), at_most=160)
            n = len(qgs)
            sgs = [sg.to(dev).clone() for _ in range(n)]
            zgs = [zg.to(dev).clone() for _ in range(n)]
            f = lambda i: fwd(og, act, qgs[i % n], sgs[i % n], None, zgs[i % n])
            kern = kernel_of(f)
            ms, _ = _timed(f, iters, torch)
            secondary.append(_entry(f"g64 a16w{bits} group 64 M={Mg} K={Kg} N={Ng} fp16 (the reference test's shape)", ms,
                                    "hbm", Ng * Kg * bits / 8 + 4.0 * (Kg // 64) * Ng + 2.0 * Mg * Kg + 2.0 * Mg * Ng, kern))
            del qgs, sgs, zgs
        torch.cuda.empty_cache()

    # ----------- other: shapes off the configured list whose kernel choice was settled by timing it against forced alternatives
    if "other" in legs:
        # A8W8, 64 rows over 24576 channels (between one and two rounds of the few-row kernel's workgroups)
        Mo, No, Ko = 64, 24576, 8192
        xq = workloads.activations(Mo, Ko, torch.float16, seed=80, outlier_frac=0.01).to(dev)
        qo = torch.empty(Mo, Ko, dtype=torch.int8, device=dev)
        so = torch.empty(Mo, dtype=torch.float16, device=dev)
        launchers.hip_dynamic_quantize(qo, xq, so)
        wo_cpu, wos_cpu = workloads.int8_weights(No, Ko, seed=81)
        wo = rotating(wo_cpu.to(dev), total_bytes=600e6, at_least=3)
        n = len(wo)
        wos = wos_cpu.to(dev)
        oo = torch.empty(Mo, No, dtype=torch.bfloat16, device=dev)
        f = lambda i: launchers.hip_gemm_a8w8_forward(oo, qo, wo[i % n], so, wos)
        kern = kernel_of(f)
        ms, _ = _timed(f, iters, torch)
        secondary.append(_entry(f"other a8w8 M={Mo} K={Ko} N={No} bf16", ms, "hbm", float(No) * Ko + Mo * Ko + 2.0 * Mo * No, kern))
        # A16W8 per channel, 64 rows over 22016 channels (a little more than one round of 64-row workgroups)
        s8 = wos_cpu[:22016].half().to(dev)
        act = workloads.activations(64, 4096, torch.float16, seed=82).to(dev)
        o8 = torch.empty(64, 22016, dtype=torch.float16, device=dev)
        w8v = [w[:22016, :4096].contiguous() for w in wo]
        f = lambda i: launchers.hip_gemm_a16w8_forward(o8, act, w8v[i % n], s8)
        kern = kernel_of(f)
        ms, _ = _timed(f, iters, torch)
        secondary.append(_entry("other a16w8 M=64 K=4096 N=22016 fp16", ms, "hbm", 22016.0 * 4096 + 2.0 * 64 * (4096 + 22016), kern))
        del wo, w8v
        torch.cuda.empty_cache()
        # A16W4 g128, one row of 28672 values (beyond the decode kernels' LDS copy); groups of 64 at 64 rows
        for (Mv, Nv, Kv, gv) in ((1, 8192, 28672, 128), (64, 11008, 4096, 64)):
            qv, sv, zv, _, _ = workloads.int4_group_weights(Nv, Kv, gv, seed=83)
            qvs = rotating(qv.to(dev), total_bytes=600e6, at_least=3)
            n = len(qvs)
            svd, zvd = sv.to(dev), zv.to(dev)
            act = workloads.activations(Mv, Kv, torch.bfloat16, seed=84).to(dev)
            ov = torch.empty(Mv, Nv, dtype=torch.bfloat16, device=dev)
            f = lambda i: launchers.hip_gemm_a16w4_forward(ov, act, qvs[i % n], svd, None, zvd)
            kern = kernel_of(f)
            ms, _ = _timed(f, iters, torch)
            secondary.append(_entry(f"other a16w4 g{gv} M={Mv} K={Kv} N={Nv} bf16", ms, "hbm",
                                    Nv * Kv / 2.0 + 4.0 * (Kv // gv) * Nv + 2.0 * Mv * (Kv + Nv), kern))
            del qvs
        torch.cuda.empty_cache()

    # --------------------- splitk: A8W8 shapes whose K the library splits over workgroups, and the unsplit kernel
    if "splitk" in legs:
        for (Ms, Ns, Ks) in ((256, 4096, 8192), (128, 2048, 16384), (384, 1920, 13312)):
            xq = workloads.activations(Ms, Ks, torch.float16, seed=70, outlier_frac=0.01).to(dev)
            qs_ = torch.empty(Ms, Ks, dtype=torch.int8, device=dev)
            ss_ = torch.empty(Ms, dtype=torch.float16, device=dev)
            launchers.hip_dynamic_quantize(qs_, xq, ss_)
            wk_cpu, wks_cpu = workloads.int8_weights(Ns, Ks, seed=71)
            wk = rotating(wk_cpu.to(dev))
            n = len(wk)
            wks = wks_cpu.to(dev)
            ok = torch.empty(Ms, Ns, dtype=torch.bfloat16, device=dev)
            split = lambda i: launchers.hip_gemm_a8w8_forward(ok, qs_, wk[i % n], ss_, wks)
            st = _lib.current_stream(torch.device(dev))
            plain = lambda i: _lib.check(lib.fnn_gemm_a8w8(
                ok.data_ptr(), qs_.data_ptr(), wk[i % n].data_ptr(), ss_.data_ptr(), wks.data_ptr(), Ms, Ns, Ks, Ks, Ks, Ns,
                _lib.dtype_code(ok.dtype), _lib.dtype_code(ss_.dtype), _lib.dtype_code(wks.dtype), st))
            k_split, k_plain = kernel_of(split), kernel_of(plain)
            ms_split, _ = _timed(split, iters, torch)
            ms_plain, _ = _timed(plain, iters, torch)
            secondary.append(_entry(f"splitk a8w8 M={Ms} K={Ks} N={Ns} bf16", ms_split, "mfma", 2.0 * Ms * Ns * Ks, k_split,
                                    unsplit_us=round(ms_plain * 1e3, 2), unsplit_kernel=k_plain))
            del wk
        torch.cuda.empty_cache()

    # ------------------------------------------------------- rows: the row kernels on an 8192 x 8192 matrix
    if "rows" in legs:
        Mr, Kr = 8192, 8192
        hs = [workloads.activations(Mr, Kr, torch.bfloat16, seed=5, outlier_frac=0.01).to(dev) for _ in range(3)]
        norm = flashnn_amd.RMSNormDquant(Kr).to(dev)
        norm.weight.data = workloads.rmsnorm_gamma(Kr).to(dev)
        f = lambda i: norm(hs[i % 3])
        kern = kernel_of(f)
        ms, _ = _timed(f, 50, torch)
        secondary.append(_entry(f"rmsnorm_dquant bf16 M={Mr} K={Kr}", ms, "hbm", 3.0 * Mr * Kr + 4.0 * Kr + 2.0 * Mr, kern,
                                "rmsnorm_dquant M=8192 K=8192"))
        # the layers one step before the path, same matrix
        for name, mod, wr in (("rmsnorm", flashnn_amd.RMSNorm(Kr), 2.0), ("layernorm", flashnn_amd.LayerNorm(Kr), 2.0),
                              ("layernorm_dquant", flashnn_amd.LayernormDquant(Kr), 1.0)):
            mod = mod.to(torch.bfloat16).to(dev)
            f = lambda i: mod(hs[i % 3])
            kern = kernel_of(f)
            ms, _ = _timed(f, 50, torch)
            secondary.append(_entry(f"{name} bf16 M={Mr} K={Kr}", ms, "hbm", (2.0 + wr) * Mr * Kr, kern))
        del hs
        torch.cuda.empty_cache()

    # ------------------------------------------------ moe: mixture of experts (decode-sized batches)
    if "moe" in legs:
        E, Nm, Km, top_k, BMm = 8, 28672, 4096, 2, 16     # Mixtral-8x7B-like gate+up projection
        g = torch.Generator(device=dev).manual_seed(7)

        def routing(Mt):
            tw, tid = torch.topk(torch.softmax(torch.randn(Mt, E, generator=torch.Generator().manual_seed(8)), -1), top_k)
            sid, eid, used = workloads.moe_align_block_size(tid, BMm, E)
            active = len(set(tid.flatten().tolist()))
            return [t.to(dev) for t in (tw.float().contiguous(), tid, sid, eid, used)] + [active]

        bm = torch.randint(-127, 128, (E, Nm, Km), dtype=torch.int8, device=dev, generator=g)
        acm = torch.rand(E, Nm, device=dev, generator=g) * 9e-3 + 1e-3
        for Mt in (16, 64):
            xm = workloads.activations(Mt, Km, torch.float16, seed=72, outlier_frac=0.01).to(dev)
            am = torch.empty(Mt, Km, dtype=torch.int8, device=dev)
            arm = torch.empty(Mt, dtype=torch.float16, device=dev)
            launchers.hip_dynamic_quantize(am, xm, arm)
            tw, tid, sid, eid, used, active = routing(Mt)
            cm = torch.empty(Mt, top_k, Nm, dtype=torch.bfloat16, device=dev)
            f = lambda i: flashnn_amd.fused_moe_a8w8_forward(am, bm, cm, arm, acm, tw, tid, sid, eid, used, True, top_k, BMm)
            kern = kernel_of(f)
            ms, _ = _timed(f, 20, torch)
            secondary.append(_entry(f"fused_moe_a8w8 tokens={Mt} E={E} top_k={top_k} K={Km} N={Nm} block={BMm} "
                                    f"({active} experts in use)", ms, "hbm",
                                    float(active) * Nm * Km + 2.0 * Mt * top_k * Nm, kern))
        # a prompt's worth of tokens: the MFMA tiles over the sorted rows (one tile height per block size)
        Mt = 4096
        xm = workloads.activations(Mt, Km, torch.float16, seed=74, outlier_frac=0.01).to(dev)
        am = torch.empty(Mt, Km, dtype=torch.int8, device=dev)
        arm = torch.empty(Mt, dtype=torch.float16, device=dev)
        launchers.hip_dynamic_quantize(am, xm, arm)
        cm = torch.empty(Mt, top_k, Nm, dtype=torch.bfloat16, device=dev)
        tw, tid = torch.topk(torch.softmax(torch.randn(Mt, E, generator=torch.Generator().manual_seed(8)), -1), top_k)
        for blk in (64, 128, 256):
            sid, eid, used = workloads.moe_align_block_size(tid, blk, E)
            rows_padded = int(used[0])
            twd, tidd, sid, eid, used = [t.to(dev) for t in (tw.float().contiguous(), tid, sid, eid, used)]
            f = lambda i: flashnn_amd.fused_moe_a8w8_forward(am, bm, cm, arm, acm, twd, tidd, sid, eid, used, True, top_k, blk)
            kern = kernel_of(f)
            ms, _ = _timed(f, 10, torch)
            secondary.append(_entry(f"fused_moe_a8w8 tokens={Mt} E={E} top_k={top_k} K={Km} N={Nm} block={blk} "
                                    f"({rows_padded} sorted rows)", ms, "mfma", 2.0 * Mt * top_k * Nm * Km, kern,
                                    f"moe a8w8 {Mt} tokens block {blk}"))
        del bm
        torch.cuda.empty_cache()
        # int4 expert weights of the same layer: per-channel tables, then tables per group of 128 ([E, N, K/128])
        N2 = Nm // 2
        b4 = torch.randint(-128, 128, (E, N2, Km), dtype=torch.int8, device=dev, generator=g)
        for label, tshape, Mts in (("per-channel", (E, Nm), (16, 64)), ("group 128", (E, Nm, Km // 128), (16,))):
            sc4 = (torch.rand(*tshape, device=dev, generator=g) * 9e-3 + 1e-3).to(torch.bfloat16)
            zp4m = torch.randint(-3, 4, tshape, device=dev, generator=g).to(torch.bfloat16)
            for Mt in Mts:
                a4 = workloads.activations(Mt, Km, torch.bfloat16, seed=73).to(dev)
                tw, tid, sid, eid, used, active = routing(Mt)
                cm = torch.empty(Mt, top_k, Nm, dtype=torch.bfloat16, device=dev)
                f = lambda i: flashnn_amd.fused_moe_a16w4_forward(a4, b4, cm, sc4, zp4m, tw, tid, sid, eid, used, True,
                                                                  top_k, BMm)
                kern = kernel_of(f)
                ms, _ = _timed(f, 20, torch)
                tables = 4.0 * Nm * (Km // 128) if len(tshape) == 3 else 4.0 * Nm
                secondary.append(_entry(f"fused_moe_a16w4 {label} tokens={Mt} E={E} top_k={top_k} K={Km} N={Nm} "
                                        f"block={BMm} ({active} experts in use)", ms, "hbm",
                                        float(active) * (N2 * Km + tables) + 2.0 * Mt * top_k * Nm, kern))
        # a prompt's worth of tokens, per-channel tables: the tiled MFMA kernel over the sorted rows
        sc4 = (torch.rand(E, Nm, device=dev, generator=g) * 9e-3 + 1e-3).to(torch.bfloat16)
        zp4m = torch.randint(-3, 4, (E, Nm), device=dev, generator=g).to(torch.bfloat16)
        Mt = 4096
        a4 = workloads.activations(Mt, Km, torch.bfloat16, seed=75).to(dev)
        cm = torch.empty(Mt, top_k, Nm, dtype=torch.bfloat16, device=dev)
        tw, tid = torch.topk(torch.softmax(torch.randn(Mt, E, generator=torch.Generator().manual_seed(8)), -1), top_k)
        for blk in (64, 256):
            sid, eid, used = workloads.moe_align_block_size(tid, blk, E)
            rows_padded = int(used[0])
            twd, tidd, sid, eid, used = [t.to(dev) for t in (tw.float().contiguous(), tid, sid, eid, used)]
            f = lambda i: flashnn_amd.fused_moe_a16w4_forward(a4, b4, cm, sc4, zp4m, twd, tidd, sid, eid, used, True,
                                                              top_k, blk)
            kern = kernel_of(f)
            ms, _ = _timed(f, 5, torch)
            secondary.append(_entry(f"fused_moe_a16w4 per-channel tokens={Mt} E={E} top_k={top_k} K={Km} N={Nm} block={blk} "
                                    f"({rows_padded} sorted rows)", ms, "mfma16", 2.0 * Mt * top_k * Nm * Km, kern,
                                    f"moe a16w4 {Mt} tokens block {blk}"))
        # ... and tables per group of 128 in the launcher's [E, N, K/128] layout (128-row tiles, fp32 scaling per slab)
        sc4 = (torch.rand(E, Nm, Km // 128, device=dev, generator=g) * 9e-3 + 1e-3).to(torch.bfloat16)
        zp4m = torch.randint(-3, 4, (E, Nm, Km // 128), device=dev, generator=g).to(torch.bfloat16)
        sid, eid, used = workloads.moe_align_block_size(tid, 128, E)
        rows_padded = int(used[0])
        twd, tidd, sid, eid, used = [t.to(dev) for t in (tw.float().contiguous(), tid, sid, eid, used)]
        f = lambda i: flashnn_amd.fused_moe_a16w4_forward(a4, b4, cm, sc4, zp4m, twd, tidd, sid, eid, used, True, top_k, 128)
        kern = kernel_of(f)
        ms, _ = _timed(f, 5, torch)
        secondary.append(_entry(f"fused_moe_a16w4 group 128 tokens={Mt} E={E} top_k={top_k} K={Km} N={Nm} block=128 "
                                f"({rows_padded} sorted rows)", ms, "mfma16", 2.0 * Mt * top_k * Nm * Km, kern))
        del b4
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ CPU baseline
    cpu_baseline = None
    if not args.no_cpu:
        from oracle import torch_path as T
        cores = torch.get_num_threads()
        Mq, Kq, Nq = primary["M"], primary["K"], primary["N"]

        def cpu_step():
            q, s = T.dynamic_quantize(x_cpu)
            return T.gemm_a8w8(q, w_qkv, s.float(), ws_qkv, torch.bfloat16)

        cpu_step()
        ts = []
        for _ in range(3):
            t0 = time.perf_counter()
            cpu_step()
            ts.append(time.perf_counter() - t0)
        t_cpu = sorted(ts)[1]
        act1 = workloads.activations(1, K4, torch.bfloat16, seed=3)
        t0 = time.perf_counter()
        T.gemm_weight_only(act1, packed, scale4, None, zp4, torch.bfloat16)
        t_cpu4 = time.perf_counter() - t0
        # the reference's own CPU-runnable case (c1)
        t0 = time.perf_counter()
        for _ in range(5):
            q, s = T.dynamic_quantize(x1_cpu)
            T.gemm_a8w8(q, w1_cpu, s.float(), ws1_cpu, torch.float16)
        t_cpu1 = (time.perf_counter() - t0) / 5
        cpu_baseline = {"value": round(primary["ops"] / t_cpu / 1e12, 4), "unit": "TOPS", "cores": cores, "kind": "port",
                        "sample": f"the whole step (dynamic quant + fp32-matmul A8W8, M={Mq} K={Kq} N={Nq}) through "
                                  f"the torch-op restatement of the reference's CPU path, median of 3 runs "
                                  f"({t_cpu * 1e3:.0f} ms each)",
                        "c1_m16_ms": round(t_cpu1 * 1e3, 2),
                        "a16w4_decode_m1_ms": round(t_cpu4 * 1e3, 1),
                        "a16w4_decode_m1_weight_GBps": round((N4 * K4 / 2 + 4 * (K4 // 128) * N4) / t_cpu4 / 1e9, 3)}

    # the second half of the metric, beside the first: A16W4 decode at M = 1 against the 8 TB/s of HBM3E, on
    # the layout the reference's operator takes and on the packed form (bytes actually read = algorithmic bytes)
    roofline["a16w4_decode_m1"] = {
        name: {"kernel": e["k"], "bound": "hbm", "us_per_launch": e["us"], "achieved": e["ach"], "peak": PEAK_HBM_GBS,
               "unit": "GB/s", "frac": e["frac"], "traffic": e.get("traffic")}
        for name, e in decode.items()}
    value = primary["ops"] / (primary["ms_step"] * 1e-3) / 1e12
    result = {
        "metric": "a8w8_int8_tops_m2048", "value": round(value, 2), "unit": "TOPS", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "preroll_steps": primary["preroll_steps"], "ms_per_step": round(primary["ms_step"], 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "DynamicQuant(fp16 [2048,4096], 1% outlier channels x20) + A8W8 GEMM "
                               "M=2048 K=4096 N=12288, int8 per-channel weights, bf16 out (Llama-7B QKV prefill)",
                   "kernels": [primary["k_quant"], primary["k_gemm"]],
                   "rotating_operand_sets": primary["nset"], "device": props.name, "cus": props.multi_processor_count,
                   "host_wall_ms_per_step": round(primary["wall_ms"], 5)},
        "roofline": roofline, "cpu_baseline": cpu_baseline, "secondary": secondary,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
