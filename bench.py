#!/usr/bin/env python3
"""Benchmark of the quantized-GEMM hot path on one MI355X.

Primary workload ("step"): per-token dynamic int8 quantisation of fp16 activations
[2048, 4096] followed by the A8W8 GEMM against int8 weights [12288, 4096] with the fused
per-token x per-channel scale epilogue writing bf16 (the Llama-7B QKV prefill shape).
`value` is 2*M*N*K / step time in TOPS with all inputs resident in HBM.

Also measured in the same run and reported in the same JSON line:
  roofline          the A8W8 GEMM kernel alone against the dense int8 MFMA peak
  secondary         the other configurations: the remaining prefill shapes, A16W4 group-128 at
                    M = 1 .. 256 (M=1 is the decode GEMV of the second headline metric), A8W8 with
                    few activation rows, A16W8 decode and the row kernels, each against its bound
  cpu_baseline      the reference's torch CPU path (oracle/torch_path.py) on the host cores

Operand sets are rotated so that the working set exceeds the 256 MB Infinity Cache; kernel
durations come from HIP events recorded on the stream the kernels run on.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0     # MI355X dense int8 MFMA, published (5.0 POP/s)
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E, published (8 TB/s)


def _events_ms(fn, iters, torch, preroll_s=0.04):
    """Average duration of fn() over `iters` back-to-back calls, HIP events on the current stream.
    The calls are preceded by an untimed pre-roll of the same call: host-side input generation between the
    measurements leaves the device idle long enough for its clocks to drop, and a hundred launches of a
    20 us kernel would otherwise be over before they have come back."""
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
    start.record()
    for i in range(iters):
        fn(i)
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters


def _traffic(kernel):
    """HBM bytes per launch measured with rocprofv3 --pmc (profiles/traffic.json), or None."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        return json.load(f).get(kernel)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="", help="comma list of legs: a8w8,a16w4,rows,moe,calib (default: all but calib)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (one MI355X per box); run with --gpus 1. "
                 "The configurations are per-GPU shapes: column-parallel layers shard N without any exchange, "
                 "row-parallel layers shard K and all-reduce the [M, N] partial results.")

    import torch

    import flashnn_amd
    from flashnn_amd import _lib, launchers, workloads

    _lib.load()
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = "cuda:0"
    legs = set(args.only.split(",")) if args.only else {"a8w8", "a16w4", "rows", "moe"}
    props = torch.cuda.get_device_properties(0)
    result = {}

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

    # ------------------------------------------------------------------ primary: A8W8
    M, K, N = 2048, 4096, 12288
    x_cpu = workloads.activations(M, K, torch.float16, seed=0, outlier_frac=0.01)
    w_cpu, ws_cpu = workloads.int8_weights(N, K, seed=1)
    nset = 4   # 4 x (8 + 50 + 50 + 17) MB > 256 MB
    xs = [x_cpu.to(dev).clone() for _ in range(nset)]
    ws = [w_cpu.to(dev).clone() for _ in range(nset)]
    wscale = ws_cpu.to(dev)
    qs = [torch.empty(M, K, dtype=torch.int8, device=dev) for _ in range(nset)]
    ss = [torch.empty(M, dtype=torch.float16, device=dev) for _ in range(nset)]
    outs = [torch.empty(M, N, dtype=torch.bfloat16, device=dev) for _ in range(nset)]

    def step(i):
        j = i % nset
        launchers.hip_dynamic_quantize(qs[j], xs[j], ss[j])
        launchers.hip_gemm_a8w8_forward(outs[j], qs[j], ws[j], ss[j], wscale)

    def gemm_only(i):
        j = i % nset
        launchers.hip_gemm_a8w8_forward(outs[j], qs[j], ws[j], ss[j], wscale)

    def quant_only(i):
        j = i % nset
        launchers.hip_dynamic_quantize(qs[j], xs[j], ss[j])

    # The device leaves its idle clocks only after some tens of milliseconds of work (measured: 113 us per
    # step right after 20 warm-up steps, 102 us from 200 warm-up steps on), so whatever --warmup says the
    # steps are preceded by an untimed pre-roll of about 60 ms of the same step.
    preroll_steps = 0
    t_pre = time.perf_counter()
    while time.perf_counter() - t_pre < 0.06:
        for i in range(50):
            step(i)
        torch.cuda.synchronize()
        preroll_steps += 50
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ms_step = _events_ms(step, args.steps, torch)
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ops = 2.0 * M * N * K
    value = ops / (ms_step * 1e-3) / 1e12
    ms_gemm = _events_ms(gemm_only, args.steps, torch)
    ms_quant = _events_ms(quant_only, args.steps, torch)
    gemm_tops = ops / (ms_gemm * 1e-3) / 1e12
    roofline = {"kernel": "gemm_a8w8_ring_kernel", "bound": "mfma", "achieved": round(gemm_tops, 2),
                "peak": PEAK_INT8_TOPS, "unit": "TOP/s", "frac": round(gemm_tops / PEAK_INT8_TOPS, 4),
                "us_per_launch": round(ms_gemm * 1e3, 2), "traffic": _traffic("gemm_a8w8_ring_kernel")}
    # what this device sustains on int8 MFMAs alone (operands in registers, about 0.1 s each): the
    # clock follows the power drawn, so random operand bytes run well below the datasheet rate
    import ctypes
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
    secondary = []
    qbytes = 3.0 * M * K + 2.0 * M
    secondary.append({"workload": f"dynamic_quant fp16 M={M} K={K}", "kernel": "dynamic_quant_vec_kernel",
                      "us_per_launch": round(ms_quant * 1e3, 2),
                      "roofline": {"bound": "hbm", "achieved": round(qbytes / (ms_quant * 1e-3) / 1e9, 1),
                                   "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                   "frac": round(qbytes / (ms_quant * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                                   "traffic": _traffic("dynamic_quant_vec_kernel")}})
    del xs, ws, outs
    torch.cuda.empty_cache()

    # other prefill shapes (reported)
    if "a8w8" in legs:
        for name, (k2, n2) in workloads.A8W8_PREFILL_SHAPES.items():
            if name == "qkv":
                continue
            a2 = [torch.randint(-127, 128, (M, k2), dtype=torch.int8, device=dev) for _ in range(3)]
            b2 = [torch.randint(-127, 128, (n2, k2), dtype=torch.int8, device=dev) for _ in range(3)]
            o2 = [torch.empty(M, n2, dtype=torch.bfloat16, device=dev) for _ in range(3)]
            s2 = torch.rand(M, device=dev).half()
            c2 = torch.rand(n2, device=dev)
            f = lambda i: launchers.hip_gemm_a8w8_forward(o2[i % 3], a2[i % 3], b2[i % 3], s2, c2)
            for i in range(5):
                f(i)
            ms = _events_ms(f, 50, torch)
            t = 2.0 * M * n2 * k2 / (ms * 1e-3) / 1e12
            secondary.append({"workload": f"a8w8 {name} M={M} K={k2} N={n2} bf16", "kernel": "gemm_a8w8_ring_kernel",
                              "us_per_launch": round(ms * 1e3, 2),
                              "roofline": {"bound": "mfma", "achieved": round(t, 2), "peak": PEAK_INT8_TOPS,
                                           "unit": "TOP/s", "frac": round(t / PEAK_INT8_TOPS, 4), "traffic": None}})
            del a2, b2, o2
        torch.cuda.empty_cache()

    # -------------------------------------------------------------- A16W4 decode GEMV
    K4, N4 = workloads.A16W4_SHAPE
    packed, scale4, zp4, _, _ = workloads.int4_group_weights(N4, K4, 128)
    if "a16w4" in legs:
        nset4 = 5   # 5 x 125 MB
        pk = [packed.to(dev).clone() for _ in range(nset4)]
        sc = [scale4.to(dev).clone() for _ in range(nset4)]
        zp = [zp4.to(dev).clone() for _ in range(nset4)]
        for m4 in (1, 4, 16, 64, 256):
            act = workloads.activations(m4, K4, torch.bfloat16, seed=3).to(dev)
            o4 = torch.empty(m4, N4, dtype=torch.bfloat16, device=dev)
            f = lambda i: launchers.hip_gemm_a16w4_forward(o4, act, pk[i % nset4], sc[i % nset4], None, zp[i % nset4])
            for i in range(10):
                f(i)
            ms = _events_ms(f, 100, torch)
            wbytes = N4 * K4 / 2 + 2 * (K4 // 128) * N4 * 2
            allbytes = wbytes + 2.0 * m4 * K4 + 2.0 * m4 * N4
            gbs = allbytes / (ms * 1e-3) / 1e9
            secondary.append({"workload": f"a16w4 g128 decode M={m4} K={K4} N={N4} bf16",
                              "kernel": "gemm_wo_gemv_kernel" if m4 <= 4 else "gemm_wo_panel_kernel", "us_per_launch": round(ms * 1e3, 2),
                              "weight_GBps": round(wbytes / (ms * 1e-3) / 1e9, 1),
                              "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
                                           "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4),
                                           "traffic": _traffic("gemm_wo_gemv_kernel") if m4 == 1 else None}})
        del pk, sc, zp
        torch.cuda.empty_cache()

    # ------------------------------------- few activation rows: RMSNorm+quant -> A8W8, K = N = 8192
    if "a8w8" in legs:
        k5 = n5 = 8192
        w5 = [torch.randint(-127, 128, (n5, k5), dtype=torch.int8, device=dev) for _ in range(5)]
        c5 = torch.rand(n5, device=dev) * 0.01
        for m5 in (1, 32):
            a5 = torch.randint(-127, 128, (m5, k5), dtype=torch.int8, device=dev)
            s5 = torch.rand(m5, device=dev).bfloat16()
            o5 = torch.empty(m5, n5, dtype=torch.bfloat16, device=dev)
            f = lambda i: launchers.hip_gemm_a8w8_forward(o5, a5, w5[i % 5], s5, c5)
            for i in range(10):
                f(i)
            ms = _events_ms(f, 100, torch)
            b5 = float(n5) * k5 + m5 * k5 + 2.0 * m5 * n5 + 2.0 * m5 + 4.0 * n5
            secondary.append({"workload": f"a8w8 few rows M={m5} K={k5} N={n5} bf16",
                              "kernel": "gemm_a8w8_skinny_kernel" if m5 == 1 else "gemm_a8w8_panel_kernel",
                              "us_per_launch": round(ms * 1e3, 2),
                              "roofline": {"bound": "hbm", "achieved": round(b5 / (ms * 1e-3) / 1e9, 1),
                                           "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                           "frac": round(b5 / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "traffic": None}})
        del w5
        torch.cuda.empty_cache()

    # ------------------------------------------------------- A16W8 decode + row kernels
    if "rows" in legs:
        for (k8, n8) in workloads.A16W8_DECODE_SHAPES:
            nset8 = max(3, int(600e6 // (k8 * n8)) + 1)
            w8 = [torch.randint(-127, 128, (n8, k8), dtype=torch.int8, device=dev) for _ in range(nset8)]
            s8 = torch.rand(n8, device=dev).half() * 0.01
            for m8 in (1, 8, 32):
                act = workloads.activations(m8, k8, torch.float16, seed=4).to(dev)
                o8 = torch.empty(m8, n8, dtype=torch.float16, device=dev)
                f = lambda i: launchers.hip_gemm_a16w8_forward(o8, act, w8[i % nset8], s8)
                for i in range(10):
                    f(i)
                ms = _events_ms(f, 100, torch)
                b8 = n8 * k8 + 2.0 * n8 + 2.0 * m8 * k8 + 2.0 * m8 * n8
                secondary.append({"workload": f"a16w8 decode M={m8} K={k8} N={n8} fp16",
                                  "kernel": "gemm_wo_decode_lds_kernel" if m8 == 1 else "gemm_wo_panel_kernel",
                                  "us_per_launch": round(ms * 1e3, 2),
                                  "roofline": {"bound": "hbm", "achieved": round(b8 / (ms * 1e-3) / 1e9, 1),
                                               "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                               "frac": round(b8 / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "traffic": None}})
            del w8
        Mr, Kr = 8192, 8192
        hs = [workloads.activations(Mr, Kr, torch.bfloat16, seed=5, outlier_frac=0.01).to(dev) for _ in range(3)]
        norm = flashnn_amd.RMSNormDquant(Kr).to(dev)
        norm.weight.data = workloads.rmsnorm_gamma(Kr).to(dev)
        f = lambda i: norm(hs[i % 3])
        for i in range(5):
            f(i)
        ms = _events_ms(f, 50, torch)
        rb = 3.0 * Mr * Kr + 4.0 * Kr + 2.0 * Mr
        secondary.append({"workload": f"rmsnorm_dquant bf16 M={Mr} K={Kr}", "kernel": "rmsnorm_dquant_vec_kernel",
                          "us_per_launch": round(ms * 1e3, 2),
                          "roofline": {"bound": "hbm", "achieved": round(rb / (ms * 1e-3) / 1e9, 1),
                                       "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                       "frac": round(rb / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "traffic": None}})
        # the layers one step before the path, same matrix
        for name, mod, kern, wr in (("rmsnorm", flashnn_amd.RMSNorm(Kr), "norm_vec_kernel", 2.0),
                                    ("layernorm", flashnn_amd.LayerNorm(Kr), "norm_vec_kernel", 2.0),
                                    ("layernorm_dquant", flashnn_amd.LayernormDquant(Kr), "norm_vec_kernel", 1.0)):
            mod = mod.to(torch.bfloat16).to(dev)
            f = lambda i: mod(hs[i % 3])
            for i in range(5):
                f(i)
            ms = _events_ms(f, 50, torch)
            nb = (2.0 + wr) * Mr * Kr
            secondary.append({"workload": f"{name} bf16 M={Mr} K={Kr}", "kernel": kern,
                              "us_per_launch": round(ms * 1e3, 2),
                              "roofline": {"bound": "hbm", "achieved": round(nb / (ms * 1e-3) / 1e9, 1),
                                           "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                           "frac": round(nb / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "traffic": None}})
        del hs
        torch.cuda.empty_cache()

    # ------------------------------------------------ mixture of experts, int8 (decode-sized batches)
    if "moe" in legs:
        E, Nm, Km, top_k, BMm = 8, 28672, 4096, 2, 16     # Mixtral-8x7B-like gate+up projection
        g = torch.Generator(device=dev).manual_seed(7)
        bm = torch.randint(-127, 128, (E, Nm, Km), dtype=torch.int8, device=dev, generator=g)
        acm = torch.rand(E, Nm, device=dev, generator=g) * 0.01
        for Mt in (16, 64):
            am = torch.randint(-127, 128, (Mt, Km), dtype=torch.int8, device=dev, generator=g)
            arm = torch.rand(Mt, device=dev, generator=g).half()
            tw, tid = torch.topk(torch.softmax(torch.randn(Mt, E, generator=torch.Generator().manual_seed(8)), -1), top_k)
            sid, eid, used = workloads.moe_align_block_size(tid, BMm, E)
            active = len(set(tid.flatten().tolist()))
            tw, tid, sid, eid, used = (t.to(dev) for t in (tw.float().contiguous(), tid, sid, eid, used))
            cm = torch.empty(Mt, top_k, Nm, dtype=torch.bfloat16, device=dev)
            f = lambda i: flashnn_amd.fused_moe_a8w8_forward(am, bm, cm, arm, acm, tw, tid, sid, eid, used, True, top_k, BMm)
            for i in range(3):
                f(i)
            ms = _events_ms(f, 20, torch)
            mb_ = float(active) * Nm * Km + 2.0 * Mt * top_k * Nm      # weights of the experts in use + output
            secondary.append({"workload": f"fused_moe_a8w8 tokens={Mt} E={E} top_k={top_k} K={Km} N={Nm} block={BMm} "
                                          f"({active} experts in use)", "kernel": "gemm_a8w8_panel_kernel",
                              "us_per_launch": round(ms * 1e3, 2),
                              "roofline": {"bound": "hbm", "achieved": round(mb_ / (ms * 1e-3) / 1e9, 1),
                                           "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                           "frac": round(mb_ / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "traffic": None}})
        del bm
        torch.cuda.empty_cache()
        # int4 expert weights, per-channel scales, same layer
        N2 = Nm // 2
        b4 = torch.randint(-128, 128, (E, N2, Km), dtype=torch.int8, device=dev, generator=g)
        sc4 = (torch.rand(E, Nm, device=dev, generator=g) * 0.01).to(torch.bfloat16)
        zp4m = torch.randint(-3, 4, (E, Nm), device=dev, generator=g).to(torch.bfloat16)
        for Mt in (16, 64):
            a4 = torch.randn(Mt, Km, device=dev, generator=g).to(torch.bfloat16)
            tw, tid = torch.topk(torch.softmax(torch.randn(Mt, E, generator=torch.Generator().manual_seed(8)), -1), top_k)
            sid, eid, used = workloads.moe_align_block_size(tid, BMm, E)
            active = len(set(tid.flatten().tolist()))
            tw, tid, sid, eid, used = (t.to(dev) for t in (tw.float().contiguous(), tid, sid, eid, used))
            cm = torch.empty(Mt, top_k, Nm, dtype=torch.bfloat16, device=dev)
            f = lambda i: flashnn_amd.fused_moe_a16w4_forward(a4, b4, cm, sc4, zp4m, tw, tid, sid, eid, used, True, top_k, BMm)
            for i in range(3):
                f(i)
            ms = _events_ms(f, 20, torch)
            mb_ = float(active) * N2 * Km + 2.0 * Mt * top_k * Nm
            secondary.append({"workload": f"fused_moe_a16w4 per-channel tokens={Mt} E={E} top_k={top_k} K={Km} N={Nm} "
                                          f"block={BMm} ({active} experts in use)", "kernel": "gemm_wo_panel_kernel",
                              "us_per_launch": round(ms * 1e3, 2),
                              "roofline": {"bound": "hbm", "achieved": round(mb_ / (ms * 1e-3) / 1e9, 1),
                                           "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                           "frac": round(mb_ / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "traffic": None}})
        # ... and with scales and zero points per group of 128, [E, N, K/128] as the reference lays them out
        sc4g = (torch.rand(E, Nm, Km // 128, device=dev, generator=g) * 0.01).to(torch.bfloat16)
        zp4g = torch.randint(-3, 4, (E, Nm, Km // 128), device=dev, generator=g).to(torch.bfloat16)
        a4 = torch.randn(16, Km, device=dev, generator=g).to(torch.bfloat16)
        tw, tid = torch.topk(torch.softmax(torch.randn(16, E, generator=torch.Generator().manual_seed(8)), -1), top_k)
        sid, eid, used = workloads.moe_align_block_size(tid, BMm, E)
        active = len(set(tid.flatten().tolist()))
        tw, tid, sid, eid, used = (t.to(dev) for t in (tw.float().contiguous(), tid, sid, eid, used))
        cm = torch.empty(16, top_k, Nm, dtype=torch.bfloat16, device=dev)
        f = lambda i: flashnn_amd.fused_moe_a16w4_forward(a4, b4, cm, sc4g, zp4g, tw, tid, sid, eid, used, True, top_k, BMm)
        for i in range(3):
            f(i)
        ms = _events_ms(f, 20, torch)
        mb_ = float(active) * (N2 * Km + 4.0 * Nm * (Km // 128)) + 2.0 * 16 * top_k * Nm
        secondary.append({"workload": f"fused_moe_a16w4 group 128 tokens=16 E={E} top_k={top_k} K={Km} N={Nm} "
                                      f"block={BMm} ({active} experts in use)", "kernel": "gemm_wo_panel_kernel",
                          "us_per_launch": round(ms * 1e3, 2),
                          "roofline": {"bound": "hbm", "achieved": round(mb_ / (ms * 1e-3) / 1e9, 1),
                                       "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                       "frac": round(mb_ / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "traffic": None}})
        del b4
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ CPU baseline
    cpu_baseline = None
    if not args.no_cpu:
        from oracle import torch_path as T
        cores = torch.get_num_threads()

        def cpu_step():
            q, s = T.dynamic_quantize(x_cpu)
            return T.gemm_a8w8(q, w_cpu, s.float(), ws_cpu, torch.bfloat16)

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
        cpu_baseline = {"value": round(ops / t_cpu / 1e12, 4), "unit": "TOPS", "cores": cores, "kind": "port",
                        "sample": f"the whole step (dynamic quant + fp32-matmul A8W8, M={M} K={K} N={N}) through "
                                  f"the torch-op restatement of the reference's CPU path, median of 3 runs "
                                  f"({t_cpu * 1e3:.0f} ms each)",
                        "a16w4_decode_m1_ms": round(t_cpu4 * 1e3, 1),
                        "a16w4_decode_m1_weight_GBps": round((N4 * K4 / 2 + 4 * (K4 // 128) * N4) / t_cpu4 / 1e9, 3)}

    result = {
        "metric": "a8w8_int8_tops_m2048", "value": round(value, 2), "unit": "TOPS", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "preroll_steps": preroll_steps, "ms_per_step": round(ms_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "DynamicQuant(fp16 [2048,4096], 1% outlier channels x20) + A8W8 GEMM "
                               "M=2048 K=4096 N=12288, int8 per-channel weights, bf16 out (Llama-7B QKV prefill)",
                   "rotating_operand_sets": nset, "device": props.name, "cus": props.multi_processor_count,
                   "host_wall_ms_per_step": round(wall_ms, 5)},
        "roofline": roofline, "cpu_baseline": cpu_baseline, "secondary": secondary,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
