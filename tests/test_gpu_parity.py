"""GPU parity tests: the HIP kernels, called through the C ABI, against the CPU oracle on the
same seeded inputs.  int8 outputs, fp16 scales and int32 accumulators must be bit-exact;
fp16/bf16 GEMM outputs must be within rtol 1e-2 / atol 1e-2 of the reference's torch path."""
import sys

import numpy as np
import pytest
import torch

import flashnn_amd
from flashnn_amd import _lib, launchers, workloads
from oracle import flashnn_oracle as O

pytestmark = pytest.mark.gpu

RTOL = ATOL = 1e-2   # tolerance stated for the fp16/bf16 outputs
DEV = "cuda:0"


@pytest.fixture(autouse=True)
def _announce(request):
    # name the case before any GPU work starts, so that a fault can be attributed
    print(f"[gpu-case] {request.node.nodeid}", file=sys.__stderr__, flush=True)
    yield
    torch.cuda.synchronize()


def _tag(dt):
    return O.tag_of(torch.empty(0, dtype=dt))


# ---------------------------------------------------------------------- dynamic quant
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(32, 32), (64, 64), (128, 128), (117, 987), (2560, 8000), (16, 4096),
                                   (3, 11008), (5, 16384), (2, 35584), (1, 8), (3, 17792), (2, 40960),
                                   (2, 40968)])
def test_dynamic_quant_bit_exact(dtype, shape):
    torch.manual_seed(0)
    x = (torch.rand(shape) * 2 - 1).to(dtype) if shape[0] % 2 else torch.randn(shape).to(dtype)
    q, s = flashnn_amd.DynamicQuantize()(x.to(DEV))
    q_o, s_o = O.dynamic_quantize(O.to_np(x), _tag(dtype))
    assert q.dtype == torch.int8 and s.dtype == torch.float16 and s.shape == (shape[0],)
    assert np.array_equal(s.cpu().numpy(), s_o)
    assert np.array_equal(q.cpu().numpy(), q_o)


def test_dynamic_quant_outliers_and_zero_row():
    x = workloads.activations(2048, 4096, torch.float16, seed=5, outlier_frac=0.01)
    x[7] = 0
    q, s = flashnn_amd.DynamicQuantize()(x.to(DEV))
    q_o, s_o = O.dynamic_quantize(O.to_np(x), O.F16)
    assert np.array_equal(q.cpu().numpy(), q_o) and np.array_equal(s.cpu().numpy(), s_o)
    assert not q[7].any() and s[7] == 0
    rows = np.abs(q_o.astype(np.int32)).max(axis=1)
    assert (np.delete(rows, 7) == 127).all()


def test_dynamic_quant_bf16_row_maximum_is_clamped():
    """bf16 rows whose maximum would quantise to 128 (see the oracle test of the same name): the kernel
    clamps, bit-exact with the oracle, max |q| >= 127, never a sign flip of a large activation."""
    torch.manual_seed(3)
    x = torch.randn(4096, 1024).bfloat16()
    for j in range(42, 63):
        x[j, :] = 0
        x[j, 5] = 1.0 + j / 128.0
        x[j, 6] = -0.5
    xn = O.to_np(x)
    q, s = flashnn_amd.DynamicQuantize()(x.to(DEV))
    q_o, s_o = O.dynamic_quantize(xn, O.BF16)
    assert np.array_equal(q.cpu().numpy(), q_o) and np.array_equal(s.cpu().numpy(), s_o)
    qn = q.cpu().numpy()
    big = np.abs(xn) > s_o.astype(np.float32)[:, None]
    assert (np.sign(qn[big]) == np.sign(xn[big])).all()
    assert (qn[42:63, 5] == 127).all()
    # the strided (non-vector) kernel: K not a multiple of 8
    x2 = x[:64, :1021].contiguous()
    q2, s2 = flashnn_amd.DynamicQuantize()(x2.to(DEV))
    q2_o, s2_o = O.dynamic_quantize(O.to_np(x2), O.BF16)
    assert np.array_equal(q2.cpu().numpy(), q2_o) and np.array_equal(s2.cpu().numpy(), s2_o)


# -------------------------------------------------------------------- rmsnorm + quant
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 128), (3, 32, 1024), (32, 8192), (7, 1000), (2, 20480), (3, 35584),
                                   (2, 40960), (1, 41000),
                                   # many short rows: the one-wave-per-row kernel (1, 2 and 4 vectors per lane,
                                   # ragged last vector row, a row count that is no multiple of four)
                                   (2050, 2048), (2049, 1000), (4096, 512), (2051, 264), (3, 700, 1024)])
@pytest.mark.parametrize("gamma_dtype", [torch.float32, None])
def test_rmsnorm_dquant_bit_exact(dtype, shape, gamma_dtype):
    torch.manual_seed(1)
    x = workloads.activations(int(np.prod(shape[:-1])), shape[-1], dtype, seed=11, outlier_frac=0.01).reshape(shape)
    gamma = workloads.rmsnorm_gamma(shape[-1]).to(gamma_dtype or dtype)
    mod = flashnn_amd.RMSNormDquant(shape[-1], eps=1e-6).to(DEV)
    mod.weight.data = gamma.to(DEV)
    q, s = mod(x.to(DEV))
    q_o, s_o = O.rmsnorm_dquant(O.to_np(x), O.to_np(gamma), 1e-6, _tag(dtype))
    assert q.shape == x.shape and s.shape == x.shape[:-1] and s.dtype == dtype
    assert np.array_equal(s.float().cpu().numpy(), s_o)
    assert np.array_equal(q.cpu().numpy(), q_o)


# ------------------------------------------------------------------------ A8W8 GEMM
def _rand_i8(shape, seed, lo=-128, hi=128):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi, shape, generator=g, dtype=torch.int8)


# every tile of the MFMA kernel: (rows, columns, waves); (0, 0, 0) = the library's own choice
TILES = [(0, 0, 0), (256, 256, 0), (256, 192, 0), (256, 128, 0), (128, 128, 0), (64, 128, 0), (256, 256, 4)]


def _scaled(out_ty, a, b, ar, ac, tile):
    out = torch.empty((a.shape[0], b.shape[0]), dtype=out_ty, device=a.device)
    return launchers.hip_gemm_a8w8_forward(out, a, b, ar, ac, tile=tile)


@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("mnk", [(128, 128, 128), (300, 200, 512), (512, 768, 1024), (16, 4096, 4096),
                                 (257, 129, 640), (64, 320, 1152), (130, 100, 2048)])
def test_a8w8_accumulators_bit_exact(tile, mnk):
    M, N, K = mnk
    a, b = _rand_i8((M, K), 1), _rand_i8((N, K), 2)
    acc = launchers.hip_gemm_a8w8_int32(a.to(DEV), b.to(DEV), tile).cpu().numpy()
    assert np.array_equal(acc, O.gemm_a8w8_acc(a.numpy(), b.numpy()))


@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("mnk", [(300, 200, 544), (257, 385, 576), (64, 320, 608), (130, 100, 1056),
                                 (10, 1920, 1760), (40, 260, 7392), (520, 390, 8896)])
def test_a8w8_partial_last_slab_bit_exact(tile, mnk):
    """K a multiple of 32 but not of 128 (the FFN shapes of models sharded over 4 or 8 GPUs): the
    last 128-byte slab holds one to three k-steps; few-row problems take the tiled kernel too."""
    M, N, K = mnk
    a, b = _rand_i8((M, K), 21), _rand_i8((N, K), 22)
    acc = launchers.hip_gemm_a8w8_int32(a.to(DEV), b.to(DEV), tile).cpu().numpy()
    g = torch.Generator().manual_seed(23)
    ar = (torch.rand(M, 1, generator=g) * 0.05).half()
    ac = (torch.rand(1, N, generator=g) * 0.05).half()
    out = _scaled(torch.float16, a.to(DEV), b.to(DEV), ar.to(DEV), ac.to(DEV), tile if tile[0] else None)
    want = O.gemm_a8w8_acc(a.numpy(), b.numpy())
    assert np.array_equal(acc, want)
    assert np.array_equal(out.float().cpu().numpy(), O.gemm_a8w8_epilogue_fp32(want, O.to_np(ar), O.to_np(ac), O.F16))


@pytest.mark.parametrize("tile,mn", [((64, 128, 0), (720, 773)), ((64, 128, 0), (1100, 300)),
                                     ((128, 128, 0), (1290, 650)), ((256, 128, 0), (2310, 1100)),
                                     ((256, 192, 0), (2400, 1000)), ((256, 192, 0), (2600, 200)),
                                     ((256, 256, 0), (2600, 1300))])
def test_a8w8_tile_numbering_many_tile_rows(tile, mn):
    """More than 8 tile rows and a number of tile columns that is no multiple of 4: the tiles are numbered
    in groups of 4 tile columns, and the last group is narrower."""
    M, N = mn
    K = 512
    a, b = _rand_i8((M, K), 31), _rand_i8((N, K), 32)
    acc = launchers.hip_gemm_a8w8_int32(a.to(DEV), b.to(DEV), tile).cpu().numpy()
    assert np.array_equal(acc, O.gemm_a8w8_acc(a.numpy(), b.numpy()))


@pytest.mark.parametrize("mnk", [(2080, 2060, 512), (2200, 2100, 1184), (700, 6200, 640)])
def test_a8w8_128x128_pairs_bit_exact(mnk):
    """More than 256 tiles of 128x128: the launcher takes the version of the tile that fits two workgroups
    on a CU (two a-stages, scales staged in the third b-stage before the epilogue).  Accumulators and the
    scaled 16-bit output, K a multiple of 128 and not."""
    M, N, K = mnk
    assert ((M + 127) // 128) * ((N + 127) // 128) > 256
    a, b = _rand_i8((M, K), 41), _rand_i8((N, K), 42)
    acc = launchers.hip_gemm_a8w8_int32(a.to(DEV), b.to(DEV), (128, 128, 0)).cpu().numpy()
    g = torch.Generator().manual_seed(43)
    ar = (torch.rand(M, 1, generator=g) * 0.05).half()
    ac = (torch.rand(1, N, generator=g) * 0.05).half()
    out = _scaled(torch.bfloat16, a.to(DEV), b.to(DEV), ar.to(DEV), ac.to(DEV), (128, 128, 0))
    want = O.gemm_a8w8_acc(a.numpy(), b.numpy())
    assert np.array_equal(acc, want)
    assert np.array_equal(out.float().cpu().numpy(), O.gemm_a8w8_epilogue_fp32(want, O.to_np(ar), O.to_np(ac), O.BF16))


@pytest.mark.parametrize("mnk", [(5, 7, 100), (130, 70, 1000), (64, 64, 8), (33, 65, 129)])
def test_a8w8_guarded_kernel_bit_exact(mnk):
    M, N, K = mnk
    a, b = _rand_i8((M, K), 3), _rand_i8((N, K), 4)
    acc = launchers.hip_gemm_a8w8_int32(a.to(DEV), b.to(DEV)).cpu().numpy()
    assert np.array_equal(acc, O.gemm_a8w8_acc(a.numpy(), b.numpy()))


@pytest.mark.parametrize("M", [1, 7, 16, 17, 33, 48, 64])
@pytest.mark.parametrize("nk", [(1000, 64), (16, 448), (4100, 4096), (520, 8192),
                                # shared activation slabs: 16-, 32- and 64-row workgroups, uneven K parts
                                (4096, 4096), (8192, 1152), (16384, 1024), (2048, 11008),
                                # K a multiple of 32 only: the last slab holds 32, 64 or 96 bytes
                                (4096, 1056), (8192, 7392), (2048, 8896), (1920, 1120), (16, 1088)])
def test_a8w8_few_rows_bit_exact(M, nk):
    """Up to 64 activation rows take the weight-streaming kernel: accumulators and scaled outputs,
    N not a multiple of the 16-row tile, fewer k-steps than waves."""
    N, K = nk
    a, b = _rand_i8((M, K), 10 + M), _rand_i8((N, K), 11)
    acc = launchers.hip_gemm_a8w8_int32(a.to(DEV), b.to(DEV)).cpu().numpy()
    want = O.gemm_a8w8_acc(a.numpy(), b.numpy())
    assert np.array_equal(acc, want)
    g = torch.Generator().manual_seed(12)
    out_ty = torch.float16 if M % 2 else torch.bfloat16
    ar = (torch.rand(M, 1, generator=g) * 0.05).to(out_ty)
    ac = (torch.rand(1, N, generator=g) * 0.05).float()
    out = flashnn_amd.GemmA8W8(out_ty)(a.to(DEV), b.to(DEV), ar.to(DEV), ac.to(DEV))
    assert np.array_equal(out.float().cpu().numpy(),
                          O.gemm_a8w8_epilogue_fp32(want, O.to_np(ar), O.to_np(ac), _tag(out_ty)))


@pytest.mark.parametrize("M,N,K,kernel", [(33, 16640, 1024, "ring"), (64, 17792, 512, "ring"), (48, 24576, 1056, "ring"),
                                          (17, 28672, 1024, "ring"), (64, 16384, 1024, "panel"), (16, 17792, 1024, "panel"),
                                          (64, 32768, 1024, "panel")])
def test_a8w8_between_one_and_two_rounds_of_few_row_workgroups(M, N, K, kernel):
    """17 .. 64 rows over 16385 .. 32767 channels run on the tiled kernel (one round of 64x128 tiles) instead of
    257 .. 511 workgroups of the few-row kernel; the neighbouring shapes stay where they were.  Same bits."""
    a, b = _rand_i8((M, K), 61), _rand_i8((N, K), 62)
    acc = flashnn_amd.launchers.hip_gemm_a8w8_int32(a.to(DEV), b.to(DEV)).cpu().numpy()
    assert _lib.last_kernel().startswith(f"gemm_a8w8_{kernel}_kernel"), _lib.last_kernel()
    assert np.array_equal(acc, O.gemm_a8w8_acc(a.numpy(), b.numpy()))


@pytest.mark.parametrize("M,N,K,kernel", [(2, 4096, 4096, "skinny"), (16, 4096, 1024, "skinny"), (9, 1024, 11008, "skinny"),
                                          (16, 8192, 3072, "skinny"), (8, 8192, 8192, "skinny"), (3, 16384, 8192, "skinny"),
                                          (17, 4096, 4096, "panel"), (16, 4112, 4096, "panel"), (16, 8192, 3200, "panel"),
                                          (9, 16384, 8192, "panel"), (8, 16384, 8064, "panel"), (8, 8176, 8192, "panel"),
                                          (4, 4096, 1056, "panel"), (16, 16384, 8192, "panel<1,2"), (16, 16384, 4096, "panel<2,4"),
                                          (16, 16384, 8320, "panel<2,4")])
def test_a8w8_up_to_16_rows_which_few_row_kernel(M, N, K, kernel):
    """Up to 16 rows: the kernel that splits K over the waves of a 16-channel workgroup where there are few
    workgroups (N <= 4096, or N <= 8192 with K <= 3072) and for up to 8 rows of K >= 8192 over N >= 8192; the
    shared-slab kernel next to those ranges (and for any K that is no multiple of 128) - with 32 instead of 64 weight
    rows per workgroup where the rows lie a multiple of 8 KiB apart.  Same bits either way."""
    a, b = _rand_i8((M, K), 63), _rand_i8((N, K), 64)
    acc = flashnn_amd.launchers.hip_gemm_a8w8_int32(a.to(DEV), b.to(DEV)).cpu().numpy()
    kernel, _, blocks = kernel.partition("<")
    assert _lib.last_kernel().startswith(f"gemm_a8w8_{kernel}_kernel" + ("<" + blocks if blocks else "")), _lib.last_kernel()
    assert np.array_equal(acc, O.gemm_a8w8_acc(a.numpy(), b.numpy()))
    g = torch.Generator().manual_seed(65)
    ar, ac = (torch.rand(M, generator=g) * 0.05).half(), (torch.rand(N, generator=g) * 0.05).half()
    out = flashnn_amd.GemmA8W8(torch.bfloat16)(a.to(DEV), b.to(DEV), ar.to(DEV), ac.to(DEV)).float().cpu().numpy()
    assert _lib.last_kernel().startswith(f"gemm_a8w8_{kernel}_kernel"), _lib.last_kernel()
    assert np.array_equal(out, O.gemm_a8w8_epilogue_fp32(acc, O.to_np(ar), O.to_np(ac), O.BF16))


@pytest.mark.parametrize("M,N,tile", [(100, 33024, "256,192"), (128, 38912, "256,192"), (65, 32768, "128,128"), (129, 33024, None)])
def test_a8w8_few_rows_over_a_little_more_than_one_round_of_tiles(M, N, tile):
    """Up to 128 rows over 32769 .. 38912 channels take one round of 256x192 tiles (rows beyond M are padding)
    instead of 257 .. 304 tiles of 128 columns in pairs; the shapes next to that range keep their tiles."""
    K = 512
    a, b = _rand_i8((M, K), 71), _rand_i8((N, K), 72)
    acc = flashnn_amd.launchers.hip_gemm_a8w8_int32(a.to(DEV), b.to(DEV)).cpu().numpy()
    if tile:
        assert _lib.last_kernel() == f"gemm_a8w8_ring_kernel<{tile},4>", _lib.last_kernel()
    assert np.array_equal(acc, O.gemm_a8w8_acc(a.numpy(), b.numpy()))


def test_a8w8_saturation_and_identity():
    a = torch.full((256, 4096), -128, dtype=torch.int8)
    acc = launchers.hip_gemm_a8w8_int32(a.to(DEV), a.to(DEV))
    assert bool((acc == 67108864).all())          # 2^26: no fp32 accumulation, no saturation
    eye = torch.eye(128, dtype=torch.int8)
    b = _rand_i8((128, 128), 5)
    acc = launchers.hip_gemm_a8w8_int32(eye.to(DEV), b.to(DEV)).cpu()
    assert torch.equal(acc, b.t().int())


@pytest.mark.parametrize("out_ty,scale_ty", [(torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
                                             (torch.bfloat16, torch.float32), (torch.float16, torch.float32)])
@pytest.mark.parametrize("mnk", [(128, 128, 128), (16, 4096, 4096), (300, 520, 512), (33, 65, 129)])
def test_a8w8_scaled_output(out_ty, scale_ty, mnk):
    M, N, K = mnk
    a, b = _rand_i8((M, K), 6, -128, 127), _rand_i8((N, K), 7, -128, 127)
    g = torch.Generator().manual_seed(8)
    ar = (torch.rand(M, 1, generator=g) * 0.05).to(scale_ty)
    ac = (torch.rand(1, N, generator=g) * 0.05).to(scale_ty)
    out = flashnn_amd.GemmA8W8(out_ty)(a.to(DEV), b.to(DEV), ar.to(DEV), ac.to(DEV))
    assert out.dtype == out_ty and out.shape == (M, N)
    got = out.float().cpu().numpy()
    acc = O.gemm_a8w8_acc(a.numpy(), b.numpy())
    # same fp32 operations in the same order: identical bits
    assert np.array_equal(got, O.gemm_a8w8_epilogue_fp32(acc, O.to_np(ar), O.to_np(ac), _tag(out_ty)))
    np.testing.assert_allclose(got, O.gemm_a8w8(a.numpy(), b.numpy(), O.to_np(ar), O.to_np(ac), _tag(out_ty)),
                               rtol=RTOL, atol=ATOL)


def test_dynamic_quant_then_a8w8_small_config():
    """DynamicQuant + A8W8, M=16 K=4096 N=4096, fp16 out: the CPU-runnable configuration."""
    x = workloads.activations(16, 4096, torch.float16, seed=0)
    w, ws = workloads.int8_weights(4096, 4096)
    q, s = flashnn_amd.DynamicQuantize()(x.to(DEV))
    out = flashnn_amd.GemmA8W8(torch.float16)(q, w.to(DEV), s, ws.to(DEV))
    q_o, s_o = O.dynamic_quantize(O.to_np(x), O.F16)
    assert np.array_equal(q.cpu().numpy(), q_o) and np.array_equal(s.cpu().numpy(), s_o)
    acc = launchers.hip_gemm_a8w8_int32(q, w.to(DEV)).cpu().numpy()
    assert np.array_equal(acc, O.gemm_a8w8_acc(q_o, w.numpy()))
    want = O.gemm_a8w8(q_o, w.numpy(), s_o.astype(np.float32), ws.numpy(), O.F16)
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("name", ["qkv", "o", "gate_up", "down"])
def test_a8w8_prefill_full_size(name):
    """M=2048 prefill shapes: accumulators of sampled rows bit-exact, all outputs within
    tolerance for those rows, and a checksum identity over the whole result:
    sum_n acc[m,n] = a[m,:] . (sum_n b[n,:])."""
    K, N = workloads.A8W8_PREFILL_SHAPES[name]
    M = 2048
    x = workloads.activations(M, K, torch.float16, seed=21, outlier_frac=0.01)
    w, ws = workloads.int8_weights(N, K, seed=22)
    q, s = flashnn_amd.DynamicQuantize()(x.to(DEV))
    q_o, s_o = O.dynamic_quantize(O.to_np(x), O.F16)
    assert np.array_equal(q.cpu().numpy(), q_o)
    wd = w.to(DEV)
    acc = launchers.hip_gemm_a8w8_int32(q, wd)
    rows = np.random.default_rng(0).choice(M, 48, replace=False)
    rows[:2] = (0, M - 1)
    acc_rows = acc[torch.from_numpy(rows).to(DEV)].cpu().numpy()
    assert np.array_equal(acc_rows, O.gemm_a8w8_acc(q_o[rows], w.numpy()))
    colsum = w.numpy().astype(np.int64).sum(axis=0)
    assert np.array_equal(acc.sum(dim=1, dtype=torch.int64).cpu().numpy(), q_o.astype(np.int64) @ colsum)
    out = flashnn_amd.GemmA8W8(torch.bfloat16)(q, wd, s, ws.to(DEV))
    want = O.gemm_a8w8_epilogue_fp32(acc_rows, s_o.astype(np.float32)[rows], ws.numpy(), O.BF16)
    assert np.array_equal(out[torch.from_numpy(rows).to(DEV)].float().cpu().numpy(), want)


_SWEEP_B = {}


@pytest.mark.parametrize("M", [1, 10, 40, 764, 2048, 4096, 8192])
@pytest.mark.parametrize("nk", workloads.sharded_model_gemm_shapes())
def test_a8w8_reference_sweep_shapes(nk, M):
    """The (N, K) pairs and row counts of the reference's A8W8 sweep, inputs drawn as its own test
    draws them (benchmark/benchmark_gemm_a8w8_amd.py:104-124: randint(-12, 12), fp16 scales from
    rand, fp16 out).  Sampled rows x sampled columns of the result, tile edges included, must equal
    the oracle bit for bit; a checksum identity covers every accumulator."""
    N, K = nk
    g = torch.Generator(device=DEV).manual_seed(N * 31 + K)
    if nk not in _SWEEP_B:
        _SWEEP_B.clear()
        _SWEEP_B[nk] = torch.randint(-12, 12, (N, K), dtype=torch.int8, device=DEV, generator=g)
    b = _SWEEP_B[nk]
    g.manual_seed(M * 7 + 1)
    a = torch.randint(-12, 12, (M, K), dtype=torch.int8, device=DEV, generator=g)
    ar = torch.rand(M, 1, device=DEV, generator=g).half()
    ac = torch.rand(1, N, device=DEV, generator=g).half()
    out = flashnn_amd.GemmA8W8(out_ty=torch.half)(a, b, ar, ac)
    acc = launchers.hip_gemm_a8w8_int32(a, b)
    rng = np.random.default_rng(M + N)
    rows = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, 14)]))
    cols = np.unique(np.concatenate([[0, N - 1, N - N % 192 - 1], rng.integers(0, N, 125)]))
    ri, ci = torch.from_numpy(rows).to(DEV), torch.from_numpy(cols).to(DEV)
    want = O.gemm_a8w8_acc(a[ri].cpu().numpy(), b[ci].cpu().numpy())
    assert np.array_equal(acc[ri][:, ci].cpu().numpy(), want)
    want_out = O.gemm_a8w8_epilogue_fp32(want, O.to_np(ar[ri].cpu()), O.to_np(ac[:, ci].cpu()), O.F16)
    assert np.array_equal(out[ri][:, ci].float().cpu().numpy(), want_out)
    # sum_n acc[m, n] = a[m, :] . sum_n b[n, :], in exact integers
    colsum = b.sum(dim=0, dtype=torch.int64)
    assert torch.equal(acc.sum(dim=1, dtype=torch.int64), (a.to(torch.int64) * colsum).sum(dim=1))


def _a8w8_ws_call(hip_lib, out, a, b, ar, ac, ws, plan=None):
    M, K = a.shape
    N = b.shape[0]
    args = (out.data_ptr(), a.data_ptr(), b.data_ptr(), ar.data_ptr(), ac.data_ptr(), M, N, K, K, K, N,
            _lib.dtype_code(out.dtype), _lib.dtype_code(ar.dtype), _lib.dtype_code(ac.dtype))
    st = _lib.current_stream(a.device)
    if plan is None:
        return hip_lib.fnn_gemm_a8w8_ws(*args, ws.data_ptr(), ws.numel(), st)
    return hip_lib.fnn_gemm_a8w8_ws_tiled(*args, *plan, ws.data_ptr(), ws.numel(), st)


@pytest.mark.parametrize("plan", [(256, 128, 2), (256, 128, 3), (256, 192, 2), (256, 192, 5), (128, 128, 2), (128, 128, 4),
                                  (128, 128, 7)])
@pytest.mark.parametrize("mnk", [(300, 520, 4096), (128, 1024, 8192), (257, 385, 5152), (96, 200, 4128), (640, 256, 6240)])
def test_a8w8_split_k_bit_exact(hip_lib, plan, mnk):
    """K cut into parts that meet in a workspace: the int32 sums do not depend on the order of arrival, so
    the scaled output equals the unsplit kernel's and the oracle's bit for bit - for every tile, number of
    parts, ragged edges and a partial last slab; the counters are zero again afterwards; a second call on
    the same workspace (holding the first call's slots) gives the same bits."""
    M, N, K = mnk
    a, b = _rand_i8((M, K), 61).to(DEV), _rand_i8((N, K), 62).to(DEV)
    g = torch.Generator().manual_seed(63)
    ar = (torch.rand(M, generator=g) * 1e-2 + 1e-3).half().to(DEV)
    ac = (torch.rand(N, generator=g) * 1e-2 + 1e-3).float().to(DEV)
    ws = torch.zeros(24 << 20, dtype=torch.uint8, device=DEV)
    ws[4096:] = 0x5a                                   # only the counters need to start at zero
    want = O.gemm_a8w8_epilogue_fp32(O.gemm_a8w8_acc(a.cpu().numpy(), b.cpu().numpy()), O.to_np(ar.cpu()),
                                     ac.cpu().numpy(), O.BF16)
    for rep in range(2):
        out = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=DEV)
        rc = _a8w8_ws_call(hip_lib, out, a, b, ar, ac, ws, plan)
        assert rc == 0, hip_lib.fnn_last_error()
        assert _lib.last_kernel() == f"gemm_a8w8_ring_kernel(split K)<{plan[0]},{plan[1]},{plan[2]}>"
        assert np.array_equal(out.float().cpu().numpy(), want)
        assert int(ws[:4096].view(torch.int32).abs().sum()) == 0
    plain = torch.empty_like(out)
    launchers.hip_gemm_a8w8_forward(plain, a, b, ar, ac, tile=(plan[0], plan[1], 0))
    assert torch.equal(plain, out)


@pytest.mark.parametrize("mnk", [(256, 4096, 8192), (128, 2304, 16384), (384, 1920, 13312), (100, 1000, 9248), (2048, 4096, 4096),
                                 (1024, 1920, 13312), (512, 3584, 18944), (256, 8960, 13312), (256, 4096, 6144)])
def test_a8w8_workspace_entry_matches_plain(hip_lib, mnk):
    """fnn_gemm_a8w8_ws: shapes the library splits (and one it does not) against fnn_gemm_a8w8, bit for bit,
    through the operator too (its launcher keeps a workspace per stream); a workspace smaller than the
    shape needs runs unsplit."""
    M, N, K = mnk
    g = torch.Generator(device=DEV).manual_seed(K + M)
    a = torch.randint(-128, 128, (M, K), dtype=torch.int8, device=DEV, generator=g)
    b = torch.randint(-128, 128, (N, K), dtype=torch.int8, device=DEV, generator=g)
    ar = (torch.rand(M, device=DEV, generator=g) * 1e-2 + 1e-3).half()
    ac = (torch.rand(N, device=DEV, generator=g) * 1e-2 + 1e-3).half()
    need = hip_lib.fnn_gemm_a8w8_workspace_bytes(M, N, K)
    assert (need > 0) == (M < 2048) and need <= (32 << 20) + 4096
    plain = torch.empty(M, N, dtype=torch.float16, device=DEV)
    assert hip_lib.fnn_gemm_a8w8(plain.data_ptr(), a.data_ptr(), b.data_ptr(), ar.data_ptr(), ac.data_ptr(), M, N, K, K, K, N,
                                 0, 0, 0, _lib.current_stream(a.device)) == 0
    unsplit_kernel = _lib.last_kernel()
    ws = torch.empty((32 << 20) + 4096, dtype=torch.uint8, device=DEV)
    assert hip_lib.fnn_workspace_init(ws.data_ptr(), ws.numel(), _lib.current_stream(a.device)) == 0
    out = torch.empty_like(plain)
    assert _a8w8_ws_call(hip_lib, out, a, b, ar, ac, ws) == 0
    assert ("split K" in _lib.last_kernel()) == (need > 0)
    assert torch.equal(out, plain)
    via_op = flashnn_amd.GemmA8W8(torch.float16)(a, b, ar, ac)
    assert ("split K" in _lib.last_kernel()) == (need > 0) and torch.equal(via_op, plain)
    if need:
        out.zero_()
        assert _a8w8_ws_call(hip_lib, out, a, b, ar, ac, ws[:need - 16]) == 0      # a split into fewer parts, or none
        assert torch.equal(out, plain)
        out.zero_()
        assert _a8w8_ws_call(hip_lib, out, a, b, ar, ac, ws[:4096]) == 0           # room for the counters only
        assert _lib.last_kernel() == unsplit_kernel and torch.equal(out, plain)
    want = O.gemm_a8w8_epilogue_fp32(O.gemm_a8w8_acc(a[:3].cpu().numpy(), b.cpu().numpy()), O.to_np(ar[:3].cpu()),
                                     O.to_np(ac.cpu()), O.F16)
    assert np.array_equal(out[:3].float().cpu().numpy(), want)


@pytest.mark.parametrize("side", ["activations", "weights"])
def test_a8w8_operand_of_2_gib_and_more(side):
    """An operand whose last rows lie 2^31 bytes and more behind its first (a long prefill; a very wide
    head) runs on the tiled MFMA kernel in bands, not on the any-shape kernel: the rows beyond the limit
    equal, bit for bit, a call on those rows alone, both checksum identities hold over every accumulator,
    and the scaled output of the far rows equals the oracle's epilogue."""
    K, small = 8192, 384
    big = (1 << 31) // K + 300                      # rows 262144.. start beyond 2^31 bytes
    g = torch.Generator(device=DEV).manual_seed(77)
    far = torch.randint(-128, 128, (big, K), dtype=torch.int8, device=DEV, generator=g)
    near = torch.randint(-128, 128, (small, K), dtype=torch.int8, device=DEV, generator=g)
    a, b = (far, near) if side == "activations" else (near, far)
    acc = launchers.hip_gemm_a8w8_int32(a, b)
    assert _lib.last_kernel().startswith("gemm_a8w8_ring_kernel")
    tail = slice(big - 812, big)
    if side == "activations":
        assert torch.equal(acc[tail], launchers.hip_gemm_a8w8_int32(a[tail].contiguous(), b))
    else:
        assert torch.equal(acc[:, tail], launchers.hip_gemm_a8w8_int32(a, b[tail].contiguous()))
    colsum = b.sum(dim=0, dtype=torch.int64)
    rowsum = a.sum(dim=0, dtype=torch.int64)
    assert torch.equal(acc.sum(dim=1, dtype=torch.int64), (a.to(torch.int64) * colsum).sum(dim=1))
    assert torch.equal(acc.sum(dim=0, dtype=torch.int64), (b.to(torch.int64) * rowsum).sum(dim=1))
    M, N = a.shape[0], b.shape[0]
    ar = (torch.rand(M, device=DEV, generator=g) * 1e-2 + 1e-3).half()
    ac = (torch.rand(N, device=DEV, generator=g) * 1e-2 + 1e-3).float()
    out = flashnn_amd.GemmA8W8(torch.bfloat16)(a, b, ar, ac)
    ri = torch.arange(big - 5, big, device=DEV) if side == "activations" else torch.arange(0, 5, device=DEV)
    ci = torch.arange(0, 7, device=DEV) if side == "activations" else torch.arange(big - 7, big, device=DEV)
    want = O.gemm_a8w8_epilogue_fp32(acc[ri][:, ci].cpu().numpy(), O.to_np(ar[ri].cpu()), ac[ci].cpu().numpy(), O.BF16)
    assert np.array_equal(out[ri][:, ci].float().cpu().numpy(), want)


def test_foreign_hip_error_is_left_alone(hip_lib):
    """An error the caller's own HIP calls left on the thread is neither reported by a library call as its
    own nor cleared by it."""
    import ctypes
    path = next(line.split()[-1] for line in open("/proc/self/maps") if "libamdhip64" in line)
    hip = ctypes.CDLL(path)
    x = torch.randn(8, 256, device=DEV).half()
    q = torch.empty(8, 256, dtype=torch.int8, device=DEV)
    s = torch.empty(8, dtype=torch.float16, device=DEV)
    torch.cuda.synchronize()
    assert hip.hipGetLastError() == 0
    bad = hip.hipSetDevice(12345)                      # fails without touching the GPU
    assert bad != 0 and hip.hipPeekAtLastError() == bad
    rc = hip_lib.fnn_dynamic_quant(q.data_ptr(), s.data_ptr(), x.data_ptr(), 8, 256, 256, 256, 0,
                                   _lib.current_stream(x.device))
    assert rc == 0
    assert hip.hipGetLastError() == bad                 # still there; now taken off the thread
    assert hip.hipGetLastError() == 0
    torch.cuda.synchronize()
    q_o, s_o = O.dynamic_quantize(O.to_np(x.cpu()), O.F16)
    assert np.array_equal(q.cpu().numpy(), q_o) and np.array_equal(s.cpu().numpy(), s_o)


def test_first_use_log_and_kernel_names():
    """FLASHNN_HIP_LOG=1: one line on stderr per kernel variant, the first time it is launched; and
    fnn_last_kernel() names what the last call ran."""
    import os
    import subprocess
    prog = (
        "import torch, flashnn_amd\n"
        "from flashnn_amd import _lib\n"
        "x = torch.randn(64, 1024, device='cuda:0').half()\n"
        "op = flashnn_amd.DynamicQuantize()\n"
        "q, s = op(x); q, s = op(x)\n"
        "print(_lib.last_kernel())\n"
        "w = torch.randint(-128, 128, (256, 1024), dtype=torch.int8, device='cuda:0')\n"
        "flashnn_amd.GemmA8W8()(q, w, s, torch.ones(256, device='cuda:0').half())\n"
        "print(_lib.last_kernel())\n"
        "torch.cuda.synchronize()\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, FLASHNN_HIP_LOG="1", PYTHONPATH=root)
    r = subprocess.run([sys.executable, "-c", prog], env=env, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr
    lines = [l for l in r.stderr.splitlines() if l.startswith("[flashnn_hip]")]
    assert lines[0] == "[flashnn_hip] first launch of dynamic_quant_vec_kernel<1,0,0>"
    assert len(lines) == 2 and len(set(lines)) == 2
    names = r.stdout.split()
    assert names[0] == "dynamic_quant_vec_kernel<1,0,0>" and names[1] in lines[1]
    # without the variable nothing is printed
    env.pop("FLASHNN_HIP_LOG")
    r = subprocess.run([sys.executable, "-c", prog], env=env, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and "[flashnn_hip]" not in r.stderr


def test_a8w8_tuned_config_cache(tmp_path, monkeypatch):
    """With tuning on, the first launch of a shape times the candidate tiles and records the best under
    the reference's method name; the next launch (and a fresh reader of the file) uses the record; the
    result is the same bits either way."""
    import json
    from flashnn_amd import tuned_configs as TC
    path = tmp_path / "best.json"
    monkeypatch.setenv("FLASHNN_AMD_TUNED_CONFIGS", str(path))
    TC.CACHE.reset()                    # the process-wide cache reads the environment once
    M, N, K = 300, 520, 1024
    a, b = _rand_i8((M, K), 31), _rand_i8((N, K), 32)
    g = torch.Generator().manual_seed(33)
    ar, ac = (torch.rand(M, 1, generator=g) * 0.05).half(), (torch.rand(1, N, generator=g) * 0.05).half()
    op = flashnn_amd.GemmA8W8(torch.float16)
    plain = op(a.to(DEV), b.to(DEV), ar.to(DEV), ac.to(DEV)).cpu()
    assert not path.exists()
    flashnn_amd.set_autotune_triton_kernels(True)
    try:
        tuned = op(a.to(DEV), b.to(DEV), ar.to(DEV), ac.to(DEV)).cpu()
    finally:
        flashnn_amd.set_autotune_triton_kernels(False)
    data = json.load(open(path))
    assert list(data) == [f"gemm_a8w8_{M}_{N}_{K}"]
    tile = TC.deserialize_best_config(data[f"gemm_a8w8_{M}_{N}_{K}"])
    assert tile in TC.A8W8_CANDIDATES
    again = op(a.to(DEV), b.to(DEV), ar.to(DEV), ac.to(DEV)).cpu()     # from the record, tuning off
    assert torch.equal(plain, tuned) and torch.equal(plain, again)
    assert TC.TunedConfigs().lookup(f"gemm_a8w8_{M}_{N}_{K}") == tile
    assert TC.CACHE.shape_tile("gemm_a8w8", M, N, K) == tile
    monkeypatch.undo()
    TC.CACHE.reset()
    want = O.gemm_a8w8_epilogue_fp32(O.gemm_a8w8_acc(a.numpy(), b.numpy()), O.to_np(ar), O.to_np(ac), O.F16)
    assert np.array_equal(plain.float().numpy(), want)


def test_a8w8_tuned_config_with_split_k(tmp_path, monkeypatch):
    """A long-K shape with few tiles: the candidates include splits of K (met through the launcher's
    workspace); whatever wins is recorded with its SPLIT_K and used again, and every candidate - the named
    splits included - gives the bits of the plain call.  Splits the shape does not admit are skipped."""
    import json
    from flashnn_amd import tuned_configs as TC
    path = tmp_path / "best.json"
    monkeypatch.setenv("FLASHNN_AMD_TUNED_CONFIGS", str(path))
    TC.CACHE.reset()
    M, N, K = 200, 1024, 8192
    a, b = _rand_i8((M, K), 41), _rand_i8((N, K), 42)
    g = torch.Generator().manual_seed(43)
    ar, ac = (torch.rand(M, generator=g) * 0.05).half(), (torch.rand(N, generator=g) * 0.05).half()
    ad, bd, ard, acd = a.to(DEV), b.to(DEV), ar.to(DEV), ac.to(DEV)
    want = O.gemm_a8w8_epilogue_fp32(O.gemm_a8w8_acc(a.numpy(), b.numpy()), O.to_np(ar), O.to_np(ac), O.BF16)
    for cand in TC.A8W8_CANDIDATES:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        launchers.hip_gemm_a8w8_forward(out, ad, bd, ard, acd, tile=cand)
        if cand[3] > 1:
            assert _lib.last_kernel() == f"gemm_a8w8_ring_kernel(split K)<128,128,{cand[3]}>"
        assert np.array_equal(out.float().cpu().numpy(), want), cand
    with pytest.raises(_lib.FlashnnHipError):      # 64 slabs cannot make 17 parts of four
        launchers.hip_gemm_a8w8_forward(out, ad, bd, ard, acd, tile=(128, 128, 0, 17))
    op = flashnn_amd.GemmA8W8(torch.bfloat16)
    flashnn_amd.set_autotune_triton_kernels(True)
    try:
        tuned = op(ad, bd, ard, acd)
    finally:
        flashnn_amd.set_autotune_triton_kernels(False)
    entry = json.load(open(path))[f"gemm_a8w8_{M}_{N}_{K}"]
    tile = TC.deserialize_best_config(entry)
    assert tile in TC.A8W8_CANDIDATES and (tile[3] <= 1) == ("SPLIT_K" not in entry[0])
    again = op(ad, bd, ard, acd)
    assert np.array_equal(tuned.float().cpu().numpy(), want) and torch.equal(tuned, again)
    # a short K admits no split at all: the tuner skips those candidates instead of failing
    a2, b2 = _rand_i8((96, 640), 44), _rand_i8((256, 640), 45)
    flashnn_amd.set_autotune_triton_kernels(True)
    try:
        short = flashnn_amd.GemmA8W8(torch.float16)(a2.to(DEV), b2.to(DEV), ard[:96], acd[:256])
    finally:
        flashnn_amd.set_autotune_triton_kernels(False)
    want2 = O.gemm_a8w8_epilogue_fp32(O.gemm_a8w8_acc(a2.numpy(), b2.numpy()), O.to_np(ar[:96]), O.to_np(ac[:256]), O.F16)
    assert np.array_equal(short.float().cpu().numpy(), want2)
    assert TC.deserialize_best_config(json.load(open(path))["gemm_a8w8_96_256_640"])[3] <= 1
    monkeypatch.undo()
    TC.CACHE.reset()


# ------------------------------------------------------------------ mixture of experts
@pytest.mark.parametrize("out_ty", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("mul_w", [False, True])
@pytest.mark.parametrize("shape", [
    # M, E, N, K, top_k, BM
    (16, 8, 1024, 1024, 2, 16), (33, 8, 4096, 2048, 2, 32), (64, 4, 2064, 1056, 1, 64), (200, 8, 512, 1120, 2, 128),
    (7, 16, 1040, 4096, 4, 16), (3, 60, 256, 1024, 6, 16),
    # shapes of the guarded kernel: short K, block size not a multiple of 16
    (9, 4, 48, 80, 2, 16), (20, 3, 64, 1024, 2, 8)])
def test_fused_moe_a8w8_bit_exact(shape, mul_w, out_ty):
    """fused_moe_a8w8_forward against the oracle: every routed row, bit for bit; rows that the sorted
    list does not name keep the value they held."""
    M, E, N, K, top_k, BM = shape
    g = torch.Generator().manual_seed(M * 131 + E)
    a = torch.randint(-128, 128, (M, K), dtype=torch.int8, generator=g)
    b = torch.randint(-128, 128, (E, N, K), dtype=torch.int8, generator=g)
    ar = (torch.rand(M, generator=g) * 0.05).to(out_ty)
    ac = (torch.rand(E, N, generator=g) * 0.05).float()
    w, ids = torch.topk(torch.softmax(torch.randn(M, E, generator=g), -1), top_k, dim=-1)
    w = w.float().contiguous()
    s, e, used = workloads.moe_align_block_size(ids, BM, E)
    for cut in (False, True):
        if cut:                      # pretend the list ends after its first block
            used = torch.tensor([BM], dtype=torch.int32)
        c = torch.full((M, top_k, N), 3.0, dtype=out_ty)
        want = O.fused_moe_a8w8(a.numpy(), b.numpy(), c.float().reshape(M * top_k, N).numpy().copy(), O.to_np(ar),
                                ac.numpy(), w.numpy(), s.numpy(), e.numpy(), used.numpy(), mul_w, top_k, BM, _tag(out_ty))
        cd = c.to(DEV)
        got = flashnn_amd.fused_moe_a8w8_forward(a.to(DEV), b.to(DEV), cd, ar.to(DEV), ac.to(DEV), w.to(DEV), ids.to(DEV),
                                                 s.to(DEV), e.to(DEV), used.to(DEV), mul_w, top_k, BM)
        assert got is cd
        assert np.array_equal(cd.float().cpu().reshape(M * top_k, N).numpy(), want)
        if cut:
            assert (want == 3.0).any()


@pytest.mark.parametrize("out_ty", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [
    # M, E, N, K, top_k, BM, tile rows: prompt-sized batches, which take the MFMA tiles over the sorted rows
    (1024, 8, 1024, 1024, 2, 64, 64), (1500, 8, 384, 1056, 2, 128, 128), (1100, 4, 528, 2048, 2, 256, 256),
    (2048, 8, 560, 1024, 1, 64, 64), (1300, 6, 1008, 1184, 3, 192, 64), (700, 2, 144, 4096, 2, 128, 128),
    (40, 8, 272, 1024, 2, 128, 128)])
def test_fused_moe_a8w8_many_rows_bit_exact(shape, out_ty):
    """Many routed rows per expert: the tiled kernel gathers activation rows by the sorted list and scatters
    the results; bit for bit against the oracle, with and without the routing weight, also when the list is
    cut short (the tiles beyond it do nothing) and when some experts receive no rows."""
    M, E, N, K, top_k, BM, tile_rows = shape
    g = torch.Generator().manual_seed(M * 17 + E)
    a = torch.randint(-128, 128, (M, K), dtype=torch.int8, generator=g)
    b = torch.randint(-128, 128, (E, N, K), dtype=torch.int8, generator=g)
    ar = (torch.rand(M, generator=g) * 0.05).to(out_ty)
    ac = (torch.rand(E, N, generator=g) * 0.05).float()
    logits = torch.randn(M, E, generator=g)
    if E >= 6:
        logits[:, 1] = -1e9                 # an expert that nobody is routed to
    w, ids = torch.topk(torch.softmax(logits, -1), top_k, dim=-1)
    w = w.float().contiguous()
    s, e, used = workloads.moe_align_block_size(ids, BM, E)
    full = int(used[0])
    for mul_w, cut in ((True, full), (False, full), (True, (full // BM // 2) * BM)):
        used_c = torch.tensor([cut], dtype=torch.int32)
        c = torch.full((M, top_k, N), 3.0, dtype=out_ty)
        want = O.fused_moe_a8w8(a.numpy(), b.numpy(), c.float().reshape(M * top_k, N).numpy().copy(), O.to_np(ar),
                                ac.numpy(), w.numpy(), s.numpy(), e.numpy(), used_c.numpy(), mul_w, top_k, BM, _tag(out_ty))
        cd = c.to(DEV)
        flashnn_amd.fused_moe_a8w8_forward(a.to(DEV), b.to(DEV), cd, ar.to(DEV), ac.to(DEV), w.to(DEV), ids.to(DEV),
                                           s.to(DEV), e.to(DEV), used_c.to(DEV), mul_w, top_k, BM)
        assert _lib.last_kernel() == f"gemm_a8w8_ring_kernel(moe)<{tile_rows},{256 if tile_rows == 256 else 128},4>"
        assert np.array_equal(cd.float().cpu().reshape(M * top_k, N).numpy(), want)
        if cut < full:
            assert (want == 3.0).any()


@pytest.mark.parametrize("shape", [(16, 8, 1024, 1024, 2, 16), (1024, 8, 1024, 1024, 2, 64), (9, 4, 48, 80, 2, 16)])
def test_fused_moe_a8w8_strided_operands(shape):
    """Tokens, expert weights and output that are column slices of wider buffers (the launcher passes their row and
    expert strides): the bits of the call on contiguous copies, on the few-row, the tiled and the guarded kernel, and
    nothing written outside the output's columns."""
    M, E, N, K, top_k, BM = shape
    g = torch.Generator().manual_seed(M + 7)
    abuf = torch.randint(-128, 128, (M, K + 64), dtype=torch.int8, generator=g).to(DEV)
    bbuf = torch.randint(-128, 128, (E, N + 3, K + 32), dtype=torch.int8, generator=g).to(DEV)
    a, b = abuf[:, 16:16 + K], bbuf[:, 1:1 + N, 16:16 + K]
    ar = (torch.rand(M, generator=g) * 0.05).half().to(DEV)
    ac = (torch.rand(E, N, generator=g) * 0.05).float().to(DEV)
    w, ids = torch.topk(torch.softmax(torch.randn(M, E, generator=g), -1), top_k, dim=-1)
    w = w.float().contiguous()
    s_, e_, used = workloads.moe_align_block_size(ids, BM, E)
    cbuf = torch.full((M, top_k, N + 24), 3.0, dtype=torch.float16, device=DEV)
    c = cbuf[:, :, 8:8 + N]
    args = (ar, ac, w.to(DEV), ids.to(DEV), s_.to(DEV), e_.to(DEV), used.to(DEV), True, top_k, BM)
    flashnn_amd.fused_moe_a8w8_forward(a, b, c, *args)
    strided_kernel = _lib.last_kernel()
    plain = torch.full((M, top_k, N), 3.0, dtype=torch.float16, device=DEV)
    flashnn_amd.fused_moe_a8w8_forward(a.contiguous(), b.contiguous(), plain, *args)
    assert _lib.last_kernel() == strided_kernel, (strided_kernel, _lib.last_kernel())
    assert torch.equal(c, plain), strided_kernel
    assert bool((cbuf[:, :, :8] == 3).all()) and bool((cbuf[:, :, 8 + N:] == 3).all())


@pytest.mark.parametrize("act_ty", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("group,zp_kind", [(0, "float"), (0, None), (0, "int8"), (128, "float"), (128, None), (128, "int8"),
                                           (64, "int8")])
@pytest.mark.parametrize("shape", [
    # M, E, packed rows (half the output channels), K, top_k, BM
    (16, 8, 512, 1024, 2, 16), (33, 4, 1024, 2048, 2, 32), (70, 4, 528, 1152, 1, 64), (5, 16, 128, 4096, 4, 16),
    (16, 4, 256, 1056, 2, 16),     # K a multiple of 32 only (per-channel scales stay on the fast kernel)
    # the guarded kernel: short K, block size not a multiple of 16
    (9, 3, 16, 128, 2, 16), (12, 3, 32, 1024, 2, 8)])
def test_fused_moe_a16w4_close(shape, group, zp_kind, act_ty):
    """fused_moe_a16w4_forward against the oracle within the tolerance stated for 16-bit GEMM outputs;
    per-channel scales with floating zero points take the weight-streaming kernel, everything else the
    guarded one.  Rows the sorted list does not name keep their value."""
    M, E, N2, K, top_k, BM = shape
    g = torch.Generator().manual_seed(M * 17 + E + group)
    a = torch.randn(M, K, generator=g).to(act_ty)
    w = torch.randint(-8, 8, (E, 2 * N2, K), dtype=torch.int8, generator=g)
    packed = torch.stack([torch.from_numpy(O.pack_int4(w[e].numpy())) for e in range(E)])
    sshape = (E, 2 * N2) if group == 0 else (E, 2 * N2, K // group)
    scale = torch.empty(sshape).uniform_(1e-3, 1e-2, generator=g).to(act_ty)
    zp = None
    if zp_kind is not None:
        zp = torch.randint(-3, 4, sshape, generator=g)
        zp = zp.to(torch.int8) if zp_kind == "int8" else zp.to(act_ty)
    tw, ids = torch.topk(torch.softmax(torch.randn(M, E, generator=g), -1), top_k, dim=-1)
    tw = tw.float().contiguous()
    s, e, used = workloads.moe_align_block_size(ids, BM, E)
    c = torch.full((M, top_k, 2 * N2), 3.0, dtype=act_ty)
    want = O.fused_moe_a16w4(O.to_np(a), packed.numpy(), c.float().reshape(M * top_k, 2 * N2).numpy().copy(), O.to_np(scale),
                             None if zp is None else O.to_np(zp.float()), tw.numpy(), s.numpy(), e.numpy(), used.numpy(),
                             True, top_k, BM, _tag(act_ty), _tag(act_ty))
    cd = c.to(DEV)
    flashnn_amd.fused_moe_a16w4_forward(a.to(DEV), packed.to(DEV), cd, scale.to(DEV), None if zp is None else zp.to(DEV),
                                        tw.to(DEV), ids.to(DEV), s.to(DEV), e.to(DEV), used.to(DEV), True, top_k, BM)
    np.testing.assert_allclose(cd.float().cpu().reshape(M * top_k, 2 * N2).numpy(), want, rtol=RTOL, atol=ATOL)
    if (group == 0 and K >= 1024 and K % 32 == 0 or group == 128 and K % 1024 == 0) and (2 * N2) % 32 == 0 and BM % 16 == 0:
        assert _lib.last_kernel().startswith("gemm_wo_panel_kernel(moe)")      # int8 zero points included
    # the same list cut after its first block: every other routed row keeps the fill value
    cd2 = c.to(DEV)
    flashnn_amd.fused_moe_a16w4_forward(a.to(DEV), packed.to(DEV), cd2, scale.to(DEV), None if zp is None else zp.to(DEV),
                                        tw.to(DEV), ids.to(DEV), s.to(DEV), e.to(DEV),
                                        torch.tensor([BM], dtype=torch.int32, device=DEV), False, top_k, BM)
    first = [t for t in s[:BM].tolist() if t < M * top_k]
    rest = [t for t in range(M * top_k) if t not in first]
    got2 = cd2.float().cpu().reshape(M * top_k, 2 * N2)
    assert bool((got2[rest] == 3.0).all()) and not bool((got2[first] == 3.0).all())


@pytest.mark.parametrize("group", [0, 128])
@pytest.mark.parametrize("shape", [(16, 8, 512, 1024, 2, 16), (1024, 8, 256, 1024, 2, 128), (9, 3, 16, 128, 2, 16)])
def test_fused_moe_a16w4_strided_operands(shape, group):
    """Tokens, packed expert weights and output as column slices of wider buffers: the bits of the call on contiguous
    copies, on the few-row, the tiled and the guarded kernel; nothing written outside the output's columns."""
    M, E, N2, K, top_k, BM = shape
    g = torch.Generator().manual_seed(M + 11)
    abuf = torch.randn(M, K + 64, generator=g).half().to(DEV)
    bbuf = torch.randint(-128, 128, (E, N2 + 3, K + 32), dtype=torch.int8, generator=g).to(DEV)
    a, b = abuf[:, 8:8 + K], bbuf[:, 2:2 + N2, 16:16 + K]
    sshape = (E, 2 * N2) if group == 0 else (E, 2 * N2, K // group)
    scale = torch.empty(sshape).uniform_(1e-3, 1e-2, generator=g).half().to(DEV)
    zp = torch.randint(-3, 4, sshape, generator=g).half().to(DEV)
    tw, ids = torch.topk(torch.softmax(torch.randn(M, E, generator=g), -1), top_k, dim=-1)
    tw = tw.float().contiguous()
    s_, e_, used = workloads.moe_align_block_size(ids, BM, E)
    cbuf = torch.full((M, top_k, 2 * N2 + 24), 3.0, dtype=torch.float16, device=DEV)
    c = cbuf[:, :, 8:8 + 2 * N2]
    args = (scale, zp, tw.to(DEV), ids.to(DEV), s_.to(DEV), e_.to(DEV), used.to(DEV), True, top_k, BM)
    flashnn_amd.fused_moe_a16w4_forward(a, b, c, *args)
    strided_kernel = _lib.last_kernel()
    plain = torch.full((M, top_k, 2 * N2), 3.0, dtype=torch.float16, device=DEV)
    flashnn_amd.fused_moe_a16w4_forward(a.contiguous(), b.contiguous(), plain, *args)
    assert _lib.last_kernel() == strided_kernel, (strided_kernel, _lib.last_kernel())
    assert torch.equal(c, plain), strided_kernel
    assert bool((cbuf[:, :, :8] == 3).all()) and bool((cbuf[:, :, 8 + 2 * N2:] == 3).all())


@pytest.mark.parametrize("act_ty", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("zp_kind", ["float", None])
@pytest.mark.parametrize("group", [0, 128])
@pytest.mark.parametrize("shape", [
    # M, E, packed rows (half the output channels), K, top_k, BM, tile rows
    (1024, 8, 256, 1024, 2, 128, 128), (1100, 4, 192, 2048, 2, 256, 256), (40, 8, 128, 1280, 2, 128, 128),
    (1500, 6, 64, 4096, 1, 384, 128)])
def test_fused_moe_a16w4_many_rows_close(shape, group, zp_kind, act_ty):
    """Many routed rows per expert, tables per channel or per group of 128: the tiled MFMA kernel gathers
    activation rows by the sorted list and scatters the results; the tolerance of 16-bit GEMM outputs against
    the oracle, with the routing weight and without, the list whole and cut short, one expert without rows."""
    M, E, N2, K, top_k, BM, tile_rows = shape
    g = torch.Generator().manual_seed(M * 19 + E)
    a = torch.randn(M, K, generator=g).to(act_ty)
    w = torch.randint(-8, 8, (E, 2 * N2, K), dtype=torch.int8, generator=g)
    packed = torch.stack([torch.from_numpy(O.pack_int4(w[e].numpy())) for e in range(E)])
    sshape = (E, 2 * N2) if group == 0 else (E, 2 * N2, K // group)
    scale = torch.empty(sshape).uniform_(1e-3, 1e-2, generator=g).to(act_ty)
    zp = None if zp_kind is None else torch.randint(-3, 4, sshape, generator=g).to(act_ty)
    logits = torch.randn(M, E, generator=g)
    if E >= 6:
        logits[:, 1] = -1e9
    tw, ids = torch.topk(torch.softmax(logits, -1), top_k, dim=-1)
    tw = tw.float().contiguous()
    s, e, used = workloads.moe_align_block_size(ids, BM, E)
    full = int(used[0])
    for mul_w, cut in ((True, full), (False, full), (True, (full // BM // 2) * BM)):
        used_c = torch.tensor([cut], dtype=torch.int32)
        c = torch.full((M, top_k, 2 * N2), 3.0, dtype=act_ty)
        want = O.fused_moe_a16w4(O.to_np(a), packed.numpy(), c.float().reshape(M * top_k, 2 * N2).numpy().copy(),
                                 O.to_np(scale), None if zp is None else O.to_np(zp.float()), tw.numpy(), s.numpy(),
                                 e.numpy(), used_c.numpy(), mul_w, top_k, BM, _tag(act_ty), _tag(act_ty))
        cd = c.to(DEV)
        flashnn_amd.fused_moe_a16w4_forward(a.to(DEV), packed.to(DEV), cd, scale.to(DEV), None if zp is None else zp.to(DEV),
                                            tw.to(DEV), ids.to(DEV), s.to(DEV), e.to(DEV), used_c.to(DEV), mul_w, top_k, BM)
        assert _lib.last_kernel() == (f"gemm_wo_tile_kernel(moe)<4,{tile_rows},128>" if group == 0 else
                                      "gemm_wo_tile_kernel(moe, group tables)<4,128,128>")
        got = cd.float().cpu().reshape(M * top_k, 2 * N2).numpy()
        bad = np.abs(got - want) > ATOL + RTOL * np.abs(want)
        if bad.any():
            # tables per group: the reference rounds every dequantised weight to the table type, this kernel
            # scales each group's sum in fp32 - the bounded allowance of the weight-only tests, by the same rule
            assert group == 128 and bad.mean() <= BREACH_SHARE[_tag(act_ty)], f"{int(bad.sum())} of {bad.size}"
            exact = O.fused_moe_a16w4(O.to_np(a), packed.numpy(), c.float().reshape(M * top_k, 2 * N2).numpy().copy(),
                                      O.to_np(scale), None if zp is None else O.to_np(zp.float()), tw.numpy(), s.numpy(),
                                      e.numpy(), used_c.numpy(), mul_w, top_k, BM, _tag(act_ty), O.F32)
            assert (np.abs(got[bad] - exact[bad]) <= np.abs(want[bad] - exact[bad])).all()
        if cut < full:
            # rows the cut list does not name keep the fill value, all others are written
            assert (want == 3.0).all(axis=1).any() and np.array_equal((got == 3.0).all(axis=1), (want == 3.0).all(axis=1))


# ------------------------------------------------------------------ weight-only GEMM
def _wo_inputs(M, N, K, group, bits, act_ty, scale_ty, with_zp, with_bias, seed):
    g = torch.Generator().manual_seed(seed)
    act = torch.randn(M, K, generator=g).to(act_ty)
    lo, hi = (-128, 128) if bits == 8 else (-8, 8)
    w = torch.randint(lo, hi, (N, K), generator=g, dtype=torch.int8)
    sshape = (N,) if group == 0 else (K // group, N)
    scale = torch.empty(sshape).uniform_(1e-3, 1e-2, generator=g).to(scale_ty)
    zp = torch.randint(lo // 2, hi // 2, sshape, generator=g).to(scale_ty) if with_zp else None
    bias = torch.randn(N, generator=g).to(act_ty) if with_bias else None
    qw = w if bits == 8 else torch.from_numpy(O.pack_int4(w.numpy()))
    return act, w, qw, scale, zp, bias


WO_BREACHES = []   # (case, outputs beyond the stated tolerance, outputs) of the cases that had any

# The kernels that scale channel or group sums in fp32 where the reference rounds every dequantised weight to
# the table type (flashnn/quant_gemm.py:14-36).  The reference's rounding moves an output by about
# 2^-11 |w| sqrt(K) (2^-8 with bf16 tables), which on outputs near zero of long dot products exceeds
# rtol = atol = 1e-2 although the kernel is the more accurate of the two.  Only these kernels may leave the
# stated tolerance, only on a bounded share of the outputs, and only towards the float64 value; every kernel
# that says it rounds per weight - the tiled kernel for more than 64 rows (fp16 tables, or bf16 tables with bf16
# activations) and the few-row kernels with per-channel tables of the activations' type (fp16; bf16 over int8
# weights) - is held to the tolerance without exception.
FP32_SCALING_KERNELS = {"gemm_wo_panel_kernel", "gemm_wo_stream_kernel", "gemm_wo_any_kernel", "gemm_wo_decode_kernel",
                        "gemm_wo_decode_lds_kernel", "gemm_wo_gemv_kernel", "gemm_wo_gemv_flat_kernel",
                        "gemm_wo_tile_kernel"}
BREACH_SHARE = {"f16": 0.005, "bf16": 0.10, "f32": 0.005}     # by table type


def _wo_check(act, w, qw, scale, zp, bias, group, bits, out_ty, strict=False, cols=None):
    """The stated tolerance, unscaled: |got - oracle| <= 1e-2 + 1e-2 |oracle|, the oracle being the reference's
    torch path with its per-weight rounding of the dequantised weights to the table type (fp16 for group
    tables).  A kernel that rounds the same way (it says so in its name, or the caller passes `strict`) must
    keep every output inside.  The kernels listed in FP32_SCALING_KERNELS may leave it on at most
    BREACH_SHARE of the outputs, each of which must then be at least as close to the float64 value as the
    oracle's is; the cases and counts are reported.  `cols` (indices): the oracle is worked out for these
    channels only (wide matrices)."""
    d = lambda t: None if t is None else t.to(DEV)
    out = flashnn_amd.GemmWeightOnly(out_ty)(d(act), d(qw), d(scale), d(bias), d(zp))
    assert out.dtype == out_ty and out.shape == (act.shape[0], w.shape[0])
    kernel = _lib.last_kernel()
    strict = strict or "per-weight rounding" in kernel
    got = out.float().cpu().numpy()
    if cols is not None:
        got, w = got[:, cols], w[cols]
        scale = scale[..., cols]
        zp = None if zp is None else zp[..., cols]
        bias = None if bias is None else bias[cols]
    n = lambda t: None if t is None else O.to_np(t)
    want = O.weight_only_gemm(n(act), w.numpy(), n(scale), n(zp), n(bias), _tag(scale.dtype), _tag(out_ty),
                              group, bits == 4)
    exact = O.weight_only_gemm_f64(n(act), w.numpy(), n(scale), n(zp), n(bias), group)
    tol = ATOL + RTOL * np.abs(want)
    if bits == 8 and bias is not None:
        # the reference's int8 branch rounds the product to the output type before it adds the bias
        # (flashnn/quant_gemm.py:168-173), and so do the kernels; a product whose fp32 sum, added in another
        # order, falls on the other side of a rounding boundary then differs by one step of the output type at
        # the product's magnitude, which shows where product and bias nearly cancel
        product = np.abs(want - O.to_np(bias).astype(np.float32)[None, :])
        tol = tol + (2.0 ** -7 if out_ty == torch.bfloat16 else 2.0 ** -10) * product
    bad = np.abs(got - want) > tol
    if bad.any():
        import os
        case = os.environ.get("PYTEST_CURRENT_TEST", "?").split(" ")[0]
        WO_BREACHES.append((f"{case} [{kernel}; act {_tag(act.dtype)}, tables {_tag(scale.dtype)}, "
                            f"M={act.shape[0]} N={w.shape[0]} K={act.shape[1]} group={group}]", int(bad.sum()), bad.size))
        assert not strict, f"{int(bad.sum())} outputs beyond the stated tolerance on a reference-rounding path ({kernel})"
        assert kernel.split("<")[0] in FP32_SCALING_KERNELS, kernel
        assert bad.mean() <= BREACH_SHARE[_tag(scale.dtype)], f"{bad.mean():.4f} of the outputs beyond the tolerance ({kernel})"
        assert (np.abs(got[bad] - exact[bad]) <= np.abs(want[bad] - exact[bad])).all()
    # ... and as close to the mathematical value as one output rounding (and fp32 accumulation) allows
    spread = max(1.0, float(np.sqrt(np.mean(want.astype(np.float64) ** 2))))
    ulp = 2.0 ** -9 if out_ty == torch.float16 else 2.0 ** -6
    # (the reference's rounding itself moves an output by about 2^-11 |w| sqrt(K); with bf16 tables by 2^-8 |w| sqrt(K))
    slack = (2e-3 if not strict else 8e-3 if scale.dtype != torch.bfloat16 else 6.4e-2) * spread
    assert (np.abs(got - exact) <= np.abs(exact) * ulp + slack).all()


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("group", [0, 64, 128])
@pytest.mark.parametrize("M", [1, 3, 8, 16, 17, 33, 64, 70])
def test_weight_only_small(bits, group, M):
    act_ty = torch.float16 if M % 2 else torch.bfloat16
    case = _wo_inputs(M, 96, 512, group, bits, act_ty, torch.float16, with_zp=bool(M & 1), with_bias=bool(M & 2), seed=M)
    _wo_check(*case, group, bits, act_ty)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("act_ty,scale_ty", [(torch.float16, torch.float32), (torch.bfloat16, torch.bfloat16),
                                             (torch.bfloat16, torch.float16)])
def test_weight_only_dtypes_and_edges(bits, act_ty, scale_ty):
    # N not a multiple of the tile, K = 64 (fewer steps than waves), zero points and bias
    case = _wo_inputs(5, 50, 64, 0, bits, act_ty, scale_ty, True, True, seed=3)
    _wo_check(*case, 0, bits, act_ty)
    case = _wo_inputs(2, 1024, 4096, 64, bits, act_ty, scale_ty, True, False, seed=4)
    _wo_check(*case, 64, bits, act_ty)
    # shapes the streaming kernel does not take (K % 64 != 0, group 32): guarded kernel
    case = _wo_inputs(3, 24, 96, 32, bits, act_ty, scale_ty, True, True, seed=5)
    _wo_check(*case, 32, bits, act_ty)


def test_weight_only_reference_test_shape():
    """M, N, K = 3, 1024, 4096 fp16, int8 weights, bias / sub-channel(64) / asymmetric sweeps
    (tests/quant_gemm/test_gemm_weight_only.py:160-181)."""
    for group in (0, 64):
        for with_zp in (False, True):
            for with_bias in (False, True):
                case = _wo_inputs(3, 1024, 4096, group, 8, torch.float16, torch.float16, with_zp, with_bias, seed=9)
                _wo_check(*case, group, 8, torch.float16, strict=True)
                assert _lib.last_kernel().startswith("gemm_wo_decode_lds_kernel(per-weight rounding)"), _lib.last_kernel()


@pytest.mark.parametrize("bits,group,M,N,K,kernel", [
    (8, 0, 2, 4096, 4096, "gemm_wo_decode_lds_kernel"), (8, 0, 4, 4096, 4096, "gemm_wo_decode_lds_kernel"),
    (4, 128, 4, 8192, 2048, "gemm_wo_decode_lds_kernel"), (4, 0, 3, 2048, 1024, "gemm_wo_decode_lds_kernel"),
    (8, 128, 2, 2048, 8192, "gemm_wo_decode_lds_kernel"),
    (8, 0, 4, 4608, 1024, "gemm_wo_panel_kernel"),          # more than 4096 weight rows
    (8, 0, 3, 2048, 8192, "gemm_wo_panel_kernel"),          # three rows of 8192 values do not fit the LDS copy
    (8, 0, 5, 4096, 4096, "gemm_wo_panel_kernel"),          # five rows
    (4, 128, 4, 8704, 1024, "gemm_wo_panel_kernel")])
def test_weight_only_two_to_four_rows_over_few_weight_rows(bits, group, M, N, K, kernel):
    """2 to 4 activation rows over at most 4096 weight rows run on the decode kernel where its LDS copy of the
    activations fits, on the panel kernel otherwise; both round alike."""
    for act_ty in (torch.float16, torch.bfloat16):
        case = _wo_inputs(M, N, K, group, bits, act_ty, torch.float16, True, M == 2, seed=300 + M)
        _wo_check(*case, group, bits, act_ty, cols=np.r_[0:128, N - 128:N])
        assert _lib.last_kernel().startswith(kernel), _lib.last_kernel()
        assert ("per-weight rounding" in _lib.last_kernel()) == (group == 0 and act_ty == torch.float16), _lib.last_kernel()


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("group", [32, 64])
@pytest.mark.parametrize("M,N,K", [(1, 1024, 4096), (3, 1024, 4096), (8, 520, 1152), (5, 4096, 2944), (2, 96, 128)])
def test_weight_only_small_groups_decode(bits, group, M, N, K):
    """Tables per group of 32 or 64 with fp16 activations and tables: every weight is dequantised and rounded to
    fp16 as the reference's block dequantisation does, so the stated tolerance holds without exception."""
    for with_zp in (False, True):
        case = _wo_inputs(M, N, K, group, bits, torch.float16, torch.float16, with_zp, M == 3, seed=M + K)
        _wo_check(*case, group, bits, torch.float16, strict=True)
        assert _lib.last_kernel().startswith("gemm_wo_decode_lds_kernel")


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("group", [0, 128])
@pytest.mark.parametrize("M,K", [(9, 1024), (16, 2048), (33, 1024), (64, 2048), (100, 1024)])
def test_weight_only_many_rows(bits, group, M, K):
    """9 .. 100 activation rows over >= 8192 weight rows: the kernel that shares activation slabs
    between four weight tiles (one, two and four 16-row blocks per pass, one and two passes)."""
    N = 8192 * (2 if bits == 4 else 1)
    act_ty = torch.float16 if M % 2 else torch.bfloat16
    scale_ty = torch.bfloat16 if M == 33 else torch.float16
    case = _wo_inputs(M, N, K, group, bits, act_ty, scale_ty, with_zp=M != 16, with_bias=M in (9, 64), seed=M)
    _wo_check(*case, group, bits, act_ty)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("group", [0, 128])
@pytest.mark.parametrize("M,N8,K", [(5, 1024, 1152), (20, 2048, 1024), (40, 1040, 2304), (33, 6400, 1280)])
def test_weight_only_many_rows_small_matrices(bits, group, M, N8, K):
    """Few weight rows: 16- and 32-row workgroups, K parts that differ by one slab (K = 9, 18 and 10
    slabs of 128 over 8 or 4 parts), several passes over the activation rows."""
    N = N8 * (2 if bits == 4 else 1)
    act_ty = torch.float16 if M % 2 else torch.bfloat16
    case = _wo_inputs(M, N, K, group, bits, act_ty, torch.float16, with_zp=M != 20, with_bias=M == 5, seed=100 + M)
    _wo_check(*case, group, bits, act_ty)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("M", [1, 5, 33, 70])
@pytest.mark.parametrize("N8,K", [(1024, 1056), (512, 7392), (2064, 1120), (256, 8896)])
def test_weight_only_partial_last_slab(bits, M, N8, K):
    """Per-channel scales with K a multiple of 32 but not of 128 (K = 7392, 8896: the FFN shapes of models
    sharded over 4 or 8 GPUs): the last 128-k slab holds 32, 64 or 96 values.  Zero points and bias on."""
    N = N8 * (2 if bits == 4 else 1)
    act_ty = torch.float16 if M % 2 else torch.bfloat16
    case = _wo_inputs(M, N, K, 0, bits, act_ty, torch.float16, with_zp=True, with_bias=M == 5, seed=300 + M)
    _wo_check(*case, 0, bits, act_ty)


def test_weight_only_partial_last_slab_one_hot():
    """One-hot activation rows whose single entry lies in the partial last slab, or just before it, pick
    single weight columns exactly; an entry of ones shows that nothing beyond K is added."""
    M, N, K = 6, 512, 1120          # 8 slabs of 128 + 96
    act = torch.zeros(M, K, dtype=torch.float16)
    cols = [1023, 1024, 1055, 1056, 1119]
    for i, c in enumerate(cols):
        act[i, c] = 1.0
    act[5] = 1.0
    g = torch.Generator().manual_seed(7)
    w = torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=g)
    scale = torch.ones(N, dtype=torch.float16)
    out = flashnn_amd.GemmWeightOnly(torch.float16)(act.to(DEV), w.to(DEV), scale.to(DEV)).float().cpu()
    for i, c in enumerate(cols):
        assert torch.equal(out[i], w[:, c].float())
    assert torch.equal(out[5], w.float().sum(dim=1).half().float())


def test_weight_only_many_rows_one_hot():
    """Rows of the activation matrix that hold a single non-zero entry pick single weight columns:
    checks the k order inside the slabs and the row -> output mapping exactly."""
    M, N, K = 48, 16384, 2048
    g = torch.Generator().manual_seed(77)
    w = torch.randint(-8, 8, (N, K), generator=g, dtype=torch.int8)
    scale = torch.empty(K // 128, N).uniform_(1e-3, 1e-2, generator=g).half()
    zp = torch.randint(-4, 4, (K // 128, N), generator=g).half()
    ks = torch.randperm(K, generator=g)[:M]
    act = torch.zeros(M, K, dtype=torch.float16)
    act[torch.arange(M), ks] = 2.0
    qw = torch.from_numpy(O.pack_int4(w.numpy()))
    out = flashnn_amd.GemmWeightOnly(torch.float16)(act.to(DEV), qw.to(DEV), scale.to(DEV), None, zp.to(DEV))
    want = 2.0 * (w[:, ks].float() - zp[ks // 128].float().t()) * scale[ks // 128].float().t()   # [N, M]
    np.testing.assert_allclose(out.float().cpu().numpy(), want.t().half().float().numpy(), rtol=2.0 ** -10, atol=1e-6)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("group", [0, 128])
@pytest.mark.parametrize("M,N,K", [(65, 16512, 512), (128, 16512, 1024), (200, 8320, 2560), (256, 16512, 768), (300, 8320, 1536),
                                   (520, 5632, 512)])
def test_weight_only_tiled_large_m(bits, group, M, N, K):
    """More than 64 activation rows on matrices wide enough for more than 128 tiles: the tiled MFMA kernel (128-
    and 256-row tiles, a partial last row tile, 2 to 20 slabs: every position of the two- and three-stage
    rings), zero points, bias, fp16 and bf16 activations and tables; the oracle on three bands of channels."""
    act_ty = torch.float16 if M in (65, 200, 300) else torch.bfloat16
    scale_ty = torch.bfloat16 if M in (300, 520) else torch.float16      # (520: bf16 rows with bf16 tables)
    case = _wo_inputs(M, N, K, group, bits, act_ty, scale_ty, with_zp=M != 128, with_bias=M in (65, 256), seed=700 + M)
    cols = np.r_[0:64, N // 2 - 32:N // 2 + 32, N - 64:N]
    _wo_check(*case, group, bits, act_ty, cols=cols)
    assert _lib.last_kernel().startswith("gemm_wo_tile_kernel"), _lib.last_kernel()
    # activations and tables of one 16-bit type: every weight rounded as the reference rounds it
    assert ("per-weight rounding" in _lib.last_kernel()) == (M != 300), _lib.last_kernel()


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("group", [0, 128])
@pytest.mark.parametrize("M,N,K", [(65, 256, 512), (128, 384, 1024), (200, 128, 2560), (256, 512, 768), (300, 256, 1536),
                                   (520, 128, 512), (512, 4096, 1024)])
def test_weight_only_large_m_on_narrow_matrices(bits, group, M, N, K):
    """More than 64 activation rows where the tiled kernel would have 128 tiles or fewer: 64-row passes of the
    panel kernel, as many as the rows need."""
    act_ty = torch.float16 if (M + N) % 256 else torch.bfloat16
    scale_ty = torch.bfloat16 if M == 300 else torch.float16
    case = _wo_inputs(M, N, K, group, bits, act_ty, scale_ty, with_zp=M != 128, with_bias=M in (65, 256), seed=700 + M)
    _wo_check(*case, group, bits, act_ty, cols=None if N <= 512 else np.r_[0:64, N - 64:N])
    # (the panel kernel wants at least 1024 values of K: shorter rows stay on the tiled kernel)
    assert _lib.last_kernel().startswith("gemm_wo_panel_kernel" if K >= 1024 else "gemm_wo_tile_kernel"), _lib.last_kernel()


@pytest.mark.parametrize("M,N,want", [(64, 17792, "<8,2,4>"), (24, 22016, "<8,2,4>"), (48, 37888, "<8,2,4>"), (64, 16384, "<8,4,4>"),
                                      (64, 27648, "<8,4,4>"), (16, 17792, "<8,1,4>")])
def test_a16w8_a_little_more_than_one_round_of_64_row_workgroups(M, N, want):
    """int8 weights, more than 16 rows, 257 .. 384 or 513 .. 640 workgroups of 64 weight rows: passes of 32 activation
    rows (two workgroups share a CU) instead of one pass of 64; the neighbouring shapes keep the model's choice."""
    case = _wo_inputs(M, N, 1024, 128, 8, torch.bfloat16, torch.float16, with_zp=True, with_bias=False, seed=M + N)
    _wo_check(*case, 128, 8, torch.bfloat16, cols=np.r_[0:64, N // 2 - 32:N // 2 + 32, N - 64:N])
    assert _lib.last_kernel() == "gemm_wo_panel_kernel" + want, _lib.last_kernel()


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("group", [64, 256, 512])
@pytest.mark.parametrize("M,N,K", [(5, 1024, 1024), (16, 4096, 2048), (40, 1056, 2560), (64, 8192, 1024), (100, 2048, 1536),
                                   (200, 8320, 2560), (300, 512, 4096)])
def test_weight_only_groups_of_64_256_512(bits, group, M, N, K):
    """Tables per group of 64 (two groups per 128-value slab, each half folded with its own table row) and of 256
    or 512 values (a table row serves 2 or 4 slabs) on the MFMA kernels: the panel kernel up to 64 rows and in
    64-row passes, the tiled kernel on wide matrices with groups of 256 and 512."""
    if K % group:
        K = (K // group) * group
    act_ty = torch.float16 if M % 16 else torch.bfloat16
    scale_ty = torch.bfloat16 if M == 40 else torch.float16
    case = _wo_inputs(M, N, K, group, bits, act_ty, scale_ty, with_zp=M != 16, with_bias=M in (5, 200), seed=900 + M + group)
    _wo_check(*case, group, bits, act_ty, cols=None if N <= 1056 else np.r_[0:64, N // 2 - 32:N // 2 + 32, N - 64:N])
    tiled = M > 64 and group != 64 and N == 8320
    # (groups of 64 with up to 8 rows, fp16 throughout, stay on the kernel that rounds per weight as the reference does)
    want_kernel = "gemm_wo_tile_kernel" if tiled else "gemm_wo_decode_lds_kernel" if (group, M) == (64, 5) else "gemm_wo_panel_kernel"
    assert _lib.last_kernel().startswith(want_kernel), _lib.last_kernel()


@pytest.mark.parametrize("group,M,N", [(64, 48, 4096), (256, 48, 4096), (512, 24, 2048), (64, 150, 1024), (256, 200, 16640), (512, 130, 16640)])
def test_weight_only_group_rows_one_hot(group, M, N):
    """One-hot activation rows pick single weight columns, each scaled by the table row of its own group: a table
    row taken from a neighbouring group shows as a wrong scale or zero point (tables differ from group to group)."""
    K = 2048
    g = torch.Generator().manual_seed(group + M)
    w = torch.randint(-8, 8, (N, K), generator=g, dtype=torch.int8)
    scale = torch.empty(K // group, N).uniform_(1e-3, 1e-2, generator=g).half()
    zp = torch.randint(-4, 4, (K // group, N), generator=g).half()
    ks = torch.randperm(K, generator=g)[:M]
    ks[:4] = torch.tensor([0, group - 1, group, K - 1])
    act = torch.zeros(M, K, dtype=torch.float16)
    act[torch.arange(M), ks] = 2.0
    qw = torch.from_numpy(O.pack_int4(w.numpy()))
    out = flashnn_amd.GemmWeightOnly(torch.float16)(act.to(DEV), qw.to(DEV), scale.to(DEV), None, zp.to(DEV))
    assert _lib.last_kernel().startswith("gemm_wo_tile_kernel" if N == 16640 else "gemm_wo_panel_kernel"), _lib.last_kernel()
    want = 2.0 * (w[:, ks].float() - zp[ks // group].float().t()) * scale[ks // group].float().t()   # [N, M]
    np.testing.assert_allclose(out.float().cpu().numpy(), want.t().half().float().numpy(), rtol=2.0 ** -10, atol=1e-6)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("act_ty,scale_ty", [(torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
                                             (torch.bfloat16, torch.float16)])
@pytest.mark.parametrize("M,N,K", [(3, 1024, 1024), (9, 1024, 4096), (20, 520, 1152), (70, 256, 2944), (200, 96, 512)])
def test_weight_only_groups_of_32_many_rows(bits, M, N, K, act_ty, scale_ty):
    """Tables per group of 32 beyond the decode kernel's reach (more than 8 rows, or bf16 somewhere): the stream
    kernel's form whose two MFMAs of a 64-value step cover one group each, in 64-row passes."""
    case = _wo_inputs(M, N, K, 32, bits, act_ty, scale_ty, True, M == 20, seed=M + K)
    _wo_check(*case, 32, bits, act_ty)
    small_fp16 = M <= 8 and act_ty == torch.float16
    assert _lib.last_kernel().startswith("gemm_wo_decode_lds_kernel" if small_fp16 else "gemm_wo_stream_kernel"), _lib.last_kernel()


def test_weight_only_groups_of_32_one_hot():
    """One-hot rows pick single weight columns, each with the table row of its own group of 32."""
    M, N, K, group = 40, 256, 1024, 32
    g = torch.Generator().manual_seed(32)
    w = torch.randint(-8, 8, (N, K), generator=g, dtype=torch.int8)
    scale = torch.empty(K // group, N).uniform_(1e-3, 1e-2, generator=g).half()
    zp = torch.randint(-4, 4, (K // group, N), generator=g).half()
    ks = torch.randperm(K, generator=g)[:M]
    ks[:6] = torch.tensor([0, 31, 32, 63, 64, K - 1])
    act = torch.zeros(M, K, dtype=torch.float16)
    act[torch.arange(M), ks] = 2.0
    qw = torch.from_numpy(O.pack_int4(w.numpy()))
    out = flashnn_amd.GemmWeightOnly(torch.float16)(act.to(DEV), qw.to(DEV), scale.to(DEV), None, zp.to(DEV))
    assert _lib.last_kernel().startswith("gemm_wo_stream_kernel"), _lib.last_kernel()
    want = 2.0 * (w[:, ks].float() - zp[ks // group].float().t()) * scale[ks // group].float().t()   # [N, M]
    np.testing.assert_allclose(out.float().cpu().numpy(), want.t().half().float().numpy(), rtol=2.0 ** -10, atol=1e-6)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("group", [0, 128, 256, 1024])
def test_weight_only_bf16_rows_through_the_conversion_pass(hip_lib, bits, group):
    """bf16 activations, fp16 tables, more than 64 rows: with scratch memory the rows become fp16 rows (scaled
    by a power of two per row) and the tiled kernel rounds every weight as the reference does - no output
    may leave the tolerance, with rows of magnitudes from 1e-20 to 1e20 among ordinary ones; the same call
    without scratch runs the fp32-scaling kernel and stays within the tolerance of the first."""
    M, N, K = 200, 8320, 2048           # 130 tiles: the tiled kernel's side of the dispatch
    act, w, qw, scale, zp, bias = _wo_inputs(M, N, K, group, bits, torch.bfloat16, torch.float16, True, True, seed=911)
    cols = np.r_[0:64, N // 2 - 32:N // 2 + 32, N - 64:N]
    act = act.float()
    act[3] *= 1e20          # far beyond fp16's range
    act[5] *= 1e-20         # far below it
    act[7] = 0.0
    act[9, ::2] *= 3e4
    act = act.bfloat16()
    d = lambda t: t.to(DEV)
    out = flashnn_amd.GemmWeightOnly(torch.bfloat16)(d(act), d(qw), d(scale), d(bias), d(zp))
    assert _lib.last_kernel().startswith("gemm_wo_tile_kernel(per-weight rounding)")
    got = out.float().cpu().numpy()
    want = O.weight_only_gemm(O.to_np(act), w[cols].numpy(), O.to_np(scale[..., cols]), O.to_np(zp[..., cols]), O.to_np(bias[cols]),
                              O.F16, O.BF16, group, bits == 4)
    got, want = got.astype(np.float64), want.astype(np.float64)
    scale_of_row = np.maximum(1.0, np.abs(want).max(axis=1, keepdims=True) / 50.0)      # rows of 1e20 have outputs of 1e20
    # (int8: one bf16 step at the product's magnitude on top, as in _wo_check: the product is rounded before the bias is added)
    step = 2.0 ** -7 * np.abs(want - O.to_np(bias[cols]).astype(np.float64)[None, :]) if bits == 8 else 0.0
    assert (np.abs(got[:, cols] - want) <= (ATOL + RTOL * np.abs(want)) * scale_of_row + step).all()
    assert not got[7].any() or np.allclose(got[7], O.to_np(bias).astype(np.float32), atol=1e-2)
    # the plain entry point (no scratch): the fp32-scaling kernel, within the tolerance of the reference-rounding one
    plain = torch.empty_like(out)
    fn = hip_lib.fnn_gemm_a16w4 if bits == 4 else hip_lib.fnn_gemm_a16w8
    a_d, q_d, s_d, z_d, b_d = d(act), d(qw), d(scale), d(zp), d(bias)
    rc = fn(plain.data_ptr(), a_d.data_ptr(), q_d.data_ptr(), s_d.data_ptr(), b_d.data_ptr(), z_d.data_ptr(), M, N, K, K, K, N,
            group, 1, 1, 0, 0, _lib.dtype_code(b_d.dtype), _lib.current_stream(a_d.device))
    assert rc == 0 and _lib.last_kernel().startswith("gemm_wo_tile_kernel<")
    p_np = plain.float().cpu().numpy().astype(np.float64)
    step_all = 2.0 ** -7 * np.abs(got - O.to_np(bias).astype(np.float64)[None, :]) if bits == 8 else 0.0
    assert (np.abs(p_np - got) <= (2 * ATOL + 2 * RTOL * np.abs(got)) * scale_of_row + step_all).all()
    need = hip_lib.fnn_gemm_weight_only_workspace_bytes(M, N, K, group, 1, 0)
    assert need == (M * K * 2 + 255) // 256 * 256 + 4 * M
    assert hip_lib.fnn_gemm_weight_only_workspace_bytes(64, N, K, group, 1, 0) == 0        # few rows: other kernels
    assert hip_lib.fnn_gemm_weight_only_workspace_bytes(M, N, K, group, 0, 0) == 0         # fp16 rows need no conversion
    assert hip_lib.fnn_gemm_weight_only_workspace_bytes(M, N, K, group, 1, 1) == 0         # bf16 tables: fp32 scaling
    # scratch that is too small, or not 16-byte aligned, is not used: the call still succeeds, on the fp32-scaling kernel
    fn_ws = hip_lib.fnn_gemm_a16w4_ws if bits == 4 else hip_lib.fnn_gemm_a16w8_ws
    ws = torch.empty(need + 16, dtype=torch.uint8, device=DEV)
    for ptr, size, kernel in ((ws.data_ptr(), need - 1, "gemm_wo_tile_kernel<"), (ws.data_ptr() + 8, need, "gemm_wo_tile_kernel<"),
                              (ws.data_ptr(), need, "gemm_wo_tile_kernel(per-weight rounding)")):
        again = torch.zeros_like(out)
        rc = fn_ws(again.data_ptr(), a_d.data_ptr(), q_d.data_ptr(), s_d.data_ptr(), b_d.data_ptr(), z_d.data_ptr(), M, N, K, K, K, N,
                   group, 1, 1, 0, 0, _lib.dtype_code(b_d.dtype), ptr, size, _lib.current_stream(a_d.device))
        assert rc == 0 and _lib.last_kernel().startswith(kernel), (size, _lib.last_kernel())
        assert torch.equal(again, plain if "rounding" not in kernel else out)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("group", [0, 128])
@pytest.mark.parametrize("kind", ["whole", "quarter", "one_fraction", "large"])
@pytest.mark.parametrize("ty", [torch.float16, torch.bfloat16])
def test_weight_only_tiled_zero_points_whole_or_not(bits, group, kind, ty):
    """The tiled kernel's per-weight rounding takes offset and zero point in one step where every zero point of
    the tile is a whole number of moderate size, and in two otherwise; both must be the reference's rounding: whole
    zero points, quarters, a single fractional one in one tile, and whole ones too large for the short form; fp16
    activations with fp16 tables (packed fp16 arithmetic) and bf16 with bf16 (fp32 arithmetic, rounded to bf16)."""
    M, N, K = 200, 8320, 1024
    act, w, qw, scale, zp, bias = _wo_inputs(M, N, K, group, bits, ty, ty, True, False, seed=321)
    if kind == "quarter":
        zp = (zp.float() + 0.25).to(ty)
    elif kind == "one_fraction":
        zp = zp.clone()
        zp[..., 4200] = 1.5
    elif kind == "large":
        zp = zp.clone()
        zp[..., 100] = 600.0
    cols = np.r_[0:256, 4096:4352, N - 64:N]
    if kind != "large":
        _wo_check(act, w, qw, scale, zp, bias, group, bits, ty, strict=True, cols=cols)
    else:
        # (a zero point of 600 makes outputs of the size of 600 * scale * sum(a): the oracle's own rounding is then
        # further from the mathematical value than _wo_check's closeness bound allows, so only the tolerance is held)
        d = lambda t: t.to(DEV)
        got = flashnn_amd.GemmWeightOnly(ty)(d(act), d(qw), d(scale), None, d(zp)).float().cpu().numpy()[:, cols]
        want = O.weight_only_gemm(O.to_np(act), w[cols].numpy(), O.to_np(scale[..., cols]), O.to_np(zp[..., cols]), None,
                                  _tag(ty), _tag(ty), group, bits == 4)
        assert (np.abs(got - want) <= ATOL + RTOL * np.abs(want)).all()
    assert _lib.last_kernel().startswith("gemm_wo_tile_kernel(per-weight rounding)"), _lib.last_kernel()


def _close_to(got, want, out_ty):
    """Two fp32 summation orders of one dot product, each rounded once to the output type."""
    got, want = got.float().cpu().numpy(), want.float().cpu().numpy()
    step = 2.0 ** -7 if out_ty == torch.bfloat16 else 2.0 ** -10
    rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    return (np.abs(got - want) <= step * np.abs(want) + 1e-3 * rms).all()


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("group", [0, 128])
def test_weight_only_named_blocks(bits, group):
    """Every pair of blocks of the few-row kernel, named through the `_tiled` entry points, gives the result of the
    library's own choice up to the order of the fp32 additions, on the kernel variant it names; pairs the shape does
    not divide into, more than 64 rows, and a call whose default path rounds differently are refused."""
    from flashnn_amd import tuned_configs as TC
    M, N, K = 40, 2048, 2048
    act_ty = torch.float16 if group == 0 else torch.bfloat16
    act, w, qw, scale, zp, bias = _wo_inputs(M, N, K, group, bits, act_ty, torch.float16, True, True, seed=77)
    d = lambda t: t.to(DEV)
    fwd = launchers.hip_gemm_a16w8_forward if bits == 8 else launchers.hip_gemm_a16w4_forward
    plain = torch.empty(M, N, dtype=act_ty, device=DEV)
    fwd(plain, d(act), d(qw), d(scale), d(bias), d(zp))
    assert _lib.last_kernel().startswith("gemm_wo_panel_kernel"), _lib.last_kernel()
    rounding = "(per-weight rounding)" in _lib.last_kernel()
    cands = TC.weight_only_candidates(2 if bits == 4 else 1)
    assert cands[0] == (0, 0, 0, 0) and len(cands) == 7
    for cand in cands[1:]:
        out = torch.full((M, N), float("nan"), dtype=act_ty, device=DEV)
        fwd(out, d(act), d(qw), d(scale), d(bias), d(zp), tile=cand)
        mb, rt = cand[0] // 16, cand[1] // (16 * (2 if bits == 4 else 1))
        assert _lib.last_kernel() == f"gemm_wo_panel_kernel{'(per-weight rounding)' if rounding else ''}<{bits},{mb},{rt}>", (cand, _lib.last_kernel())
        assert _close_to(out, plain, act_ty), cand
    out = torch.empty(M, N, dtype=act_ty, device=DEV)
    for bad in ((48, 64), (16, 24), (64, 32 * (2 if bits == 4 else 1)), (16, 256)):     # not built: rows above the tile's, odd sizes
        with pytest.raises(_lib.FlashnnHipError):
            fwd(out, d(act), d(qw), d(scale), d(bias), d(zp), tile=bad)
    # weight rows that do not divide into 64-row tiles
    n2 = 48 * (2 if bits == 4 else 1)
    out2 = torch.empty(M, n2, dtype=act_ty, device=DEV)
    rows = n2 // (2 if bits == 4 else 1)
    with pytest.raises(_lib.FlashnnHipError):
        fwd(out2, d(act), d(qw[:rows]), d(scale[..., :n2].contiguous()), None, None, tile=cands[1])
    fwd(out2, d(act), d(qw[:rows]), d(scale[..., :n2].contiguous()), None, None, tile=cands[-1])   # 16-row tiles do
    # more than 64 rows
    act65 = torch.randn(65, K).to(act_ty)
    with pytest.raises(_lib.FlashnnHipError):
        fwd(torch.empty(65, N, dtype=act_ty, device=DEV), d(act65), d(qw), d(scale), None, None, tile=cands[1])


def test_weight_only_named_blocks_never_change_the_rounding():
    """Groups of 64 with up to 8 fp16 rows run on the decode kernel, which rounds every weight as the reference does;
    the few-row kernel would scale in fp32, so its blocks cannot be named for such a call."""
    M, N, K = 4, 1024, 2048
    act, w, qw, scale, zp, bias = _wo_inputs(M, N, K, 64, 8, torch.float16, torch.float16, True, False, seed=78)
    d = lambda t: t.to(DEV)
    out = torch.empty(M, N, dtype=torch.float16, device=DEV)
    with pytest.raises(_lib.FlashnnHipError):
        launchers.hip_gemm_a16w8_forward(out, d(act), d(qw), d(scale), None, d(zp), tile=(16, 64))
    launchers.hip_gemm_a16w8_forward(out, d(act), d(qw), d(scale), None, d(zp))
    assert "per-weight rounding" in _lib.last_kernel(), _lib.last_kernel()


def test_weight_only_tuned_config_cache(tmp_path, monkeypatch):
    """With tuning on, the first weight-only launch of a shape with up to 64 rows times the block pairs of the few-row
    kernel and records the best under the name of the reference's kernel for the call; the next launch, and a fresh
    reader of the file, use the record; more than 64 rows are not tuned."""
    import json
    from flashnn_amd import tuned_configs as TC
    path = tmp_path / "best.json"
    monkeypatch.setenv("FLASHNN_AMD_TUNED_CONFIGS", str(path))
    TC.CACHE.reset()
    M, N, K = 24, 4096, 2048
    d = lambda t: None if t is None else t.to(DEV)
    try:
        for bits, group, name in ((8, 0, f"gemm_a16w8_per_channel_{M}_{N}_{K}"), (4, 128, f"gemm_a16w4_sub_channel_g128_{M}_{N}_{K}")):
            act, w, qw, scale, zp, bias = _wo_inputs(M, N, K, group, bits, torch.bfloat16, torch.float16, True, False, seed=79)
            op = flashnn_amd.GemmWeightOnly(torch.bfloat16)
            plain = op(d(act), d(qw), d(scale), None, d(zp))
            flashnn_amd.set_autotune_triton_kernels(True)
            try:
                tuned = op(d(act), d(qw), d(scale), None, d(zp))
            finally:
                flashnn_amd.set_autotune_triton_kernels(False)
            data = json.load(open(path))
            assert name in data, list(data)
            tile = TC.deserialize_best_config(data[name])
            assert tile in TC.weight_only_candidates(2 if bits == 4 else 1)
            again = op(d(act), d(qw), d(scale), None, d(zp))
            if tile[0]:
                assert _lib.last_kernel().endswith(f"<{bits},{tile[0] // 16},{tile[1] // (16 * (2 if bits == 4 else 1))}>"), _lib.last_kernel()
            assert _close_to(tuned, plain, torch.bfloat16) and _close_to(again, plain, torch.bfloat16)
            assert TC.TunedConfigs().lookup(name) == tile
        n_records = len(json.load(open(path)))
        act, w, qw, scale, zp, bias = _wo_inputs(80, 1024, 1024, 0, 8, torch.float16, torch.float16, False, False, seed=80)
        flashnn_amd.set_autotune_triton_kernels(True)
        try:
            flashnn_amd.GemmWeightOnly(torch.float16)(d(act), d(qw), d(scale), None, None)
        finally:
            flashnn_amd.set_autotune_triton_kernels(False)
        assert len(json.load(open(path))) == n_records
    finally:
        monkeypatch.undo()
        TC.CACHE.reset()


@pytest.mark.parametrize("M", [1, 3, 8, 9, 33, 64])
@pytest.mark.parametrize("kind", ["none", "whole", "quarter", "large"])
def test_a16w8_bf16_tables_round_per_weight(M, kind):
    """int8 weights under bf16 rows with per-channel bf16 tables, 1 to 64 rows: the decode and panel kernels round
    every weight to bf16 as the reference does (fp32 arithmetic), in one step where the zero points of a wave's rows are
    whole, in two where one is fractional or large - chosen per wave, so the single large one leaves the rest on the
    short form."""
    N, K = 1024, 2048
    bf = torch.bfloat16
    act, w, qw, scale, zp, bias = _wo_inputs(M, N, K, 0, 8, bf, bf, kind != "none", M == 8, seed=900 + M)
    if kind == "quarter":
        zp = (zp.float() + 0.25).to(bf)
    elif kind == "large":
        zp = zp.clone()
        zp[100] = 600.0
    if kind != "large":
        _wo_check(act, w, qw, scale, zp, bias, 0, 8, bf, strict=True)
    else:
        # (outputs of the size of 600 * scale * sum(a): only the tolerance is held, as in the tiled kernel's test)
        d = lambda t: None if t is None else t.to(DEV)
        got = flashnn_amd.GemmWeightOnly(bf)(d(act), d(qw), d(scale), d(bias), d(zp)).float().cpu().numpy()
        want = O.weight_only_gemm(O.to_np(act), w.numpy(), O.to_np(scale), O.to_np(zp), None if bias is None else O.to_np(bias),
                                  O.BF16, O.BF16, 0, False)
        assert (np.abs(got - want) <= ATOL + RTOL * np.abs(want) + 2.0 ** -7 * np.abs(want)).all()
    assert "per-weight rounding" in _lib.last_kernel(), _lib.last_kernel()


@pytest.mark.parametrize("M", [4, 16])
def test_a16w8_bf16_one_hot_few_rows(M):
    """One-hot bf16 rows pick single int8 weights: each output is twice bf16((q - zp) * scale), bit for bit (decode
    kernel at 4 rows, panel kernel at 16)."""
    N, K = 512, 1024
    g = torch.Generator().manual_seed(79)
    bf = torch.bfloat16
    w = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
    scale = torch.empty(N).uniform_(1e-3, 1e-2, generator=g).to(bf)
    zp = torch.randint(-64, 64, (N,), generator=g).to(bf)
    ks = torch.randint(0, K, (M,), generator=g)
    act = torch.zeros(M, K, dtype=bf)
    act[torch.arange(M), ks] = 2.0
    out = flashnn_amd.GemmWeightOnly(bf)(act.to(DEV), w.to(DEV), scale.to(DEV), None, zp.to(DEV))
    assert "per-weight rounding" in _lib.last_kernel(), _lib.last_kernel()
    want = 2.0 * ((w[:, ks].float() - zp.float()[:, None]) * scale.float()[:, None]).to(bf).float()   # [N, M]
    assert torch.equal(out.float().cpu(), want.t().contiguous())


@pytest.mark.parametrize("ty", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits", [4, 8])
def test_weight_only_tiled_one_hot(bits, ty):
    """One-hot activation rows pick single weight columns exactly: the k order inside a slab, the row and
    channel mapping of the tiled kernel (group 128; 130 tiles), in the fp16 and in the bf16 form of the per-weight
    rounding: a weight is (q - zp) * scale rounded once to the table type (the zero points are whole), and twice
    that is the output without a further rounding."""
    M, N, K = 160, 8320, 1024
    g = torch.Generator().manual_seed(78)
    lo = 8 if bits == 4 else 128
    w = torch.randint(-lo, lo, (N, K), generator=g, dtype=torch.int8)
    scale = torch.empty(K // 128, N).uniform_(1e-3, 1e-2, generator=g).to(ty)
    zp = torch.randint(-lo // 2, lo // 2, (K // 128, N), generator=g).to(ty)
    ks = torch.randint(0, K, (M,), generator=g)
    act = torch.zeros(M, K, dtype=ty)
    act[torch.arange(M), ks] = 2.0
    qw = torch.from_numpy(O.pack_int4(w.numpy())) if bits == 4 else w
    out = flashnn_amd.GemmWeightOnly(ty)(act.to(DEV), qw.to(DEV), scale.to(DEV), None, zp.to(DEV))
    assert "per-weight rounding" in _lib.last_kernel(), _lib.last_kernel()
    want = 2.0 * ((w[:, ks].float() - zp[ks // 128].float().t()) * scale[ks // 128].float().t()).to(ty).float()   # [N, M]
    assert torch.equal(out.float().cpu(), want.t().contiguous())


@pytest.mark.parametrize("M", [1, 8, 32])
@pytest.mark.parametrize("kn", workloads.A16W8_DECODE_SHAPES)
def test_a16w8_decode_config(M, kn):
    K, N = kn
    act = workloads.activations(M, K, torch.float16, seed=31)
    w, s32 = workloads.int8_weights(N, K, seed=32)
    scale = s32.half()
    # fp16 activations, per-channel fp16 scales: the kernels round every weight as the reference does
    _wo_check(act, w, w, scale, None, None, 0, 8, torch.float16, strict=True)


@pytest.mark.parametrize("M", [1, 4, 16, 64, 256])
def test_a16w4_group128_config(M):
    """K=8192, N=28672, group 128, uint4 weights with uint4 zero points, bf16: checked on a
    band of output channels against the oracle (the whole matrix is too slow on the CPU)
    and through linearity on the rest: out(act) for act = e_k * c picks one weight column."""
    K, N = workloads.A16W4_SHAPE
    packed, scale, zp_ref, u, zp = workloads.int4_group_weights(N, K, 128)
    act = workloads.activations(M, K, torch.bfloat16, seed=41)
    out = flashnn_amd.GemmWeightOnly(torch.bfloat16)(act.to(DEV), packed.to(DEV), scale.to(DEV), None, zp_ref.to(DEV))
    assert out.shape == (M, N)
    bands = [slice(0, 64), slice(14336 - 32, 14336 + 32), slice(N - 64, N)]
    for band in bands:
        w_band = u[band].numpy().astype(np.int16) - 8
        want = O.weight_only_gemm(O.to_np(act), w_band, O.to_np(scale[:, band]), O.to_np(zp_ref[:, band]), None,
                                  O.F16, O.BF16, 128, True)
        np.testing.assert_allclose(out[:, band].float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    # one-hot activation: out[0, n] = c * (u[n,k] - zp[k/128,n]) * scale[k/128,n] for every n
    k = 4321
    e = torch.zeros(1, K, dtype=torch.bfloat16)
    e[0, k] = 2.0
    o1 = flashnn_amd.GemmWeightOnly(torch.bfloat16)(e.to(DEV), packed.to(DEV), scale.to(DEV), None, zp_ref.to(DEV))
    col = 2.0 * (u[:, k].float() - zp[k // 128].float()) * scale[k // 128].float()
    np.testing.assert_allclose(o1[0].float().cpu().numpy(), col.bfloat16().float().numpy(), rtol=2.0 ** -7, atol=1e-6)


def test_a16w4_prepacked_decode_config(hip_lib):
    """The one-token decode on repacked weights at K=8192, N=28672: the device's repacking equals the
    oracle's packed form byte for byte; the output stays within the tolerance of the oracle on three
    bands of channels, equals a one-hot probe of every channel, and agrees with the reference-layout
    kernel everywhere to the same tolerance."""
    K, N = workloads.A16W4_SHAPE
    packed, scale, zp_ref, u, zp = workloads.int4_group_weights(N, K, 128)
    op = flashnn_amd.GemmWeightOnly(torch.bfloat16)
    pk = op.prepack(packed.to(DEV), scale.to(DEV), zp_ref.to(DEV))
    assert pk.buffer.numel() == hip_lib.fnn_a16w4_prepacked_bytes(N, K, 128) == N * K // 2 + 4 * (K // 128) * N
    rows = slice(0, 64)                  # 128 channels = 8 tiles of the packed form, all of K
    want_pk = O.prepack_a16w4(packed[rows].numpy(), O.to_np(scale[:, :128]), O.to_np(zp_ref[:, :128]))
    assert np.array_equal(pk.buffer[:want_pk.size].cpu().numpy(), want_pk)
    last = O.prepack_a16w4(packed[-8:].numpy(), O.to_np(scale[:, -16:]), O.to_np(zp_ref[:, -16:]))
    assert np.array_equal(pk.buffer[-last.size:].cpu().numpy(), last)
    act = workloads.activations(1, K, torch.bfloat16, seed=41)
    out = op.forward_prepacked(act.to(DEV), pk)
    assert _lib.last_kernel().startswith("gemv_w4_prepacked_kernel") and out.shape == (1, N)
    for band in [slice(0, 64), slice(14336 - 32, 14336 + 32), slice(N - 64, N)]:
        w_band = u[band].numpy().astype(np.int16) - 8
        want = O.weight_only_gemm(O.to_np(act), w_band, O.to_np(scale[:, band]), O.to_np(zp_ref[:, band]), None,
                                  O.F16, O.BF16, 128, True)
        np.testing.assert_allclose(out[:, band].float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    ref_layout = op(act.to(DEV), packed.to(DEV), scale.to(DEV), None, zp_ref.to(DEV))
    np.testing.assert_allclose(out.float().cpu().numpy(), ref_layout.float().cpu().numpy(), rtol=RTOL, atol=ATOL)
    k = 4321
    e = torch.zeros(1, K, dtype=torch.bfloat16)
    e[0, k] = 2.0
    o1 = op.forward_prepacked(e.to(DEV), pk)
    col = 2.0 * (u[:, k].float() - zp[k // 128].float()) * scale[k // 128].float()
    np.testing.assert_allclose(o1[0].float().cpu().numpy(), col.bfloat16().float().numpy(), rtol=2.0 ** -7, atol=1e-6)


@pytest.mark.parametrize("N,K,act_ty,with_zp,with_bias", [(16, 1024, torch.float16, True, False), (48, 2048, torch.bfloat16, True, True),
                                                         (4096, 4096, torch.float16, False, True), (1040, 8192, torch.bfloat16, True, False),
                                                         (12288, 11264, torch.float16, True, True), (8208, 16384, torch.bfloat16, True, False)])
def test_a16w4_prepacked_shapes(hip_lib, N, K, act_ty, with_zp, with_bias):
    """Other shapes of the packed decode: one to eleven K ranges (fewer ranges than waves: the waves split
    the tiles; more: a wave walks several), tile counts that leave workgroups ragged, fp16 and bf16
    activations with a wide range of magnitudes, with and without zero points and bias - against the
    oracle, and the repacking against the oracle's byte for byte."""
    g = torch.Generator().manual_seed(N + K)
    w = torch.randint(-8, 8, (N, K), generator=g, dtype=torch.int8)
    scale = torch.empty(K // 128, N).uniform_(1e-3, 1e-2, generator=g).half()
    zp = torch.randint(-8, 8, (K // 128, N), generator=g).half() if with_zp else None
    bias = torch.randn(N, generator=g).to(act_ty) if with_bias else None
    act = torch.randn(1, K, generator=g)
    act[0, ::7] *= 300.0                 # a wide range of magnitudes inside every K range
    act[0, 5::64] *= 1e-3
    act = act.to(act_ty)
    qw = torch.from_numpy(O.pack_int4(w.numpy()))
    op = flashnn_amd.GemmWeightOnly(act_ty)
    pk = op.prepack(qw.to(DEV), scale.to(DEV), None if zp is None else zp.to(DEV))
    want_pk = O.prepack_a16w4(qw.numpy(), O.to_np(scale), None if zp is None else O.to_np(zp))
    assert np.array_equal(pk.buffer.cpu().numpy(), want_pk)
    out = op.forward_prepacked(act.to(DEV), pk, None if bias is None else bias.to(DEV))
    cols = slice(0, N) if N * K <= 1 << 24 else slice(N - 512, N)
    want = O.weight_only_gemm(O.to_np(act), w[cols].numpy(), O.to_np(scale[:, cols]), None if zp is None else O.to_np(zp[:, cols]),
                              None if bias is None else O.to_np(bias[cols]), O.F16, O.tag_of(act), 128, True)
    got = out[:, cols].float().cpu().numpy()
    # (activations up to 1000 make outputs of the order of 10^3: the tolerance is the relative one)
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL * max(1.0, float(np.abs(want).max()) / 50))
    full = op(act.to(DEV), qw.to(DEV), scale.to(DEV), None if bias is None else bias.to(DEV), None if zp is None else zp.to(DEV))
    np.testing.assert_allclose(out.float().cpu().numpy(), full.float().cpu().numpy(), rtol=RTOL,
                               atol=ATOL * max(1.0, float(full.float().abs().max()) / 50))


def test_a16w4_prepacked_argument_errors(hip_lib):
    """Shapes without a packed form and calls with more than one row are refused, not served wrongly."""
    f = hip_lib.fnn_a16w4_prepacked_bytes
    assert f(28672, 8192, 128) == 28672 * 8192 // 2 + 4 * 64 * 28672
    assert f(28672, 8192, 64) == 0 and f(28680, 8192, 128) == 0 and f(4096, 4224, 128) == 0 and f(4096, 3072, 128) == 0
    qw = torch.zeros(8, 1024, dtype=torch.int8, device=DEV)
    scale = torch.ones(8, 16, dtype=torch.float16, device=DEV)
    pk = flashnn_amd.GemmWeightOnly.prepack(qw, scale)
    with pytest.raises(AssertionError):
        flashnn_amd.GemmWeightOnly.prepack(qw, scale.bfloat16())
    # rows whose stride is not a multiple of 16 bytes are refused before anything is launched
    act = torch.zeros(2, 1028, dtype=torch.float16, device=DEV)
    out = torch.full((2, 16), 3.0, dtype=torch.float16, device=DEV)
    rc = hip_lib.fnn_gemm_a16w4_prepacked(_lib.ptr(out), _lib.ptr(act), _lib.ptr(pk.buffer), None, 2, 16, 1024, 1028, 16, 128,
                                          _lib.FNN_F16, _lib.FNN_F16, 0, _lib.current_stream(out.device))
    torch.cuda.synchronize()
    assert rc != 0 and b"16-byte aligned" in hip_lib.fnn_last_error() and bool((out == 3.0).all())


@pytest.mark.parametrize("M,N,K,act_ty,with_zp,with_bias", [
    (2, 28672, 8192, torch.bfloat16, True, False),      # 7 tiles per workgroup, 16-row pass with 2 rows in use
    (16, 28672, 8192, torch.float16, True, True),
    (17, 14336, 8192, torch.bfloat16, True, False),     # 4 tiles per workgroup, 32-row pass
    (32, 28672, 8192, torch.bfloat16, False, False),
    (33, 4096, 4096, torch.float16, True, True),        # one tile per workgroup, 64-row pass, 4 waves
    (64, 28672, 8192, torch.bfloat16, True, False),
    (100, 8192, 2048, torch.bfloat16, True, True),      # two passes of 64 rows, 2 tiles per workgroup
    (5, 8208, 16384, torch.float16, True, False),       # tiles that leave the last workgroup short, 16 ranges
    (48, 1040, 9216, torch.bfloat16, True, True),       # an odd number of ranges (one left over behind the loop)
    (3, 16, 1024, torch.float16, False, True),          # one tile, one range
    (20, 48, 2048, torch.bfloat16, True, False),
    (130, 27696, 11264, torch.float16, True, False),    # three passes; 1731 tiles: the last workgroup has 2 of 7
])
def test_a16w4_prepacked_rows(hip_lib, M, N, K, act_ty, with_zp, with_bias):
    """More than one row on the packed weights: every tile count and row block the kernel is built for,
    ranges left over behind its unrolled loop, short last workgroups, rows of very different magnitudes
    (one of them all zero) - against the oracle on a band of channels and against the reference-layout
    kernels everywhere."""
    g = torch.Generator().manual_seed(M * 7 + N + K)
    w = torch.randint(-8, 8, (N, K), generator=g, dtype=torch.int8)
    scale = torch.empty(K // 128, N).uniform_(1e-3, 1e-2, generator=g).half()
    zp = torch.randint(-8, 8, (K // 128, N), generator=g).half() if with_zp else None
    bias = torch.randn(N, generator=g).to(act_ty) if with_bias else None
    act = torch.randn(M, K, generator=g)
    act[:, ::7] *= 30.0
    act[0] *= 100.0
    act[M - 1] *= 1e-3
    if M > 2:
        act[1] = 0.0
    act = act.to(act_ty)
    qw = torch.from_numpy(O.pack_int4(w.numpy()))
    op = flashnn_amd.GemmWeightOnly(act_ty)
    pk = op.prepack(qw.to(DEV), scale.to(DEV), None if zp is None else zp.to(DEV))
    out = op.forward_prepacked(act.to(DEV), pk, None if bias is None else bias.to(DEV))
    assert _lib.last_kernel().startswith("gemm_w4_prepacked_rows_kernel") and out.shape == (M, N)
    ncol = min(N, max(16, (1 << 24) // (M * K) // 16 * 16))
    cols = slice(N - ncol, N)
    want = O.weight_only_gemm(O.to_np(act), w[cols].numpy(), O.to_np(scale[:, cols]), None if zp is None else O.to_np(zp[:, cols]),
                              None if bias is None else O.to_np(bias[cols]), O.F16, O.tag_of(act), 128, True)
    got = out[:, cols].float().cpu().numpy()
    # per row: the tolerance is relative to the row's own scale (rows differ by five orders of magnitude)
    row_scale = np.maximum(1.0, np.abs(want).max(axis=1, keepdims=True) / 50)
    assert np.all(np.abs(got - want) <= RTOL * np.abs(want) + ATOL * row_scale), float(np.abs(got - want).max())
    full = op(act.to(DEV), qw.to(DEV), scale.to(DEV), None if bias is None else bias.to(DEV), None if zp is None else zp.to(DEV))
    f = full.float().cpu().numpy()
    o = out.float().cpu().numpy()
    row_scale = np.maximum(1.0, np.abs(f).max(axis=1, keepdims=True) / 50)
    assert np.all(np.abs(o - f) <= RTOL * np.abs(f) + ATOL * row_scale), float(np.abs(o - f).max())
    if M > 2:
        zero_row = out[1].float().cpu().numpy()
        assert np.array_equal(zero_row, np.zeros(N, np.float32) if bias is None else bias.float().numpy())


@pytest.mark.parametrize("act_ty", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [9, 24, 50, 70])
@pytest.mark.parametrize("tiles_per_wg,K", [(1, 2048), (2, 1024), (4, 2048), (7, 4096)])
def test_a16w4_prepacked_rows_every_build(hip_lib, tiles_per_wg, K, M, act_ty):
    """Every build of the rows kernel on packed weights (1, 2, 4 or 7 tiles per workgroup x 16, 32 or 64 rows
    per pass, one pass or two x fp16 or bf16 rows): the output against the oracle on the last 64 channels and
    against the reference-layout kernels on all of them."""
    N = 16 * 256 * tiles_per_wg
    g = torch.Generator().manual_seed(N + K + M)
    w = torch.randint(-8, 8, (N, K), generator=g, dtype=torch.int8)
    scale = torch.empty(K // 128, N).uniform_(1e-3, 1e-2, generator=g).half()
    zp = torch.randint(-8, 8, (K // 128, N), generator=g).half()
    act = torch.randn(M, K, generator=g).to(act_ty)
    qw = torch.from_numpy(O.pack_int4(w.numpy()))
    op = flashnn_amd.GemmWeightOnly(act_ty)
    pk = op.prepack(qw.to(DEV), scale.to(DEV), zp.to(DEV))
    out = op.forward_prepacked(act.to(DEV), pk)
    kernel = _lib.last_kernel()
    assert kernel == f"gemm_w4_prepacked_rows_kernel<{1 if M <= 16 else 2 if M <= 32 else 4},{tiles_per_wg},{(M + 63) // 64}>", kernel
    cols = slice(N - 64, N)
    want = O.weight_only_gemm(O.to_np(act), w[cols].numpy(), O.to_np(scale[:, cols]), O.to_np(zp[:, cols]), None,
                              O.F16, O.tag_of(act), 128, True)
    np.testing.assert_allclose(out[:, cols].float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    full = op(act.to(DEV), qw.to(DEV), scale.to(DEV), None, zp.to(DEV))
    np.testing.assert_allclose(out.float().cpu().numpy(), full.float().cpu().numpy(), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("bits,M,N,K", [(4, 1, 24576, 8192), (4, 2, 24576, 8192), (4, 3, 20480, 8192), (4, 4, 28672, 8192),
                                        (8, 1, 12288, 8192), (4, 2, 28672, 4096), (4, 1, 16384, 8192)])
def test_weight_only_gemv_equal_chunks(bits, M, N, K):
    """Up to four rows over many channels with group 128: a workgroup's tiles x K steps are cut into eight
    equal chunks, one per wave, and a chunk covers the end of one tile and the beginning of the next
    (5, 6 and 7 tiles per workgroup; 4 tiles: two chunks per tile; K = 4096: the one-wave-per-tile kernel).
    Bands of channels at the seams against the oracle, zero points and bias on."""
    g = torch.Generator().manual_seed(500 + M + N)
    act_ty = torch.bfloat16 if M % 2 else torch.float16
    act = torch.randn(M, K, generator=g).to(act_ty)
    lo, hi = (-128, 128) if bits == 8 else (-8, 8)
    w = torch.randint(lo, hi, (N, K), generator=g, dtype=torch.int8)
    scale = torch.empty(K // 128, N).uniform_(1e-3, 1e-2, generator=g).half()
    zp = torch.randint(lo // 2, hi // 2, (K // 128, N), generator=g).half()
    bias = torch.randn(N, generator=g).to(act_ty)
    qw = w if bits == 8 else torch.from_numpy(O.pack_int4(w.numpy()))
    out = flashnn_amd.GemmWeightOnly(act_ty)(act.to(DEV), qw.to(DEV), scale.to(DEV), bias.to(DEV), zp.to(DEV))
    got = out.float().cpu().numpy()
    per_tile = 16 if bits == 4 else 8
    tiles = N // per_tile
    wpw = -(-tiles // 256)
    # the first workgroups' tiles (every seam between chunks), one workgroup in the middle, the last one
    for first in (0, (tiles // wpw // 2) * wpw, tiles - wpw):
        band = slice(first * per_tile, (first + wpw) * per_tile)
        want = O.weight_only_gemm(O.to_np(act), w[band].numpy(), O.to_np(scale[:, band]), O.to_np(zp[:, band]),
                                  O.to_np(bias[band]), O.F16, _tag(act_ty), 128, bits == 4)
        exact = O.weight_only_gemm_f64(O.to_np(act), w[band].numpy(), O.to_np(scale[:, band]), O.to_np(zp[:, band]),
                                       O.to_np(bias[band]), 128)
        bad = np.abs(got[:, band] - want) > ATOL + RTOL * np.abs(want)
        assert (np.abs(got[:, band][bad] - exact[bad]) <= np.abs(want[bad] - exact[bad])).all()
        ulp = 2.0 ** -9 if act_ty == torch.float16 else 2.0 ** -6
        spread = max(1.0, float(np.sqrt(np.mean(want.astype(np.float64) ** 2))))
        assert (np.abs(got[:, band] - exact) <= np.abs(exact) * ulp + 2e-3 * spread).all()


@pytest.mark.parametrize("bits,M,N,K,group", [(4, 1, 4096, 16384, 128), (4, 3, 2048, 16384, 128), (8, 1, 1024, 16384, 128),
                                              (8, 2, 1024, 16384, 0), (4, 8, 2048, 14336, 128)])
def test_weight_only_long_rows_within_the_lds_limit(bits, M, N, K, group):
    """Decode shapes whose staged activations would push a launch past 64 KB of dynamic LDS: the call succeeds
    (the dispatch passes such a shape to a kernel that fits or raises that kernel's limit first) and the
    result is right."""
    act, w, qw, scale, zp, bias = _wo_inputs(M, N, K, group, bits, torch.float16, torch.float16, True, False, 93)
    _wo_check(act, w, qw, scale, zp, bias, group, bits, torch.float16)
    assert _lib.last_kernel().startswith("gemm_wo_")


# ------------------------------------------------------- rmsnorm+quant -> A8W8 chain
@pytest.mark.parametrize("bits,N,K,group,act_ty", [(4, 2048, 28672, 128, torch.bfloat16), (8, 1024, 18944, 0, torch.float16),
                                                  (8, 1024, 18944, 128, torch.bfloat16), (4, 1024, 17408, 0, torch.float16),
                                                  (8, 12288, 1280, 0, torch.float16), (8, 15360, 3584, 0, torch.bfloat16)])
def test_weight_only_one_row_on_the_panel_kernel(bits, N, K, group, act_ty):
    """One activation row where the decode kernels are the slower choice: rows longer than their LDS copy of the
    activations holds (K > 16864), and int8 weights with per-channel tables over 12288 and more channels with
    K / 128 not a multiple of 32."""
    case = _wo_inputs(1, N, K, group, bits, act_ty, torch.float16, with_zp=True, with_bias=bits == 8, seed=N + K)
    _wo_check(*case, group, bits, act_ty, cols=None if N <= 2048 else np.r_[0:64, N // 2 - 32:N // 2 + 32, N - 64:N])
    assert _lib.last_kernel().startswith("gemm_wo_panel_kernel"), _lib.last_kernel()


@pytest.mark.parametrize("M", [1, 32, 512, 8192])
def test_rmsnorm_quant_gemm_chain(M):
    K = N = 8192
    h = workloads.activations(M, K, torch.bfloat16, seed=51, outlier_frac=0.01)
    gamma = workloads.rmsnorm_gamma(K)
    w, ws = workloads.int8_weights(N, K, seed=52)
    norm = flashnn_amd.RMSNormDquant(K, eps=1e-6).to(DEV)
    norm.weight.data = gamma.to(DEV)
    q, s = norm(h.to(DEV))
    out = flashnn_amd.GemmA8W8(torch.bfloat16)(q, w.to(DEV), s, ws.to(DEV))
    q_o, s_o = O.rmsnorm_dquant(O.to_np(h), gamma.numpy(), 1e-6, O.BF16)
    assert np.array_equal(q.cpu().numpy(), q_o) and np.array_equal(s.float().cpu().numpy(), s_o)
    rows = np.unique(np.linspace(0, M - 1, min(M, 24)).astype(int))
    acc_all = launchers.hip_gemm_a8w8_int32(q, w.to(DEV))
    acc = acc_all[torch.from_numpy(rows).to(DEV)].cpu().numpy()
    assert np.array_equal(acc, O.gemm_a8w8_acc(q_o[rows], w.numpy()))
    # every accumulator, through sum_n acc[m, n] = q[m, :] . sum_n w[n, :] in exact integers
    colsum = w.numpy().astype(np.int64).sum(axis=0)
    assert np.array_equal(acc_all.sum(dim=1, dtype=torch.int64).cpu().numpy(), q_o.astype(np.int64) @ colsum)
    # ... and sum_m acc[m, n] = (sum_m q[m, :]) . w[n, :]
    rowsum = torch.from_numpy(q_o.astype(np.int64).sum(axis=0)).to(DEV)
    assert torch.equal(acc_all.sum(dim=0, dtype=torch.int64), (w.to(DEV).to(torch.int64) * rowsum).sum(dim=1))
    want = O.gemm_a8w8(q_o[rows], w.numpy(), s_o[rows], ws.numpy(), O.BF16)
    np.testing.assert_allclose(out[torch.from_numpy(rows).to(DEV)].float().cpu().numpy(), want, rtol=RTOL, atol=ATOL)


# ------------------------------------------- rmsnorm, layernorm, layernorm + quant
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 128), (3, 64, 64), (7, 1000), (33, 4096), (16, 8192), (5, 50), (2, 16384), (3, 20000),
                                   (2, 35584), (1, 40960)])
@pytest.mark.parametrize("w_dtype", ["same", torch.float32])
def test_rmsnorm_bit_exact(dtype, shape, w_dtype):
    g = torch.Generator().manual_seed(21)
    K = shape[-1]
    x = torch.randn(shape, generator=g).to(dtype)
    w = torch.empty(K).uniform_(0.5, 1.5, generator=g).to(dtype if w_dtype == "same" else w_dtype)
    mod = flashnn_amd.RMSNorm(K, eps=1e-5)
    mod.weight.data = w
    out = mod.to(DEV)(x.to(DEV))
    assert out.dtype == dtype and out.shape == x.shape
    want = O.rmsnorm(O.to_np(x), O.to_np(w), 1e-5, _tag(dtype))
    assert np.array_equal(out.float().cpu().numpy(), want)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 128), (2, 4, 128), (7, 1000), (33, 4096), (16, 8192), (5, 50), (2, 16384), (3, 20000),
                                   (2, 35584), (1, 40960)])
@pytest.mark.parametrize("w_dtype", ["same", torch.float32])
def test_layernorm_and_dquant_bit_exact(dtype, shape, w_dtype):
    g = torch.Generator().manual_seed(22)
    K = shape[-1]
    x = (torch.randn(shape, generator=g) * 2 + 0.5).to(dtype)
    wd = dtype if w_dtype == "same" else w_dtype
    w = torch.empty(K).uniform_(0.5, 1.5, generator=g).to(wd)
    b = torch.randn(K, generator=g).to(wd)
    ln = flashnn_amd.LayerNorm(K, eps=1e-5)
    ln.weight.data, ln.bias.data = w, b
    out = ln.to(DEV)(x.to(DEV))
    assert out.dtype == dtype and out.shape == x.shape
    want = O.layernorm(O.to_np(x), O.to_np(w), O.to_np(b), 1e-5, _tag(dtype))
    got = out.float().cpu().numpy()
    assert np.array_equal(got, want)     # both moments are exact sums in fp64: same bits
    lq = flashnn_amd.LayernormDquant(K, eps=1e-5)
    lq.weight.data, lq.bias.data = w, b
    q, s = lq.to(DEV)(x.to(DEV))
    assert q.dtype == torch.int8 and q.shape == x.shape and s.dtype == dtype and s.shape == (x.numel() // K, 1)
    q_o, s_o = O.layernorm_dquant(O.to_np(x), O.to_np(w), O.to_np(b), 1e-5, _tag(dtype))
    assert np.array_equal(q.cpu().numpy(), q_o) and np.array_equal(s.float().cpu().numpy(), s_o)


def test_norm_layers_against_torch_reference_shapes():
    """The reference's own checks (tests/norm/test_layer_norm_dquant.py:22-41, test_rms_norm.py:34-50):
    torch.nn.LayerNorm + the test's quantiser, and the RMSNorm reference module, within their
    tolerances."""
    torch.manual_seed(0)
    for shape in ([4, 128], [2, 4, 128]):
        hidden = shape[-1]
        mod = torch.nn.LayerNorm(hidden, eps=1e-5).half()
        inp = torch.randn(shape).half()
        ref = mod(inp)
        scale = ref.abs().max(dim=-1, keepdim=True)[0] / 127
        ref_q = torch.clamp(torch.round(ref / scale), -128, 127).to(torch.int8)
        qmod = flashnn_amd.LayernormDquant(hidden, eps=1e-5).half().to(DEV)
        q, s = qmod(inp.to(DEV))
        torch.testing.assert_close(q.cpu(), ref_q, rtol=0.01, atol=2.0)
        torch.testing.assert_close(s.cpu(), scale.reshape(-1, 1), rtol=0.01, atol=0.01)
        lmod = flashnn_amd.LayerNorm(hidden, eps=1e-5).half().to(DEV)
        torch.testing.assert_close(lmod(inp.to(DEV)).cpu(), ref, atol=1e-3, rtol=1e-3)
    for shape in ([4, 128], [3, 64, 64]):
        hidden = shape[-1]
        inp = torch.randn(shape).half()
        w = torch.ones(hidden).half()
        ref = (inp.float() * torch.rsqrt(inp.float().pow(2).mean(-1, keepdim=True) + 1e-5)).type_as(inp) * w
        out = flashnn_amd.RMSNorm(hidden, eps=1e-5).half().to(DEV)(inp.to(DEV))
        torch.testing.assert_close(out.cpu(), ref, atol=1e-3, rtol=1e-3)


# ------------------------------------------------------------ streams and graph capture
def test_kernels_follow_the_current_stream():
    """Launches go to torch's current stream: work queued on a side stream behind a long-running kernel
    must see that kernel's output, and the default stream must not be needed for correctness."""
    x = workloads.activations(512, 4096, torch.float16, seed=61).to(DEV)
    w, ws = workloads.int8_weights(1024, 4096, seed=62)
    wd, wsd = w.to(DEV), ws.to(DEV)
    q_ref, s_ref = flashnn_amd.DynamicQuantize()(x)
    want = flashnn_amd.GemmA8W8(torch.bfloat16)(q_ref, wd, s_ref, wsd)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        big = torch.randn(4096, 4096, device=DEV)
        for _ in range(4):
            big = big @ big * 1e-3              # keeps the side stream busy ahead of the launches below
        x2 = x + 0                               # produced on the side stream
        q, s = flashnn_amd.DynamicQuantize()(x2)
        out = flashnn_amd.GemmA8W8(torch.bfloat16)(q, wd, s, wsd)
    side.synchronize()
    assert torch.equal(out, want) and torch.equal(q, q_ref)


def test_quant_gemm_step_under_graph_capture():
    """The C ABI neither allocates nor synchronises, so a DynamicQuant + A8W8 step (and a weight-only
    decode step) can be captured into a HIP graph; every replay, with fresh inputs copied into the
    captured buffers and eager work between the replays, must equal the eager result."""
    M, K, N = 64, 4096, 2048
    w, ws = workloads.int8_weights(N, K, seed=72)
    wd, wsd = w.to(DEV), ws.to(DEV)
    packed, scale, zp, _, _ = workloads.int4_group_weights(1024, K, 128, torch.float16, seed=73)
    packed, scale, zp = packed.to(DEV), scale.to(DEV), zp.to(DEV)
    x = torch.zeros(M, K, dtype=torch.float16, device=DEV)
    q = torch.empty(M, K, dtype=torch.int8, device=DEV)
    s = torch.empty(M, dtype=torch.float16, device=DEV)
    out = torch.empty(M, N, dtype=torch.float16, device=DEV)
    out4 = torch.empty(1, 1024, dtype=torch.float16, device=DEV)

    def step():
        launchers.hip_dynamic_quantize(q, x, s)
        launchers.hip_gemm_a8w8_forward(out, q, wd, s, wsd)
        launchers.hip_gemm_a16w4_forward(out4, x[:1], packed, scale, zero_points=zp)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                   # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for rep in range(3):
        xin = workloads.activations(M, K, torch.float16, seed=80 + rep).to(DEV)
        x.copy_(xin)
        graph.replay()
        torch.cuda.synchronize()
        got, got4 = out.clone(), out4.clone()
        out.zero_()
        out4.zero_()
        step()                                   # eager, same buffers
        torch.cuda.synchronize()
        assert torch.equal(got, out) and torch.equal(got4, out4), f"replay {rep}"
        assert bool(out.abs().sum() > 0)


def test_split_k_packed_decode_and_moe_under_graph_capture():
    """The paths with state beyond inputs and outputs, captured into a HIP graph: an A8W8 GEMM whose K the
    library splits through the launcher's workspace (counters must be back at zero after every replay), the
    decode on packed weights, the tiled weight-only GEMM on bf16 rows (its scratch comes from torch's caching
    allocator inside the capture) and a fused MoE on the tiled kernel.  Every replay, with fresh inputs and
    eager work in between, equals the eager result."""
    M, K, N = 256, 8192, 2304
    w, ws = workloads.int8_weights(N, K, seed=91)
    wd, wsd = w.to(DEV), ws.to(DEV)
    a8 = torch.zeros(M, K, dtype=torch.int8, device=DEV)
    sr = (torch.rand(M, device=DEV) * 1e-2).half()
    out8 = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    packed, scale, zp, _, _ = workloads.int4_group_weights(1024, K, 128, torch.float16, seed=92)
    packed, scale, zp = packed.to(DEV), scale.to(DEV), zp.to(DEV)
    op4 = flashnn_amd.GemmWeightOnly(torch.bfloat16)
    pk = op4.prepack(packed, scale, zp)
    xb = torch.zeros(M, K, dtype=torch.bfloat16, device=DEV)
    outp = torch.empty(1, 1024, dtype=torch.bfloat16, device=DEV)
    NW = 16640                                   # 130 tiles of 256 rows: the tiled kernel's side of the dispatch
    packed_w, scale_w, zp_w, _, _ = workloads.int4_group_weights(NW, K, 128, torch.float16, seed=94)
    packed_w, scale_w, zp_w = packed_w.to(DEV), scale_w.to(DEV), zp_w.to(DEV)
    outw = torch.empty(M, NW, dtype=torch.bfloat16, device=DEV)
    E, top_k, BM = 4, 2, 128
    be = torch.randint(-128, 128, (E, 512, 1024), dtype=torch.int8, device=DEV)
    ace = torch.rand(E, 512, device=DEV) * 1e-2
    tw, ids = torch.topk(torch.softmax(torch.randn(M, E, generator=torch.Generator().manual_seed(93)), -1), top_k)
    sid, eid, used = [t.to(DEV) for t in workloads.moe_align_block_size(ids, BM, E)]
    tw, ids = tw.float().contiguous().to(DEV), ids.to(DEV)
    outm = torch.empty(M, top_k, 512, dtype=torch.bfloat16, device=DEV)

    def step():
        launchers.hip_gemm_a8w8_forward(out8, a8, wd, sr, wsd)
        launchers.hip_gemm_a16w4_prepacked_forward(outp, xb[:1], pk)
        launchers.hip_gemm_a16w4_forward(outw, xb, packed_w, scale_w, zero_points=zp_w)
        flashnn_amd.fused_moe_a8w8_forward(a8[:, :1024], be, outm, sr, ace, tw, ids, sid, eid, used, True, top_k, BM)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                   # warm-up outside the capture (allocates the workspace)
    torch.cuda.current_stream().wait_stream(side)
    launchers.hip_gemm_a8w8_forward(out8, a8, wd, sr, wsd)
    assert _lib.last_kernel().startswith("gemm_a8w8_ring_kernel(split K)")
    launchers.hip_gemm_a16w4_forward(outw, xb, packed_w, scale_w, zero_points=zp_w)
    assert _lib.last_kernel().startswith("gemm_wo_tile_kernel(per-weight rounding)")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    outs = (out8, outp, outw, outm)
    for rep in range(3):
        a8.copy_(torch.randint(-128, 128, (M, K), dtype=torch.int8, generator=torch.Generator().manual_seed(100 + rep)).to(DEV))
        xb.copy_(workloads.activations(M, K, torch.bfloat16, seed=110 + rep).to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        for o in outs:
            o.zero_()
        step()                                   # eager, same buffers
        torch.cuda.synchronize()
        for g, o in zip(got, outs):
            assert torch.equal(g, o), f"replay {rep}"
            assert bool(o.float().abs().sum() > 0)


@pytest.mark.parametrize("M,N,K,out_ty", [(65, 2048, 8192, torch.bfloat16), (128, 1024, 4096, torch.float16), (200, 1920, 13312, torch.bfloat16),
                                          (256, 2048, 4096, torch.float16), (257, 2048, 4096, torch.bfloat16), (130, 2064, 4096, torch.float16)])
def test_a8w8_narrow_weights_run_as_passes_of_the_few_row_kernel(hip_lib, M, N, K, out_ty):
    """65 to 256 rows over a weight matrix of at most 2048 channels with rows of 4096 bytes and more: 64-row
    passes of the few-row kernel instead of a handful of tiles with K split; the same bits as the tiled
    kernel named through the C ABI, and as the oracle's epilogue on the exact accumulators."""
    a, b = _rand_i8((M, K), 5 + M).to(DEV), _rand_i8((N, K), 6 + N).to(DEV)
    g = torch.Generator().manual_seed(M + N)
    ar = (torch.rand(M, generator=g) * 0.05).half().to(DEV)
    ac = (torch.rand(N, generator=g) * 0.05).half().to(DEV)
    out = torch.empty(M, N, dtype=out_ty, device=DEV)
    launchers.hip_gemm_a8w8_forward(out, a, b, ar, ac)
    narrow = M <= 256 and N <= 2048
    assert _lib.last_kernel().startswith("gemm_a8w8_panel_kernel" if narrow else "gemm_a8w8_ring_kernel"), _lib.last_kernel()
    tiled = torch.empty_like(out)
    rc = hip_lib.fnn_gemm_a8w8_tiled(_lib.ptr(tiled), _lib.ptr(a), _lib.ptr(b), _lib.ptr(ar), _lib.ptr(ac), M, N, K, K, K, N,
                                     _lib.dtype_code(out_ty), _lib.FNN_F16, _lib.FNN_F16, 128, 128, 0, _lib.current_stream(out.device))
    assert rc == 0 and _lib.last_kernel().startswith("gemm_a8w8_ring_kernel")
    assert torch.equal(out, tiled)
    acc = O.gemm_a8w8_acc(a.cpu().numpy(), b.cpu().numpy())
    want = O.gemm_a8w8_epilogue_fp32(acc, O.to_np(ar.cpu()), O.to_np(ac.cpu()), O.tag_of(out))
    assert np.array_equal(out.float().cpu().numpy(), want.astype(np.float32))


# ------------------------------------------------------------------ strides through the C ABI
def test_c_abi_row_strides(hip_lib):
    """The launchers keep the reference's contiguity asserts, the C ABI takes row strides: operands and
    outputs that are column slices of wider buffers (lda > K, ldb > K, ldc > N) give the same bits."""
    M, N, K = 70, 144, 1056
    abuf, bbuf = _rand_i8((M, K + 64), 41).to(DEV), _rand_i8((N, K + 32), 42).to(DEV)
    a, b = abuf[:, 16:16 + K], bbuf[:, 32:32 + K]          # 16-byte aligned starts, strided rows
    g = torch.Generator().manual_seed(43)
    ar = (torch.rand(M, generator=g) * 0.05).half().to(DEV)
    ac = (torch.rand(N, generator=g) * 0.05).half().to(DEV)
    obuf = torch.full((M, N + 40), 7.0, dtype=torch.float16, device=DEV)
    out = obuf[:, 8:8 + N]
    rc = hip_lib.fnn_gemm_a8w8(out.data_ptr(), a.data_ptr(), b.data_ptr(), ar.data_ptr(), ac.data_ptr(), M, N, K,
                               a.stride(0), b.stride(0), out.stride(0), 0, 0, 0,
                               _lib.current_stream(torch.device(DEV)))
    assert rc == 0, hip_lib.fnn_last_error()
    torch.cuda.synchronize()
    want = O.gemm_a8w8_epilogue_fp32(O.gemm_a8w8_acc(a.cpu().numpy(), b.cpu().numpy()), O.to_np(ar.cpu()),
                                     O.to_np(ac.cpu()), O.F16)
    assert np.array_equal(out.float().cpu().numpy(), want)
    assert bool((obuf[:, :8] == 7).all()) and bool((obuf[:, 8 + N:] == 7).all())     # nothing written outside
    # dynamic quant with strided input and output rows
    xbuf = torch.randn(33, 1024 + 64, device=DEV).half()
    x = xbuf[:, 8:8 + 1024]
    qbuf = torch.full((33, 1024 + 16), 5, dtype=torch.int8, device=DEV)
    q = qbuf[:, 8:8 + 1024]
    sc = torch.empty(33, dtype=torch.float16, device=DEV)
    rc = hip_lib.fnn_dynamic_quant(q.data_ptr(), sc.data_ptr(), x.data_ptr(), 33, 1024, x.stride(0), q.stride(0), 0,
                                   _lib.current_stream(torch.device(DEV)))
    assert rc == 0, hip_lib.fnn_last_error()
    torch.cuda.synchronize()
    q_o, s_o = O.dynamic_quantize(O.to_np(x.cpu()), O.F16)
    assert np.array_equal(q.cpu().numpy(), q_o) and np.array_equal(sc.cpu().numpy(), s_o)
    assert bool((qbuf[:, :8] == 5).all()) and bool((qbuf[:, 8 + 1024:] == 5).all())


@pytest.mark.parametrize("M,N,K,kernel", [(1, 1024, 2048, "skinny"), (8, 1024, 2048, "skinny"), (1, 528, 1056, "panel"),
                                          (32, 2048, 1024, "panel"), (64, 8192, 1152, "panel"), (300, 520, 1056, "ring"),
                                          (40, 20480, 512, "ring"), (5, 100, 96, "any")])
def test_a8w8_c_abi_row_strides_on_every_kernel(hip_lib, M, N, K, kernel):
    """Strided operand and output rows (16-byte aligned starts) through each A8W8 kernel: the bits of the oracle, and
    nothing written outside the output's columns."""
    abuf, bbuf = _rand_i8((M, K + 64), 45).to(DEV), _rand_i8((N, K + 32), 46).to(DEV)
    a, b = abuf[:, 16:16 + K], bbuf[:, 32:32 + K]
    g = torch.Generator().manual_seed(47)
    ar = (torch.rand(M, generator=g) * 0.05).half().to(DEV)
    ac = (torch.rand(N, generator=g) * 0.05).half().to(DEV)
    obuf = torch.full((M, N + 40), 7.0, dtype=torch.bfloat16, device=DEV)
    out = obuf[:, 8:8 + N]
    rc = hip_lib.fnn_gemm_a8w8(out.data_ptr(), a.data_ptr(), b.data_ptr(), ar.data_ptr(), ac.data_ptr(), M, N, K,
                               a.stride(0), b.stride(0), out.stride(0), _lib.dtype_code(torch.bfloat16), 0, 0,
                               _lib.current_stream(torch.device(DEV)))
    assert rc == 0, hip_lib.fnn_last_error()
    torch.cuda.synchronize()
    assert _lib.last_kernel().startswith(f"gemm_a8w8_{kernel}_kernel"), _lib.last_kernel()
    want = O.gemm_a8w8_epilogue_fp32(O.gemm_a8w8_acc(a.cpu().numpy(), b.cpu().numpy()), O.to_np(ar.cpu()),
                                     O.to_np(ac.cpu()), O.BF16)
    assert np.array_equal(out.float().cpu().numpy(), want)
    assert bool((obuf[:, :8] == 7).all()) and bool((obuf[:, 8 + N:] == 7).all())


@pytest.mark.parametrize("M,K", [(33, 1024), (5, 8192), (4096, 1024), (7, 1000)])
def test_norm_entry_points_c_abi_row_strides(hip_lib, M, K):
    """RMSNorm, LayerNorm and their quantising forms with input and output rows that are column slices of wider
    buffers (ldx > K, ldo > K): the bits of the contiguous call, nothing written outside the output's columns (one
    workgroup per row, one wave per row, and the any-length kernels)."""
    dev = torch.device(DEV)
    st = _lib.current_stream(dev)
    g = torch.Generator().manual_seed(M + K)
    xbuf = torch.randn(M, K + 64, generator=g).bfloat16().to(DEV)
    x = xbuf[:, 8:8 + K]
    xc = x.contiguous()
    gamma = torch.empty(K).uniform_(0.5, 1.5, generator=g).to(DEV)
    beta = torch.randn(K, generator=g).to(DEV)
    code = _lib.dtype_code
    def run(call, out_ty, fill):
        obuf = torch.full((M, K + 32), fill, dtype=out_ty, device=DEV)
        o = obuf[:, 16:16 + K]
        plain = torch.empty(M, K, dtype=out_ty, device=DEV)
        s1, s2 = torch.empty(M, dtype=torch.bfloat16, device=DEV), torch.empty(M, dtype=torch.bfloat16, device=DEV)
        assert call(o, x, s1) == 0, hip_lib.fnn_last_error()
        assert call(plain, xc, s2) == 0, hip_lib.fnn_last_error()
        torch.cuda.synchronize()
        assert torch.equal(o, plain)
        assert bool((obuf[:, :16] == fill).all()) and bool((obuf[:, 16 + K:] == fill).all())
        return s1, s2
    bf, f32 = code(torch.bfloat16), code(torch.float32)
    run(lambda o, i, s: hip_lib.fnn_rmsnorm(o.data_ptr(), i.data_ptr(), gamma.data_ptr(), 1e-6, M, K, i.stride(0), o.stride(0),
                                            bf, f32, st), torch.bfloat16, 7.0)
    run(lambda o, i, s: hip_lib.fnn_layernorm(o.data_ptr(), i.data_ptr(), gamma.data_ptr(), beta.data_ptr(), 1e-5, M, K,
                                              i.stride(0), o.stride(0), bf, f32, st), torch.bfloat16, 7.0)
    s1, s2 = run(lambda o, i, s: hip_lib.fnn_rmsnorm_dquant(o.data_ptr(), s.data_ptr(), i.data_ptr(), gamma.data_ptr(), 1e-6, M, K,
                                                            i.stride(0), o.stride(0), bf, f32, st), torch.int8, 5)
    assert torch.equal(s1, s2)
    s1, s2 = run(lambda o, i, s: hip_lib.fnn_layernorm_dquant(o.data_ptr(), s.data_ptr(), i.data_ptr(), gamma.data_ptr(),
                                                              beta.data_ptr(), 1e-5, M, K, i.stride(0), o.stride(0), bf, f32, st),
                 torch.int8, 5)
    assert torch.equal(s1, s2)


@pytest.mark.parametrize("M", [1, 4, 16, 40, 64, 100])
def test_a16w4_prepacked_c_abi_row_strides(hip_lib, M):
    """The packed int4 GEMM with activation and output rows that are column slices of wider buffers: the bits of the
    contiguous call (one row, and 16, 32 and 64 rows per pass), nothing written outside the output's columns."""
    N, K = 2048, 1024
    g = torch.Generator().manual_seed(500 + M)
    w = torch.randint(-8, 8, (N, K), generator=g, dtype=torch.int8)
    qw = torch.from_numpy(O.pack_int4(w.numpy())).to(DEV)
    scale = torch.empty(K // 128, N).uniform_(1e-3, 1e-2, generator=g).half().to(DEV)
    zp = torch.randint(-4, 4, (K // 128, N), generator=g).half().to(DEV)
    packed = launchers.hip_a16w4_prepack(qw, scale, zp)
    bias = torch.randn(N, generator=g).bfloat16().to(DEV)
    abuf = torch.randn(M, K + 64, generator=g).bfloat16().to(DEV)
    a = abuf[:, 8:8 + K]
    ac = a.contiguous()
    obuf = torch.full((M, N + 24), 7.0, dtype=torch.bfloat16, device=DEV)
    out = obuf[:, 8:8 + N]
    plain = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    bf = _lib.dtype_code(torch.bfloat16)
    st = _lib.current_stream(torch.device(DEV))
    for o, i in ((out, a), (plain, ac)):
        rc = hip_lib.fnn_gemm_a16w4_prepacked(o.data_ptr(), i.data_ptr(), packed.buffer.data_ptr(), bias.data_ptr(), M, N, K,
                                              i.stride(0), o.stride(0), 128, bf, bf, bf, st)
        assert rc == 0, hip_lib.fnn_last_error()
    torch.cuda.synchronize()
    assert torch.equal(out, plain), _lib.last_kernel()
    assert bool((obuf[:, :8] == 7).all()) and bool((obuf[:, 8 + N:] == 7).all())
    assert torch.equal(launchers.hip_gemm_a16w4_prepacked_forward(torch.empty_like(plain), ac, packed, bias), plain)


SEEN_STRIDED_KERNELS = set()


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("group", [0, 128])
@pytest.mark.parametrize("M,N,K", [(1, 1024, 2048), (3, 1024, 2048), (3, 8704, 1024), (8, 2048, 1152), (16, 2048, 2048),
                                   (40, 1056, 2304), (70, 512, 1024), (200, 16512, 512), (1, 256, 18944), (24, 528, 512)])
def test_weight_only_c_abi_row_strides(hip_lib, bits, group, M, N, K):
    """The weight-only entry points take row strides (lda >= K, ldw >= K, ldc >= N): activations, weights and output
    that are column slices of wider buffers give the bits of the contiguous call, on every kernel family (decode,
    GEMV, panel, tiled, stream), and nothing is written outside the output's columns."""
    if group and K % group:
        pytest.skip("K is no multiple of the group size")
    act_ty = torch.float16 if (M + bits) % 2 else torch.bfloat16
    act, w, qw, scale, zp, bias = _wo_inputs(M, N, K, group, bits, act_ty, torch.float16, True, True, seed=400 + M)
    dev = torch.device(DEV)
    rows = qw.shape[0]
    abuf = torch.zeros(M, K + 64, dtype=act_ty, device=DEV)
    wbuf = torch.zeros(rows, K + 48, dtype=torch.int8, device=DEV)
    a, q = abuf[:, 8:8 + K], wbuf[:, 16:16 + K]                      # 16-byte aligned starts, strided rows
    a.copy_(act.to(DEV)); q.copy_(qw.to(DEV))
    obuf = torch.full((M, N + 24), 7.0, dtype=act_ty, device=DEV)
    out = obuf[:, 8:8 + N]
    sc, z, b = scale.to(DEV), zp.to(DEV), bias.to(DEV)
    fn = hip_lib.fnn_gemm_a16w8 if bits == 8 else hip_lib.fnn_gemm_a16w4
    code = _lib.dtype_code
    rc = fn(out.data_ptr(), a.data_ptr(), q.data_ptr(), sc.data_ptr(), b.data_ptr(), z.data_ptr(), M, N, K,
            a.stride(0), q.stride(0), out.stride(0), group, code(act_ty), code(act_ty), code(sc.dtype), code(z.dtype),
            code(b.dtype), _lib.current_stream(dev))
    assert rc == 0, hip_lib.fnn_last_error()
    strided_kernel = _lib.last_kernel()
    plain = torch.empty(M, N, dtype=act_ty, device=DEV)
    ac, qc = a.contiguous(), q.contiguous()
    rc = fn(plain.data_ptr(), ac.data_ptr(), qc.data_ptr(), sc.data_ptr(), b.data_ptr(), z.data_ptr(), M, N, K,
            K, K, N, group, code(act_ty), code(act_ty), code(sc.dtype), code(z.dtype), code(b.dtype),
            _lib.current_stream(dev))
    assert rc == 0, hip_lib.fnn_last_error()
    torch.cuda.synchronize()
    assert _lib.last_kernel() == strided_kernel, (strided_kernel, _lib.last_kernel())
    assert torch.equal(out, plain), strided_kernel
    SEEN_STRIDED_KERNELS.add(strided_kernel.split("<")[0].split("(")[0])
    assert bool((obuf[:, :8] == 7).all()) and bool((obuf[:, 8 + N:] == 7).all()), strided_kernel
    # ... and the contiguous call is the operator's result
    via_op = flashnn_amd.GemmWeightOnly(act_ty)(ac, qc, sc, b, z)
    assert torch.equal(via_op, plain) or M > 64      # (beyond 64 bf16 rows the operator adds the conversion scratch)


def test_weight_only_c_abi_row_strides_reached_every_kernel_family():
    """(runs after the cases above: they must have gone through the decode, panel, tiled and stream kernels)"""
    if len(SEEN_STRIDED_KERNELS) == 0:
        pytest.skip("the strided cases did not run in this session")
    for family in ("gemm_wo_decode_lds_kernel", "gemm_wo_panel_kernel", "gemm_wo_tile_kernel", "gemm_wo_stream_kernel"):
        assert family in SEEN_STRIDED_KERNELS, (family, sorted(SEEN_STRIDED_KERNELS))


# ----------------------------------------------------------------------------- empty inputs
def test_empty_inputs_through_the_operators():
    """No rows (or no channels) is a valid call: nothing is launched, the outputs have the right shapes."""
    x = torch.empty(0, 4096, dtype=torch.float16, device=DEV)
    q, s = flashnn_amd.DynamicQuantize()(x)
    assert q.shape == (0, 4096) and q.dtype == torch.int8 and s.shape == (0,) and s.dtype == torch.float16
    w = _rand_i8((256, 4096), 51).to(DEV)
    wscale = torch.rand(256, device=DEV).half()
    out = flashnn_amd.GemmA8W8(torch.float16)(q, w, s, wscale)
    assert out.shape == (0, 256) and out.dtype == torch.float16
    out = flashnn_amd.GemmWeightOnly(torch.float16)(x, w, wscale)
    assert out.shape == (0, 256)
    mod = flashnn_amd.RMSNormDquant(4096).to(DEV)
    q, s = mod(torch.empty(0, 4096, dtype=torch.bfloat16, device=DEV))
    assert q.shape == (0, 4096) and s.shape == (0,) and s.dtype == torch.bfloat16
    q, s = mod(torch.empty(2, 0, 4096, dtype=torch.bfloat16, device=DEV))
    assert q.shape == (2, 0, 4096) and s.shape == (2, 0)
    y = flashnn_amd.RMSNorm(4096).to(DEV)(torch.empty(0, 4096, dtype=torch.bfloat16, device=DEV))
    assert y.shape == (0, 4096)
    y = flashnn_amd.LayerNorm(4096).to(DEV)(torch.empty(0, 4096, dtype=torch.float16, device=DEV))
    assert y.shape == (0, 4096)
    torch.cuda.synchronize()


# ------------------------------------------------------------------ randomly drawn shapes
@pytest.mark.parametrize("seed", range(40))
def test_random_shapes_against_the_oracle(seed):
    """Shapes, types and options drawn at random (fixed seeds) around the edges of the kernels' fast paths:
    row counts either side of 16/32/64, channel counts that are and are not multiples of 32, K with every
    kind of tail.  A8W8 bit-exact, weight-only within the stated tolerance."""
    import random
    rnd = random.Random(1000 + seed)
    M = rnd.choice([1, 2, 5, 16, 17, 31, 32, 33, 40, 48, 63, 64, 65, 100, 129, 200, 260, 300, 513])
    N = rnd.choice([16, 32, 48, 64, 80, 96, 144, 256, 272, 512, 528, 1024, 1040, 1920, 4096, 4112])
    K = rnd.choice([32, 64, 96, 128, 160, 512, 544, 576, 608, 1024, 1056, 1088, 1120, 1152, 2048, 2080, 4096, 4128,
                    1000, 72])
    out_ty = rnd.choice([torch.float16, torch.bfloat16])
    g = torch.Generator().manual_seed(seed)
    a, b = _rand_i8((M, K), 2 * seed), _rand_i8((N, K), 2 * seed + 1)
    ar = (torch.rand(M, generator=g) * 0.05).to(rnd.choice([torch.float16, torch.bfloat16, torch.float32]))
    ac = (torch.rand(N, generator=g) * 0.05).to(rnd.choice([torch.float16, torch.bfloat16, torch.float32]))
    out = flashnn_amd.GemmA8W8(out_ty)(a.to(DEV), b.to(DEV), ar.to(DEV), ac.to(DEV))
    want = O.gemm_a8w8_epilogue_fp32(O.gemm_a8w8_acc(a.numpy(), b.numpy()), O.to_np(ar), O.to_np(ac), _tag(out_ty))
    assert np.array_equal(out.float().cpu().numpy(), want), f"a8w8 M={M} N={N} K={K} {out_ty}"

    bits = rnd.choice([8, 4])
    M = rnd.choice([1, 2, 3, 4, 5, 8, 9, 16, 17, 31, 32, 33, 48, 64, 65, 70, 100, 130])
    N = rnd.choice([16, 32, 64, 96, 128, 144, 256, 512, 528, 1024, 2048, 2064, 4096])
    K = rnd.choice([128, 256, 512, 1024, 1152, 2048, 4096, 1056, 1088, 1120, 640, 384])
    group = rnd.choice([0, 0, 128, 128, 64, 32])
    if group and K % group:
        group = 0
    act_ty = rnd.choice([torch.float16, torch.bfloat16])
    scale_ty = rnd.choice([act_ty, act_ty, torch.float32]) if group == 0 else act_ty
    case = _wo_inputs(M, N, K, group, bits, act_ty, scale_ty, with_zp=rnd.random() < 0.6,
                      with_bias=rnd.random() < 0.4, seed=seed)
    _wo_check(*case, group, bits, act_ty)
