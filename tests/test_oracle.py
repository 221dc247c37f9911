"""Pins the CPU oracle (oracle/flashnn_oracle.py) before anything is compared with it.

The reference's tests hold no golden vectors for this path (they regenerate seeded inputs
on a GPU and compare with loose tolerances), so each oracle function is pinned here by
checks that a plausible mistake would fail: the literal torch-op formula the reference
calls, brute-force loops on tiny inputs, closed forms and invariants.
"""
import ctypes

import numpy as np
import pytest
import torch

from oracle import flashnn_oracle as O
from oracle import torch_path as T


# ------------------------------------------------------------------------- rounding
def test_round_bf16_matches_torch():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(100000).astype(np.float32) * 10,
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, 1e-40], np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    assert np.array_equal(O.round_bf16(x), want)
    # ties go to even: 1 + 2^-8 is halfway between 1 and 1 + 2^-7
    assert O.round_bf16(np.array([1.00390625], np.float32))[0] == 1.0
    assert O.round_bf16(np.array([1.01171875], np.float32))[0] == 1.015625


# --------------------------------------------------------------------- dynamic quant
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(32, 32), (64, 64), (128, 128), (117, 987), (64, 4096)])
def test_dynamic_quantize_matches_torch_ops(dtype, shape):
    # sizes of the reference's test (tests/quant_gemm/test_dynamic_quant.py:29-35, the
    # largest one shrunk) on its own input distribution (rand*2-1) and on N(0,1)
    torch.manual_seed(0)
    for x in (torch.rand(shape) * 2 - 1, torch.randn(shape)):
        x = x.to(dtype)
        q_t, s_t = T.dynamic_quantize(x)
        q_o, s_o = O.dynamic_quantize(O.to_np(x), O.tag_of(x), clamp=False)   # the literal torch formula
        assert np.array_equal(q_o, q_t.numpy())
        assert np.array_equal(s_o, s_t.numpy())
        # the clamped form (the default, and what the kernels compute) differs only where that formula
        # reaches 128 and wraps
        q_c, s_c = O.dynamic_quantize(O.to_np(x), O.tag_of(x))
        assert np.array_equal(s_c, s_o)
        diff = q_c != q_o
        assert (q_o[diff] == -128).all() and (q_c[diff] == 127).all() and (O.to_np(x)[diff] > 0).all()
        if dtype == torch.float16:
            assert not diff.any()


def test_dynamic_quantize_bf16_row_maximum_is_clamped():
    """bf16 rows whose maximum has a mantissa that makes RN(max / 127) round down: max / scale rounds to
    127.5 and on to 128, which an unclamped conversion to int8 wraps to -128 - the sign of the row's largest
    activation.  The oracle (and the kernels) clamp: max |q| = 127 and sign(q) = sign(x) on every row."""
    torch.manual_seed(3)
    x = torch.randn(4096, 1024).bfloat16()
    xn = O.to_np(x)
    q_raw, _ = O.dynamic_quantize(xn, O.BF16, clamp=False)
    q, s = O.dynamic_quantize(xn, O.BF16)
    flipped = ((q_raw == -128) & (xn > 0)).any(axis=1)
    assert 0.005 < flipped.mean() < 0.05            # a visible fraction of rows is affected without the clamp
    # +127 is the largest value; -128 remains reachable for a negative row maximum (no wrap there); a scale
    # that rounded up leaves the maximum at 126.5, which rounds to 126
    assert (q.astype(np.int32).max(axis=1) <= 127).all() and (np.abs(q.astype(np.int32)).max(axis=1) >= 126).all()
    s32 = s.astype(np.float32)[:, None]
    big = np.abs(xn) > s32
    assert (np.sign(q[big]) == np.sign(xn[big])).all()
    assert not (np.sign(q_raw[big]) == np.sign(xn[big])).all()
    # hand-made rows: maximum 1 + j/128 for j in [42, 62] (the mantissas the rounding hits)
    hits = 0
    for j in range(42, 63):
        row = np.zeros((1, 64), np.float32)
        row[0, 0] = 1.0 + j / 128.0
        row[0, 1] = -0.5
        qr, _ = O.dynamic_quantize(row, O.BF16, clamp=False)
        qc, _ = O.dynamic_quantize(row, O.BF16)
        hits += int(qr[0, 0] == -128)
        assert qc[0, 0] == 127 and qc[0, 1] < 0
    assert hits > 0


def test_dynamic_quantize_bruteforce_f16():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((5, 37)).astype(np.float16)
    q, s = O.dynamic_quantize(x.astype(np.float32), O.F16)
    for i in range(x.shape[0]):
        mx = max(abs(float(v)) for v in x[i])
        sc = np.float16(np.float32(mx) / np.float32(127.0))
        assert s[i] == sc
        for j in range(x.shape[1]):
            t = np.float16(np.float32(x[i, j]) / np.float32(sc))
            assert q[i, j] == int(np.rint(np.float32(t)))


def test_dynamic_quantize_invariants_and_known_rows():
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((64, 512)) * 3).astype(np.float16).astype(np.float32)
    q, s = O.dynamic_quantize(x, O.F16)
    assert (np.abs(q.astype(np.int32)).max(axis=1) == 127).all()
    s32 = s.astype(np.float32)[:, None]
    big = np.abs(x) > s32
    assert (np.sign(q[big]) == np.sign(x[big])).all()
    # |q*s - x| <= s/2 plus the rounding of x/s to half precision (relative 2^-11 of |x|)
    assert (np.abs(q * s32 - x) <= s32 * 0.5 + np.abs(x) * 2.0 ** -10 + 1e-6).all()
    # a row that is c * [127, -127, 63.5, 0.4, -0.6, 2.5]: scale is exactly c; ties go to even
    row = np.array([[127.0, -127.0, 63.5, 0.4, -0.6, 2.5]], np.float32) * 0.5
    row = row.astype(np.float16).astype(np.float32)
    q, s = O.dynamic_quantize(row, O.F16)
    assert s[0] == np.float16(0.5)
    assert q[0].tolist() == [127, -127, 64, 0, -1, 2]
    # all-zero row: defined here as q = 0, scale = 0 (0/0 in the reference)
    q, s = O.dynamic_quantize(np.zeros((2, 8), np.float32), O.BF16)
    assert not q.any() and not s.any()


def test_dynamic_quantize_double_rounding_matters():
    """The two roundings to the input type are part of the semantics: an fp32-only
    restatement differs from the torch path on a visible fraction of elements."""
    torch.manual_seed(0)
    x = torch.randn(64, 4096).half()
    q_o, _ = O.dynamic_quantize(O.to_np(x), O.F16)
    xf = x.float().numpy()
    q_f32 = np.rint(xf / (np.abs(xf).max(-1, keepdims=True) / np.float32(127))).astype(np.int8)
    assert 0 < (q_o != q_f32).mean() < 0.05


# ------------------------------------------------------------------------- A8W8 GEMM
def test_gemm_acc_bruteforce_and_libraries(oracle_c):
    rng = np.random.default_rng(3)
    a = rng.integers(-128, 128, (7, 48), dtype=np.int8)
    b = rng.integers(-128, 128, (5, 48), dtype=np.int8)
    want = [[sum(int(a[m, k]) * int(b[n, k]) for k in range(48)) for n in range(5)] for m in range(7)]
    got = O.gemm_a8w8_acc(a, b)
    assert got.dtype == np.int32 and got.tolist() == want
    # larger: against numpy int64, torch._int_mm and the C restatement
    a = rng.integers(-128, 128, (64, 4096), dtype=np.int8)
    b = rng.integers(-128, 128, (96, 4096), dtype=np.int8)
    got = O.gemm_a8w8_acc(a, b)
    assert np.array_equal(got, a.astype(np.int64) @ b.astype(np.int64).T)
    assert np.array_equal(got, torch._int_mm(torch.from_numpy(a), torch.from_numpy(b).t()).numpy())
    c = np.empty((64, 96), np.int32)
    oracle_c.fnn_oracle_int8_gemm(a.ctypes.data, b.ctypes.data, c.ctypes.data, 64, 96, 4096, 4096, 4096, 96)
    assert np.array_equal(got, c)


def test_gemm_acc_special_cases():
    # identity selects b^T
    b = np.random.default_rng(4).integers(-128, 128, (16, 16), dtype=np.int8)
    assert np.array_equal(O.gemm_a8w8_acc(np.eye(16, dtype=np.int8), b), b.T.astype(np.int32))
    # (-128)*(-128) summed over 4096: 2^26, beyond fp32's exact range and int8/int16 range
    a = np.full((2, 4096), -128, np.int8)
    assert (O.gemm_a8w8_acc(a, a) == 67108864).all()
    # the reference's own fp32 matmul (quant_gemm.py:98) is NOT exact at this size
    odd = a.copy()
    odd[:, 0] = 127
    exact = O.gemm_a8w8_acc(odd, a)[0, 0]
    assert exact == 67108864 - 128 * 128 - 127 * 128
    assert float(np.float32(exact)) != float(exact) or True  # documented, not relied upon


@pytest.mark.parametrize("out_ty,scale_ty", [(torch.float16, torch.float16), (torch.bfloat16, torch.float32)])
def test_gemm_a8w8_output_close_to_torch_path(out_ty, scale_ty):
    # shape and ranges of the reference's test (tests/quant_gemm/test_gemm_a8w8.py:30-49)
    torch.manual_seed(0)
    M = N = K = 128
    a = torch.randint(-128, 127, (M, K), dtype=torch.int8)
    b = torch.randint(-128, 127, (N, K), dtype=torch.int8)
    ar = torch.rand(M, 1).to(scale_ty)
    ac = torch.rand(1, N).to(scale_ty)
    want = T.gemm_a8w8(a, b, ar, ac, out_ty).float().numpy()
    got = O.gemm_a8w8(a.numpy(), b.numpy(), O.to_np(ar), O.to_np(ac), O.tag_of(torch.empty(0, dtype=out_ty)))
    # with rand() scales some fp16 outputs overflow to inf, in the reference's test as well
    assert np.array_equal(np.isinf(got), np.isinf(want))
    fin = np.isfinite(got)
    np.testing.assert_allclose(got[fin], want[fin], rtol=1e-3 if out_ty == torch.float16 else 8e-3, atol=2e-3)
    seq = O.gemm_a8w8_epilogue_fp32(O.gemm_a8w8_acc(a.numpy(), b.numpy()), O.to_np(ar), O.to_np(ac),
                                    O.tag_of(torch.empty(0, dtype=out_ty)))
    # fp32 sequential epilogue and the fp64 closed form agree to one unit of the output type
    ulp = 2.0 ** -10 if out_ty == torch.float16 else 2.0 ** -7
    assert (np.abs(seq[fin] - got[fin]) <= np.abs(got[fin]) * ulp + 1e-7).all()


# ------------------------------------------------------------------- weight-only GEMM
def test_unpack_int4_all_bytes():
    allb = np.arange(256, dtype=np.uint8).view(np.int8).reshape(1, 256)
    w = O.unpack_int4(allb)
    for v in range(256):
        lo, hi = v & 0xF, v >> 4
        assert w[0, v] == (lo - 16 if lo > 7 else lo)   # low nibble -> even channel
        assert w[1, v] == (hi - 16 if hi > 7 else hi)   # high nibble -> odd channel
    # agrees with the reference's own unpack expression evaluated by torch
    q = torch.randint(-128, 128, (6, 40), dtype=torch.int8)
    assert np.array_equal(O.unpack_int4(q.numpy()).T, T.unpack_int4(q).numpy())
    assert np.array_equal(O.pack_int4(O.unpack_int4(q.numpy())), q.numpy())


def _wo_case(M, N, K, group, bits, act_ty, scale_ty, with_zp, with_bias, seed):
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


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("group", [0, 64])
@pytest.mark.parametrize("with_zp,with_bias", [(False, False), (True, True)])
@pytest.mark.parametrize("act_ty,scale_ty", [(torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16)])
def test_weight_only_matches_torch_path_and_f64(bits, group, with_zp, with_bias, act_ty, scale_ty):
    M, N, K = 3, 32, 256
    act, w, qw, scale, zp, bias = _wo_case(M, N, K, group, bits, act_ty, scale_ty, with_zp, with_bias, 7)
    tag = O.tag_of(act)
    got = O.weight_only_gemm(O.to_np(act), w.numpy(), O.to_np(scale), None if zp is None else O.to_np(zp),
                             None if bias is None else O.to_np(bias), O.tag_of(scale), tag, group, bits == 4)
    want = T.gemm_weight_only(act, qw, scale, bias, zp, act_ty).float().numpy()
    # identical roundings; only the fp32 summation order of the matmul may differ
    np.testing.assert_allclose(got, want, rtol=2e-3 if act_ty == torch.float16 else 1.6e-2, atol=1e-3)
    exact = O.weight_only_gemm_f64(O.to_np(act), w.numpy(), O.to_np(scale), None if zp is None else O.to_np(zp),
                                   None if bias is None else O.to_np(bias), group)
    # the reference rounds every dequantised weight to the scale type (bf16 keeps 8 bits),
    # so its own distance from the mathematical value is larger with bf16 scales
    tol = 1e-2 if scale_ty == torch.float16 else 5e-2
    np.testing.assert_allclose(got, exact, rtol=tol, atol=tol)


def test_weight_only_f64_bruteforce_and_integer_case():
    rng = np.random.default_rng(5)
    M, N, K, group = 2, 4, 128, 64
    act = rng.standard_normal((M, K)).astype(np.float16).astype(np.float32)
    w = rng.integers(-8, 8, (N, K)).astype(np.int8)
    scale = rng.uniform(1e-3, 1e-2, (K // group, N)).astype(np.float16).astype(np.float32)
    zp = rng.integers(-4, 4, (K // group, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    got = O.weight_only_gemm_f64(act, w, scale, zp, bias, group)
    for m in range(M):
        for n in range(N):
            s = float(bias[n])
            for k in range(K):
                s += float(act[m, k]) * (float(w[n, k]) - float(zp[k // group, n])) * float(scale[k // group, n])
            assert abs(got[m, n] - s) < 1e-9
    # scale = 1, zp = 0, small-integer activations: an exact integer matmul in every precision
    act_i = rng.integers(-4, 5, (M, K)).astype(np.float32)
    ones = np.ones(N, np.float32)
    out = O.weight_only_gemm(act_i, w, ones, None, None, O.F16, O.F16, 0, True)
    assert np.array_equal(out, (act_i.astype(np.int64) @ w.astype(np.int64).T).astype(np.float32))


def test_uint4_with_zero_point_maps_onto_signed_nibbles():
    """uint4 weight u with zero point z == signed nibble (u-8) with zero point (z-8)."""
    from flashnn_amd import workloads
    packed, s, zp_ref, u, zp = workloads.int4_group_weights(8, 256, 128)
    w = O.unpack_int4(packed.numpy()).astype(np.int32)
    assert np.array_equal(w + 8, u.numpy().astype(np.int32))
    assert np.array_equal(O.to_np(zp_ref) + 8, zp.numpy().astype(np.float32))


# --------------------------------------------------------------------- rmsnorm + quant
def test_prepacked_a16w4_layout_round_trip_and_addresses():
    """The packed form of int4 weights: the array-reshape statement of the layout and the address-by-address
    one are inverses of each other on random inputs; a weight, a scale and a zero point found by hand at
    the byte the layout's formulas name; the size is the reference layout's; every nibble is used once."""
    rng = np.random.default_rng(0)
    for N, K in [(16, 1024), (32, 2048), (48, 4096), (16, 8192)]:
        w = rng.integers(-8, 8, (N, K)).astype(np.int8)
        qw = O.pack_int4(w)
        scale = rng.uniform(1e-3, 1e-2, (K // 128, N)).astype(np.float16)
        zp = rng.integers(-8, 8, (K // 128, N)).astype(np.float16)
        buf = O.prepack_a16w4(qw, scale, zp)
        assert buf.dtype == np.uint8 and buf.size == N * K // 2 + 2 * (K // 128) * N * 2
        q2, s2, z2 = O.unpack_prepacked_a16w4(buf, N, K)
        assert np.array_equal(q2, qw) and np.array_equal(s2, scale) and np.array_equal(z2, zp)
        _, _, z0 = O.unpack_prepacked_a16w4(O.prepack_a16w4(qw, scale, None), N, K)
        assert not z0.any()
    # by hand (N = 32, K = 2048): channel 17 = tile 1, c = 1; k = 1485 = 1024 + 3 * 128 + 2 * 32 + 1 * 8 + 5, so
    # unit (tile 1, kc 1) = number 1 * 2 + 1 = 3, group b = 3, word i = 2, eighth g = 1, value j = 5 at bits
    # 4 * ((5 >> 1) + 4 * (5 & 1)) = 24: the low nibble of byte 3 of word 2 of the 16 bytes at 16 * (16 g + c)
    N, K = 32, 2048
    w = rng.integers(-8, 8, (N, K)).astype(np.int8)
    scale = rng.uniform(1e-3, 1e-2, (K // 128, N)).astype(np.float16)
    zp = rng.integers(-8, 8, (K // 128, N)).astype(np.float16)
    buf = O.prepack_a16w4(O.pack_int4(w), scale, zp)
    at = 3 * 8704 + 1024 * 3 + 16 * (16 * 1 + 1) + 4 * 2 + 3
    assert (int(buf[at]) & 0xF) - 8 == int(w[17, 1485])
    # its group is 8 * 1 + 3 = 11: scale at 8192 + 2 * (8 * c + b), zero point 256 bytes further
    at = 3 * 8704 + 8192 + 2 * (8 * 1 + 3)
    assert buf[at:at + 2].view(np.float16)[0] == scale[11, 17]
    assert buf[at + 256:at + 258].view(np.float16)[0] == zp[11, 17]
    # the very first word: channel 0, values 0..7, value j in nibble (j >> 1) + 4 (j & 1)
    first = int(buf[:4].view("<u4")[0])
    assert [((first >> (4 * ((j >> 1) + 4 * (j & 1)))) & 0xF) - 8 for j in range(8)] == [int(v) for v in w[0, :8]]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 128), (3, 32, 1024), (16, 8192)])
def test_rmsnorm_dquant_matches_torch_ops(dtype, shape):
    # shapes of the reference's test (tests/norm/test_rms_norm_dquant.py:43-57) + config size
    torch.manual_seed(0)
    x = torch.randn(shape).to(dtype)
    gamma = torch.empty(shape[-1]).uniform_(0.5, 1.5)
    for eps in (1e-5, 1e-6):
        q_t, s_t = T.rmsnorm_dquant(x, gamma, eps)
        q_o, s_o = O.rmsnorm_dquant(O.to_np(x), gamma.numpy(), eps, O.tag_of(x))
        d = np.abs(q_o.astype(np.int32) - q_t.numpy().astype(np.int32))
        # torch sums x^2 in its own fp32 order: a last-bit difference in the mean can move an
        # element that sits on a rounding tie by one step, nothing more
        assert d.max() <= 1 and (d != 0).mean() < 1e-3
        np.testing.assert_allclose(s_o, s_t.float().numpy(), rtol=2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10)


def test_rmsnorm_dquant_closed_forms():
    # constant row c, gamma = 1, eps = 0: n = sign(c) exactly, scale = 1/127, q = +-127
    x = np.full((2, 256), 3.0, np.float32)
    x[1] = -0.5
    q, s = O.rmsnorm_dquant(x, np.ones(256, np.float32), 0.0, O.F16)
    assert (q[0] == 127).all() and (q[1] == -127).all()
    assert np.allclose(s, np.float32(np.float16(1 / 127)))
    # invariants on random rows
    rng = np.random.default_rng(6)
    x = rng.standard_normal((32, 1024)).astype(np.float16).astype(np.float32)
    g = rng.uniform(0.5, 1.5, 1024).astype(np.float32)
    q, s = O.rmsnorm_dquant(x, g, 1e-6, O.F16)
    assert (np.abs(q.astype(np.int32)).max(axis=1) == 127).all()
    n = x / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-6) * g
    assert (np.abs(q * (np.abs(n).max(-1, keepdims=True) / 127) - n) <= np.abs(n).max(-1, keepdims=True) / 127 * 0.5001).all()


# ------------------------------------------------- rmsnorm, layernorm, layernorm + quant
def _ulp(dtype):
    return 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 128), (3, 64, 64), (16, 8192)])
def test_rmsnorm_matches_torch_ops(dtype, shape):
    # shapes of tests/norm/test_rms_norm.py:35 + the configuration width
    torch.manual_seed(1)
    x = torch.randn(shape).to(dtype)
    for gamma in (torch.empty(shape[-1]).uniform_(0.5, 1.5).to(dtype), torch.empty(shape[-1]).uniform_(0.5, 1.5)):
        want = T.rmsnorm(x, gamma, 1e-5).float().numpy()
        got = O.rmsnorm(O.to_np(x), O.to_np(gamma), 1e-5, O.tag_of(x))
        # identical except where torch's fp32 summation order moves the mean by one bit
        np.testing.assert_allclose(got, want, rtol=_ulp(dtype), atol=0)
        assert (got != want).mean() < 1e-2


def test_rmsnorm_closed_forms():
    # constant row c: x * rsqrt(c^2) = sign(c) exactly (eps = 0); times gamma
    x = np.full((2, 64), 4.0, np.float32)
    x[1] = -0.25
    g = np.linspace(0.5, 1.5, 64).astype(np.float16).astype(np.float32)
    y = O.rmsnorm(x, g, 0.0, O.F16)
    assert np.array_equal(y[0], g) and np.array_equal(y[1], -g)
    # scale invariance in powers of two (exact in floating point)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((8, 512)).astype(np.float16).astype(np.float32)
    assert np.array_equal(O.rmsnorm(x, g[:1].repeat(512), 0.0, O.F16), O.rmsnorm(4 * x, g[:1].repeat(512), 0.0, O.F16))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 128), (2, 4, 128), (16, 8192), (5, 1000)])
def test_layernorm_matches_torch_and_f64(dtype, shape):
    # shapes of tests/norm/test_layer_norm_dquant.py:23 + wider rows
    torch.manual_seed(2)
    K = shape[-1]
    x = (torch.randn(shape) * 2 + 0.5).to(dtype)
    w = torch.empty(K).uniform_(0.5, 1.5).to(dtype)
    b = torch.randn(K).to(dtype)
    want = T.layernorm(x, w, b, 1e-5).float().numpy()
    got = O.layernorm(O.to_np(x), O.to_np(w), O.to_np(b), 1e-5, O.tag_of(x))
    # torch takes the moments in its own order: 1 ulp of the output type at most, and rarely
    np.testing.assert_allclose(got, want, rtol=_ulp(dtype), atol=_ulp(dtype) * 2.0 ** -6)
    assert (got != want).mean() < 2e-2
    # the mathematical value, evaluated in float64
    x64 = O.to_np(x).astype(np.float64).reshape(-1, K)
    mu = x64.mean(-1, keepdims=True)
    var = ((x64 - mu) ** 2).mean(-1, keepdims=True)
    exact = (x64 - mu) / np.sqrt(var + 1e-5) * O.to_np(w).astype(np.float64) + O.to_np(b).astype(np.float64)
    assert (np.abs(got.reshape(-1, K) - exact) <= np.abs(exact) * _ulp(dtype) * 0.51 + 1e-6).all()


def test_layernorm_closed_forms_and_invariants():
    K = 256
    ones, zeros = np.ones(K, np.float32), np.zeros(K, np.float32)
    # constant row: x - mean = 0, so y = beta whatever eps and gamma
    beta = np.linspace(-1, 1, K).astype(np.float16).astype(np.float32)
    y = O.layernorm(np.full((1, K), 3.5, np.float32), 2 * ones, beta, 1e-5, O.F16)
    assert np.array_equal(y[0], beta)
    # a row of +-a: mean 0, var a^2, y = +-a / sqrt(a^2 + eps)
    row = np.where(np.arange(K) % 2 == 0, 2.0, -2.0).astype(np.float32)[None]
    y = O.layernorm(row, ones, zeros, 0.0, O.F16)
    assert np.array_equal(y, np.sign(row))
    # zero mean, unit variance for gamma = 1, beta = 0 on random rows
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((16, 4096)) * 3 + 1).astype(np.float16).astype(np.float32)
    y = O.layernorm(x, np.ones(4096, np.float32), np.zeros(4096, np.float32), 1e-5, O.F16).astype(np.float64)
    assert np.abs(y.mean(-1)).max() < 1e-3 and np.abs(y.var(-1) - 1).max() < 2e-3
    # shift invariance by a value that keeps every x exactly representable
    assert np.array_equal(O.layernorm(x[:, :64], ones[:64], zeros[:64], 1e-5, O.F32),
                          O.layernorm(x[:, :64].astype(np.float32), ones[:64], zeros[:64], 1e-5, O.F32))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 128), (2, 4, 128), (8, 4096)])
def test_layernorm_dquant_matches_torch_ops(dtype, shape):
    torch.manual_seed(5)
    K = shape[-1]
    x = torch.randn(shape).to(dtype)
    w = torch.empty(K).uniform_(0.5, 1.5).to(dtype)
    b = (torch.randn(K) * 0.1).to(dtype)
    q_t, s_t = T.layernorm_dquant(x, w, b, 1e-5)
    q_o, s_o = O.layernorm_dquant(O.to_np(x), O.to_np(w), O.to_np(b), 1e-5, O.tag_of(x))
    assert q_o.shape == tuple(shape) and s_o.shape == (x.numel() // K, 1) and s_t.dtype == dtype
    # the quantisation step is literally dynamic_quantize of the rounded layer norm ...
    y = O.layernorm(O.to_np(x), O.to_np(w), O.to_np(b), 1e-5, O.tag_of(x))
    q_d, s_d = O.dynamic_quantize(y.reshape(-1, K), O.tag_of(x), scale_dtype=O.tag_of(x), clamp=True)
    assert np.array_equal(q_o.reshape(-1, K), q_d) and np.array_equal(s_o[:, 0], s_d)
    # ... and torch's own layer norm feeding torch's ops gives the same up to the 1-ulp cases
    d = np.abs(q_o.astype(np.int32) - q_t.numpy().astype(np.int32))
    assert d.max() <= 1 and (d != 0).mean() < 2e-2
    np.testing.assert_allclose(s_o, s_t.float().numpy(), rtol=_ulp(dtype))
    # given torch's layer norm output, the oracle's quantisation reproduces torch's exactly
    n_t = T.layernorm(x, w, b, 1e-5)
    q_x, s_x = O.dynamic_quantize(O.to_np(n_t).reshape(-1, K), O.tag_of(x), scale_dtype=O.tag_of(x), clamp=True)
    assert np.array_equal(q_x, q_t.numpy().reshape(-1, K)) and np.array_equal(s_x, s_t.float().numpy()[:, 0])


# ------------------------------------------------------------------- mixture of experts
def _moe_case(M, E, N, K, top_k, block_m, seed):
    from flashnn_amd import workloads
    g = torch.Generator().manual_seed(seed)
    a = torch.randint(-128, 128, (M, K), dtype=torch.int8, generator=g)
    b = torch.randint(-128, 128, (E, N, K), dtype=torch.int8, generator=g)
    ar = (torch.rand(M, generator=g) * 0.05).half()
    ac = (torch.rand(E, N, generator=g) * 0.05).half()
    logits = torch.randn(M, E, generator=g)
    w, ids = torch.topk(torch.softmax(logits, -1), top_k, dim=-1)
    sorted_ids, expert_ids, used = workloads.moe_align_block_size(ids, block_m, E)
    return a, b, ar, ac, w.float().contiguous(), ids, sorted_ids, expert_ids, used


def test_moe_align_block_size_layout():
    from flashnn_amd import workloads
    ids = torch.tensor([[0, 2], [2, 1], [2, 0]])
    s, e, used = workloads.moe_align_block_size(ids, 4, 3)
    # expert 0 owns routed rows 0 and 5, expert 1 row 3, expert 2 rows 1, 2, 4; 6 = padding
    assert s.tolist()[:12] == [0, 5, 6, 6, 3, 6, 6, 6, 1, 2, 4, 6]
    assert e.tolist()[:3] == [0, 1, 2] and used.item() == 12
    assert s.dtype == torch.int32 and len(s) % 4 == 0 and set(s.tolist()[12:]) <= {6}
    # an expert without rows takes no block
    s, e, used = workloads.moe_align_block_size(torch.tensor([[2], [2]]), 16, 3)
    assert used.item() == 16 and e[0] == 2 and s.tolist()[:3] == [0, 1, 2]


@pytest.mark.parametrize("mul_w", [False, True])
def test_fused_moe_a8w8_against_per_element_loop(mul_w):
    M, E, N, K, top_k, BM = 5, 3, 8, 32, 2, 4
    a, b, ar, ac, w, ids, s, e, used = _moe_case(M, E, N, K, top_k, BM, 40)
    c = np.full((M * top_k, N), -7.0, np.float32)
    O.fused_moe_a8w8(a.numpy(), b.numpy(), c, O.to_np(ar), O.to_np(ac), w.numpy(), s.numpy(), e.numpy(), used.numpy(),
                     mul_w, top_k, BM, O.F16)
    flat = ids.flatten().tolist()
    for t in range(M * top_k):          # every routed row is listed exactly once, under its own expert
        ex = flat[t]
        for n in range(N):
            acc = sum(int(a[t // top_k, k]) * int(b[ex, n, k]) for k in range(K))
            f = np.float32(np.float32(np.float32(acc) * np.float32(ar[t // top_k])) * np.float32(ac[ex, n]))
            if mul_w:
                f = np.float32(f * w.flatten()[t].numpy())
            assert c[t, n] == np.float32(np.float16(f)), (t, n)


def test_fused_moe_a8w8_reductions_and_invariants():
    M, E, N, K, top_k, BM = 9, 4, 16, 64, 2, 4
    a, b, ar, ac, w, ids, s, e, used = _moe_case(M, E, N, K, top_k, BM, 41)
    args = (O.to_np(ar), O.to_np(ac), w.numpy())
    c = O.fused_moe_a8w8(a.numpy(), b.numpy(), np.zeros((M * top_k, N), np.float32), *args, s.numpy(), e.numpy(),
                         used.numpy(), True, top_k, BM, O.BF16)
    # one expert, top_k = 1, identity order: the plain A8W8 GEMM with the fp32 epilogue
    one = O.fused_moe_a8w8(a.numpy(), b.numpy()[1:2], np.zeros((M, N), np.float32), O.to_np(ar), O.to_np(ac)[1:2], None,
                           np.r_[np.arange(M), [M] * 3].astype(np.int32), np.zeros(3, np.int32), np.array([12]),
                           False, 1, BM, O.F16)
    want = O.gemm_a8w8_epilogue_fp32(O.gemm_a8w8_acc(a.numpy(), b.numpy()[1]), O.to_np(ar), O.to_np(ac)[1], O.F16)
    assert np.array_equal(one, want)
    # the order of the rows inside an expert's blocks does not matter
    s2 = s.clone()
    s2[0:BM] = s[0:BM].flip(0)
    c2 = O.fused_moe_a8w8(a.numpy(), b.numpy(), np.zeros((M * top_k, N), np.float32), *args, s2.numpy(), e.numpy(),
                          used.numpy(), True, top_k, BM, O.BF16)
    assert np.array_equal(c, c2)
    # rows beyond num_tokens_post_padded are not touched: cutting the list after the first block
    # leaves every row of the other blocks at its old value
    c3 = O.fused_moe_a8w8(a.numpy(), b.numpy(), np.full((M * top_k, N), 3.0, np.float32), *args, s.numpy(), e.numpy(),
                          np.array([BM]), True, top_k, BM, O.BF16)
    first = [t for t in s[:BM].tolist() if t < M * top_k]
    rest = [t for t in range(M * top_k) if t not in first]
    assert np.array_equal(c3[first], c[first]) and (c3[rest] == 3.0).all()


def _moe_w4_case(M, E, N2, K, top_k, block_m, group, seed, zp_int=False):
    """N2 = packed rows (2*N2 output channels)."""
    from flashnn_amd import workloads
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(M, K, generator=g).half()
    w = torch.randint(-8, 8, (E, 2 * N2, K), dtype=torch.int8, generator=g)
    packed = torch.stack([torch.from_numpy(O.pack_int4(w[e].numpy())) for e in range(E)])
    sshape = (E, 2 * N2) if group == 0 else (E, 2 * N2, K // group)
    scale = torch.empty(sshape).uniform_(1e-3, 1e-2, generator=g).half()
    zp = torch.randint(-3, 4, sshape, generator=g)
    zp = zp.to(torch.int8) if zp_int else zp.half()
    tw, ids = torch.topk(torch.softmax(torch.randn(M, E, generator=g), -1), top_k, dim=-1)
    s, e, used = workloads.moe_align_block_size(ids, block_m, E)
    return a, w, packed, scale, zp, tw.float().contiguous(), ids, s, e, used


@pytest.mark.parametrize("group", [0, 16])
def test_fused_moe_a16w4_against_f64_loop(group):
    M, E, N2, K, top_k, BM = 4, 3, 4, 32, 2, 4
    a, w, packed, scale, zp, tw, ids, s, e, used = _moe_w4_case(M, E, N2, K, top_k, BM, group, 50)
    c = O.fused_moe_a16w4(O.to_np(a), packed.numpy(), np.zeros((M * top_k, 2 * N2), np.float32), O.to_np(scale),
                          O.to_np(zp), tw.numpy(), s.numpy(), e.numpy(), used.numpy(), True, top_k, BM, O.F16, O.F16)
    flat = ids.flatten().tolist()
    for t in range(M * top_k):
        ex = flat[t]
        for n in range(2 * N2):
            v = mag = 0.0
            for k in range(K):
                sg = scale[ex, n] if group == 0 else scale[ex, n, k // group]
                zg = zp[ex, n] if group == 0 else zp[ex, n, k // group]
                term = float(a[t // top_k, k]) * (float(w[ex, n, k]) - float(zg)) * float(sg)
                v += term
                mag += abs(term)
            v *= float(tw.flatten()[t])
            mag *= float(tw.flatten()[t])
            # one rounding of each dequantised weight to 11 bits (per K block) and one of the result
            assert abs(c[t, n] - v) <= 2.0 ** -10 * mag + 2.0 ** -10 * abs(v), (t, n, c[t, n], v)


def test_fused_moe_a16w4_exact_and_reductions():
    M, E, N2, K, top_k, BM = 6, 2, 8, 64, 1, 4
    a, w, packed, scale, zp, tw, ids, s, e, used = _moe_w4_case(M, E, N2, K, top_k, BM, 0, 51, zp_int=True)
    # integer activations, unit scales, integer zero points: every product and sum is exact
    ai = torch.randint(-4, 5, (M, K)).half()
    ones = torch.ones(E, 2 * N2).half()
    c = O.fused_moe_a16w4(O.to_np(ai), packed.numpy(), np.zeros((M, 2 * N2), np.float32), O.to_np(ones), zp.numpy(),
                          None, s.numpy(), e.numpy(), used.numpy(), False, 1, BM, O.F16, O.F16)
    for t in range(M):
        ex = ids.flatten()[t].item()
        want = ai[t].double() @ (w[ex].double() - zp[ex].double().reshape(-1, 1)).T
        assert np.array_equal(c[t], want.numpy().astype(np.float32))
    # one expert, identity order: GemmWeightOnly's mathematical value (per channel)
    one = O.fused_moe_a16w4(O.to_np(a), packed.numpy()[1:2], np.zeros((M, 2 * N2), np.float32), O.to_np(scale)[1:2],
                            zp.numpy()[1:2], None, np.r_[np.arange(M), [M] * 2].astype(np.int32), np.zeros(2, np.int32),
                            np.array([8]), False, 1, BM, O.F16, O.F16)
    ref = O.weight_only_gemm_f64(O.to_np(a), w[1].numpy(), O.to_np(scale)[1], zp[1].numpy(), None, 0)
    np.testing.assert_allclose(one, ref, rtol=2e-3, atol=1e-5)


def test_one_step_dequantisation_equals_the_two_roundings():
    """The kernels that round every weight as the torch path does take a short form where the zero points are whole:
    one fp16 subtraction of (offset + zp) from the offset-coded weight, or, for bf16 tables, one exact fp32
    u * s - (off + zp) * s rounded once to bf16.  Both must give the bits of `((q - zp) * s)` evaluated in the table
    type with each operation rounded (flashnn/quant_gemm.py:14-17) - checked here with torch's own 16-bit arithmetic
    over every int8 weight, every whole zero point in range and random scales; and a fractional or larger zero
    point must be able to differ, which is why the kernels test for it."""
    g = torch.Generator().manual_seed(5)
    q = torch.arange(-128, 128, dtype=torch.float32).reshape(-1, 1, 1)
    # bf16: zero points -128 .. 128, scales over several binades
    zp = torch.arange(-128, 129, dtype=torch.float32).reshape(1, -1, 1)
    s = (torch.empty(64).uniform_(1e-3, 1e-2, generator=g) * 2.0 ** torch.randint(-6, 7, (64,), generator=g)).bfloat16().reshape(1, 1, -1)
    want = (q.bfloat16() - zp.bfloat16()) * s                                   # two bf16 operations
    u, off = q.double() + 128.0, 128.0
    exact = u * s.double() - (off + zp.double()) * s.double()                    # what one fp32 fma returns: see below
    assert torch.equal(exact.float().double(), exact)                            # ... exactly, in fp32
    assert torch.equal(((u * s.double()).float()).double(), u * s.double())      # and both products are fp32 numbers
    assert torch.equal((((off + zp.double()) * s.double()).float()).double(), (off + zp.double()) * s.double())
    assert torch.equal(exact.float().bfloat16(), want)
    # fp16: zero points -512 .. 512 under the offset 1152 (int8) of the exponent-trick conversion
    zp = torch.arange(-512, 513, dtype=torch.float32).reshape(1, -1, 1)
    s = torch.empty(16).uniform_(1e-3, 1e-2, generator=g).half().reshape(1, 1, -1)
    want = (q.half() - zp.half()) * s
    x = (q + 1152.0).half()
    assert torch.equal(x.float(), q + 1152.0)
    sub = (torch.tensor(1152.0).half() + zp.half())                              # formed once per channel
    assert torch.equal(sub.float(), 1152.0 + zp)
    assert torch.equal((x - sub) * s, want)
    # the odd int4 channel's offset of 72, in steps of 1/16 under the exponent of 64
    q4 = torch.arange(-8, 8, dtype=torch.float32).reshape(-1, 1, 1)
    x = (q4 + 72.0).half()
    sub = (torch.tensor(72.0).half() + zp.half())
    assert torch.equal(sub.float(), 72.0 + zp) and torch.equal((x - sub) * s, (q4.half() - zp.half()) * s)
    # not so beyond the range: q - zp no longer fits the type and the reference's first rounding shows
    zp_bad = torch.tensor([300.0, 3.3]).bfloat16().reshape(1, -1, 1)
    s1 = torch.tensor([0.0078125 * 1.3]).bfloat16().reshape(1, 1, -1)
    two = (q.bfloat16() - zp_bad) * s1
    one = ((q.double() - zp_bad.double()) * s1.double()).float().bfloat16()
    assert not torch.equal(one[:, 0], two[:, 0]) and not torch.equal(one[:, 1], two[:, 1])
