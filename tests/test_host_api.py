"""CPU-only checks of the boundary: the C-ABI library loads and exports every symbol the
header declares, argument errors are reported without touching a GPU, and the Python
operators mirror the reference's dispatch and error behaviour."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import flashnn_amd
from flashnn_amd import _lib, kernel_backend
from oracle import flashnn_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "flashnn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fnn_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(hip_lib):
    declared = _declared_symbols()
    assert "fnn_gemm_a16w4" in declared and "fnn_dynamic_quant" in declared
    for name in declared:
        assert hasattr(hip_lib, name), f"{name} is declared in include/flashnn_hip.h but not exported"
    assert set(_lib.exported_symbols()) == set(declared)
    assert hip_lib.fnn_version() == 2


def test_argument_errors_are_reported_without_a_gpu(hip_lib):
    null = ctypes.c_void_p(0)
    one = ctypes.c_void_p(16)
    rc = hip_lib.fnn_dynamic_quant(null, null, null, 4, 8, 8, 8, 0, null)
    assert rc == -1 and b"null pointer" in hip_lib.fnn_last_error()
    rc = hip_lib.fnn_dynamic_quant(one, one, one, 4, 8, 4, 8, 0, null)   # ldx < K
    assert rc == -1 and b"bad shape" in hip_lib.fnn_last_error()
    rc = hip_lib.fnn_dynamic_quant(one, one, one, 4, 8, 8, 8, 2, null)   # fp32 input
    assert rc == -2
    rc = hip_lib.fnn_gemm_a8w8(one, one, one, one, one, 4, 4, 128, 128, 128, 4, 2, 0, 0, null)
    assert rc == -2 and b"float16 or bfloat16" in hip_lib.fnn_last_error()
    rc = hip_lib.fnn_rmsnorm(one, one, null, 1e-5, 4, 8, 8, 8, 0, 0, null)               # no gamma
    assert rc == -1 and b"fnn_rmsnorm: null pointer" in hip_lib.fnn_last_error()
    rc = hip_lib.fnn_layernorm(one, one, one, null, 1e-5, 4, 8, 8, 8, 0, 0, null)         # no beta
    assert rc == -1 and b"fnn_layernorm: null pointer" in hip_lib.fnn_last_error()
    rc = hip_lib.fnn_layernorm_dquant(one, null, one, one, one, 1e-5, 4, 8, 8, 8, 0, 0, null)   # no scale
    assert rc == -1 and b"fnn_layernorm_dquant: null pointer" in hip_lib.fnn_last_error()
    rc = hip_lib.fnn_layernorm(one, one, one, one, 1e-5, 4, 8, 8, 4, 0, 0, null)          # ldo < K
    assert rc == -1 and b"bad shape" in hip_lib.fnn_last_error()
    rc = hip_lib.fnn_rmsnorm(one, one, one, 1e-5, 4, 8, 8, 8, 2, 0, null)                # fp32 input
    assert rc == -2 and b"fp16 or bf16" in hip_lib.fnn_last_error()
    assert hip_lib.fnn_layernorm_dquant(one, one, one, one, one, 1e-5, 0, 8, 8, 8, 1, 2, null) == 0   # M = 0
    rc = hip_lib.fnn_gemm_a16w4(one, one, one, one, null, null, 1, 7, 64, 64, 64, 7, 0, 0, 0, 0, 0, 0, null)
    assert rc == -1 and b"even" in hip_lib.fnn_last_error()
    rc = hip_lib.fnn_gemm_a16w8(one, one, one, one, null, null, 1, 8, 100, 100, 100, 8, 64, 0, 0, 0, 0, 0, null)
    assert rc == -1 and b"multiple of the group" in hip_lib.fnn_last_error()
    # row strides the kernels' 32-bit row offsets cannot reach are refused, not wrapped
    rc = hip_lib.fnn_gemm_a16w8(one, one, one, one, null, null, 4, 64, 1024, 1 << 31, 1024, 64, 0, 0, 0, 0, 0, 0, null)
    assert rc == -2 and b"row stride too large" in hip_lib.fnn_last_error()
    rc = hip_lib.fnn_gemm_a16w4(one, one, one, one, null, null, 4, 64, 1024, 1024, 1 << 31, 64, 0, 0, 0, 0, 0, 0, null)
    assert rc == -2 and b"row stride too large" in hip_lib.fnn_last_error()
    # the packed int4 form: shapes without one, rows the kernel cannot address, and bad table types are refused
    assert hip_lib.fnn_a16w4_prepacked_bytes(28672, 8192, 128) == 28672 * 8192 // 2 + 4 * 64 * 28672
    assert hip_lib.fnn_a16w4_prepacked_bytes(28672, 8192, 64) == 0 and hip_lib.fnn_a16w4_prepacked_bytes(24, 8192, 128) == 0
    assert hip_lib.fnn_a16w4_prepacked_bytes(4096, 3072, 128) == 0 and hip_lib.fnn_a16w4_prepacked_bytes(4096, 4000, 128) == 0
    rc = hip_lib.fnn_a16w4_prepack(one, one, one, null, 64, 1024, 1024, 128, 1, 0, null)       # bf16 scales
    assert rc == -2 and b"fp16 scales" in hip_lib.fnn_last_error()
    rc = hip_lib.fnn_a16w4_prepack(one, one, one, null, 64, 1000, 1000, 128, 0, 0, null)
    assert rc == -2 and b"packed form needs" in hip_lib.fnn_last_error()
    rc = hip_lib.fnn_gemm_a16w4_prepacked(one, one, one, null, 2, 64, 1024, 1 << 31, 64, 128, 0, 0, 0, null)
    assert rc == -2 and b"beyond what the kernel addresses" in hip_lib.fnn_last_error()
    rc = hip_lib.fnn_gemm_a16w4_prepacked(one, one, one, null, 2, 64, 1024, 1028, 64, 128, 0, 0, 0, null)
    assert rc == -1 and b"16-byte aligned" in hip_lib.fnn_last_error()
    assert hip_lib.fnn_gemm_a16w4_prepacked(null, null, null, null, 0, 64, 1024, 1024, 64, 128, 0, 0, 0, null) == 0
    # empty problems are a no-op
    assert hip_lib.fnn_gemm_a8w8_i32(one, one, one, 0, 4, 128, 128, 128, 4, null) == 0


def test_public_names_match_the_reference_module():
    for name in ("DynamicQuantize", "GemmA8W8", "GemmWeightOnly", "RMSNormDquant", "RMSNorm", "LayerNorm",
                 "LayernormDquant", "set_use_triton", "set_autotune_triton_kernels"):
        assert hasattr(flashnn_amd, name)
    assert flashnn_amd.GemmA8W8().out_ty == torch.float16
    assert flashnn_amd.GemmWeightOnly(torch.bfloat16).out_ty == torch.bfloat16
    m = flashnn_amd.RMSNormDquant(64)
    assert m.eps == 1e-6 and m.weight.shape == (64,) and bool((m.weight == 1).all())
    assert flashnn_amd.RMSNorm(64).eps == 1e-6
    for cls in (flashnn_amd.LayerNorm, flashnn_amd.LayernormDquant):      # flashnn/norm.py:70-80, 98-108
        for dim in (64, [64], (64,)):
            n = cls(dim)
            assert n.dim == (64,) and n.eps == 1e-5 and bool((n.weight == 1).all()) and bool((n.bias == 0).all())


def test_hip_backend_never_falls_back_silently():
    x = torch.randn(4, 64).half()
    assert kernel_backend.get_use_triton()
    with pytest.raises(_lib.FlashnnHipError):
        flashnn_amd.DynamicQuantize()(x)          # CPU tensor on the native path: loud error
    with pytest.raises(_lib.FlashnnHipError):
        flashnn_amd.RMSNormDquant(64)(x)
    for mod in (flashnn_amd.RMSNorm(64), flashnn_amd.LayerNorm(64), flashnn_amd.LayernormDquant(64)):
        with pytest.raises(_lib.FlashnnHipError):
            mod.half()(x)


def test_dispatch_and_torch_path_on_cpu():
    class Nothing(kernel_backend.BackendKernel):
        pass

    with pytest.raises(ValueError, match="No valid backend found."):
        Nothing()(1)
    torch.manual_seed(0)
    x = torch.randn(8, 256).half()
    flashnn_amd.set_use_triton(False)
    try:
        q, s = flashnn_amd.DynamicQuantize()(x)
        q_o, s_o = O.dynamic_quantize(O.to_np(x), O.F16)
        assert np.array_equal(q.numpy(), q_o) and np.array_equal(s.numpy(), s_o)
        assert s.dtype == torch.float16 and s.shape == (8,)
        # weight-only torch path, int4 layout, against the oracle
        w = torch.randint(-8, 8, (16, 256), dtype=torch.int8)
        qw = torch.from_numpy(O.pack_int4(w.numpy()))
        scale = torch.empty(4, 16).uniform_(1e-3, 1e-2).half()
        zp = torch.randint(-3, 3, (4, 16)).half()
        out = flashnn_amd.GemmWeightOnly()(x, qw, scale, None, zp)
        want = O.weight_only_gemm(O.to_np(x), w.numpy(), O.to_np(scale), O.to_np(zp), None, O.F16, O.F16, 64, True)
        np.testing.assert_allclose(out.float().numpy(), want, rtol=2e-3, atol=1e-3)
        with pytest.raises(AssertionError, match="only support int8 or int4x2"):
            flashnn_amd.GemmWeightOnly()(x, qw, torch.ones(5).half())
        qn, sn = flashnn_amd.RMSNormDquant(256)(x)
        assert qn.dtype == torch.int8 and sn.dtype == torch.float16 and sn.shape == (8,)
        # the torch paths of the norm layers against the oracle (1 ulp where torch's moments differ)
        y = flashnn_amd.RMSNorm(256).half()(x)
        np.testing.assert_allclose(y.detach().float().numpy(), O.rmsnorm(O.to_np(x), np.ones(256, np.float32), 1e-6, O.F16),
                                   rtol=2.0 ** -10)
        ln = flashnn_amd.LayerNorm(256).half()
        np.testing.assert_allclose(ln(x).detach().float().numpy(),
                                   O.layernorm(O.to_np(x), np.ones(256, np.float32), np.zeros(256, np.float32), 1e-5, O.F16),
                                   rtol=2.0 ** -10, atol=1e-6)
        ql, sl = flashnn_amd.LayernormDquant(256).half()(x)
        assert ql.dtype == torch.int8 and ql.shape == x.shape and sl.shape == (8, 1) and sl.dtype == torch.float16
    finally:
        flashnn_amd.set_use_triton(True)


def test_launcher_asserts_match_the_reference_messages():
    from flashnn_amd import launchers as L
    a = torch.zeros(4, 128, dtype=torch.int8)
    with pytest.raises(AssertionError, match="Matrix A/B must be int8 type"):
        L.hip_gemm_a8w8_forward(torch.empty(4, 4).half(), a.float(), a, torch.ones(4), torch.ones(4))
    with pytest.raises(AssertionError, match="Output type must be float16 or bfloat16"):
        L.hip_gemm_a8w8_forward(torch.empty(4, 4), a, a, torch.ones(4), torch.ones(4))
    with pytest.raises(AssertionError, match="Matrix B must be transposed"):
        L.hip_gemm_a8w8_forward(torch.empty(4, 4).half(), a, a[:, :64].contiguous(), torch.ones(4), torch.ones(4))
    with pytest.raises(AssertionError, match="Weight must be int8 type"):
        L.hip_gemm_a16w8_forward(torch.empty(4, 4).half(), a.half(), a.half(), torch.ones(4).half())
    with pytest.raises(AssertionError, match="input must be contiguous"):
        L.hip_dynamic_quantize(torch.empty(4, 64, dtype=torch.int8), torch.zeros(4, 128).half()[:, ::2],
                               torch.empty(4).half())


def test_tuned_config_file_format_and_lookup(tmp_path, monkeypatch):
    """The tuned-configuration cache keeps the reference's file format
    (flashnn/triton_kernels/triton_utils.py:38-57, 60-75): {method_name: [kwargs, launch options]}."""
    import json
    from flashnn_amd import tuned_configs as TC
    path = tmp_path / "cfg" / "best.json"
    monkeypatch.setenv("FLASHNN_AMD_TUNED_CONFIGS", str(path))
    monkeypatch.delenv("FORECE_RE_TUNE_TRITON_KERNELS", raising=False)
    cache = TC.TunedConfigs()
    assert cache.lookup("gemm_a8w8_2048_12288_4096") is None
    cache.record("gemm_a8w8_2048_12288_4096", (256, 192, 4))
    cache.record("gemm_a8w8_16_4096_4096", (0, 0, 0))
    data = json.load(open(path))
    assert data == {"gemm_a8w8_2048_12288_4096": [{"BLOCK_M": 256, "BLOCK_N": 192}, {"num_warps": 4}],
                    "gemm_a8w8_16_4096_4096": [{"BLOCK_M": 0, "BLOCK_N": 0}, {}]}
    # a fresh view (another process) reads the file back
    other = TC.TunedConfigs()
    assert other.lookup("gemm_a8w8_2048_12288_4096") == (256, 192, 4, 1) and other.lookup("gemm_a8w8_1_1_1") is None
    # forced re-tune by method-name prefix, once per process
    monkeypatch.setenv("FORECE_RE_TUNE_TRITON_KERNELS", "gemm_a8w8_2048;fuse_moe")
    assert TC.force_re_tune("gemm_a8w8_2048_12288_4096") and not TC.force_re_tune("gemm_a8w8_16_4096_4096")
    assert other.lookup("gemm_a8w8_2048_12288_4096") is None and other.lookup("gemm_a8w8_16_4096_4096") == (0, 0, 0, 0)
    other.record("gemm_a8w8_2048_12288_4096", (256, 128, 0))
    assert other.lookup("gemm_a8w8_2048_12288_4096") == (256, 128, 0, 1)
    # the per-shape answer a launcher uses: resolved once, dropped by a new record or reset()
    assert other.shape_tile("gemm_a8w8", 16, 4096, 4096) == (0, 0, 0, 0) and other.shape_tile("gemm_a8w8", 1, 1, 1) is None
    other.record("gemm_a8w8_1_1_1", (64, 128, 0))
    assert other.shape_tile("gemm_a8w8", 1, 1, 1) == (64, 128, 0, 1)
    # a split of K is part of the record (absent = 1)
    other.record("gemm_a8w8_256_4096_8192", (128, 128, 0, 4))
    assert json.load(open(path))["gemm_a8w8_256_4096_8192"] == [{"BLOCK_M": 128, "BLOCK_N": 128, "SPLIT_K": 4}, {}]
    assert TC.TunedConfigs().lookup("gemm_a8w8_256_4096_8192") == (128, 128, 0, 4)
    os.remove(path)
    assert other.shape_tile("gemm_a8w8", 1, 1, 1) == (64, 128, 0, 1)       # answered without touching the file
    other.reset()
    assert other.shape_tile("gemm_a8w8", 1, 1, 1) is None
    assert TC.serialize_best_config((128, 128)) == [{"BLOCK_M": 128, "BLOCK_N": 128}, {}]
    assert TC.deserialize_best_config([{"BLOCK_M": 256, "BLOCK_N": 192}, {}]) == (256, 192, 0, 1)
    assert TC.deserialize_best_config([{"BLOCK_M": 256, "BLOCK_N": 256}, {"num_warps": 4}]) == (256, 256, 4, 1)
    assert TC.deserialize_best_config([{"BLOCK_M": 0, "BLOCK_N": 0}, {}]) == (0, 0, 0, 0)
    assert TC.as_config((128, 128)) == (128, 128, 0, 1) and TC.as_config((0, 0, 0)) == (0, 0, 0, 0)


def test_tiled_entry_rejects_unknown_tiles(hip_lib):
    one = ctypes.c_void_p(16)
    null = ctypes.c_void_p(0)
    rc = hip_lib.fnn_gemm_a8w8_tiled(one, one, one, one, one, 4, 4, 128, 128, 128, 4, 0, 0, 0, 64, 64, 0, null)
    assert rc == -1 and b"no such tile 64x64" in hip_lib.fnn_last_error()
    rc = hip_lib.fnn_gemm_a8w8_tiled(one, one, one, one, one, 4, 4, 128, 128, 128, 4, 0, 0, 0, 128, 128, 8, null)
    assert rc == -1 and b"no such tile 128x128 with 8 waves" in hip_lib.fnn_last_error()
    rc = hip_lib.fnn_gemm_a8w8_i32_tiled(one, one, one, 4, 4, 128, 128, 128, 4, 64, 128, 8, null)
    assert rc == -1 and b"no such tile 64x128 with 8 waves" in hip_lib.fnn_last_error()
    rc = hip_lib.fnn_gemm_a8w8_tiled(one, one, one, one, one, 4, 4, 128, 128, 128, 4, 0, 0, 0, 256, 192, 8, null)
    assert rc == -1 and b"no such tile 256x192 with 8 waves" in hip_lib.fnn_last_error()


def test_a8w8_rejects_row_strides_beyond_the_band_logic(hip_lib):
    one = ctypes.c_void_p(4096)
    null = ctypes.c_void_p(0)
    rc = hip_lib.fnn_gemm_a8w8(one, one, one, one, one, 128, 128, 1024, 1 << 31, 1024, 128, 0, 0, 0, null)
    assert rc == -2 and b"row stride too large" in hip_lib.fnn_last_error()


def test_workspace_entries_reject_bad_arguments(hip_lib):
    one = ctypes.c_void_p(4096)
    odd = ctypes.c_void_p(4100)
    null = ctypes.c_void_p(0)
    base = (one, one, one, one, one, 256, 256, 8192, 8192, 8192, 256, 0, 0, 0)
    assert hip_lib.fnn_workspace_init(null, 1 << 20, null) == -1
    assert hip_lib.fnn_workspace_init(one, 100, null) == -1 and b"at least 4096 bytes" in hip_lib.fnn_last_error()
    assert hip_lib.fnn_gemm_a8w8_ws(*base, odd, 1 << 20, null) == -1 and b"16-byte aligned" in hip_lib.fnn_last_error()
    assert hip_lib.fnn_gemm_a8w8_ws(*base, null, 1 << 20, null) == -1
    # a named split the shape cannot take, an unknown tile for a split, a workspace that is too small
    assert hip_lib.fnn_gemm_a8w8_ws_tiled(*base, 256, 128, 40, one, 1 << 30, null) == -1
    assert b"cannot be split 40 ways" in hip_lib.fnn_last_error()
    assert hip_lib.fnn_gemm_a8w8_ws_tiled(*base, 64, 128, 2, one, 1 << 30, null) == -1
    assert hip_lib.fnn_gemm_a8w8_ws_tiled(*base, 256, 128, 2, one, 8192, null) == -1
    assert b"the split needs 528384" in hip_lib.fnn_last_error()
    assert hip_lib.fnn_gemm_a8w8_ws_tiled(*base, 256, 128, -1, one, 1 << 30, null) == -1
    # which shapes the library would split, and that nothing needs more than 32 MiB + 4 KiB
    f = hip_lib.fnn_gemm_a8w8_workspace_bytes
    assert f(2048, 12288, 4096) == 0 and f(16, 4096, 8192) == 0 and f(512, 8192, 8192) == 0
    assert f(256, 4096, 4096) == 0 and f(1024, 4096, 4096) == 0
    assert f(256, 4096, 8192) == 4096 + 64 * 4 * 65536
    assert f(1024, 1920, 13312) == 4096 + 120 * 2 * 65536        # one unit per CU
    assert f(384, 8192, 14784) == 4096 + 192 * 2 * 65536         # a long K and few tile rows: two units per CU
    assert f(764, 3584, 18944) == 0                              # six tile rows share the weights: unsplit
    assert all(f(M, N, K) <= (32 << 20) + 4096 for M in (65, 100, 128, 500, 1000, 3000) for N in (128, 1000, 4096, 20000)
               for K in (6144, 8192, 16384, 32768))


def test_empty_calls_need_no_addresses(hip_lib):
    """M = 0 / N = 0 returns before anything is launched and accepts NULL tensors (an empty torch tensor
    has data_ptr() == 0); with rows present the same NULLs are rejected."""
    null = ctypes.c_void_p(0)
    assert hip_lib.fnn_dynamic_quant(null, null, null, 0, 4096, 4096, 4096, 0, null) == 0
    assert hip_lib.fnn_dynamic_quant(null, null, null, 1, 4096, 4096, 4096, 0, null) == -1
    assert b"null pointer" in hip_lib.fnn_last_error()
    assert hip_lib.fnn_rmsnorm_dquant(null, null, null, null, 1e-6, 0, 4096, 4096, 4096, 1, 2, null) == 0
    assert hip_lib.fnn_layernorm(null, null, null, null, 1e-5, 0, 4096, 4096, 4096, 0, 0, null) == 0
    assert hip_lib.fnn_gemm_a8w8(null, null, null, null, null, 0, 256, 4096, 4096, 4096, 256, 0, 0, 0, null) == 0
    assert hip_lib.fnn_gemm_a8w8(null, null, null, null, null, 8, 0, 4096, 4096, 4096, 0, 0, 0, 0, null) == 0
    assert hip_lib.fnn_gemm_a8w8(null, null, null, null, null, 8, 256, 4096, 4096, 4096, 256, 0, 0, 0, null) == -1
    assert hip_lib.fnn_gemm_a16w8(null, null, null, null, null, null, 0, 256, 4096, 4096, 4096, 256, 0,
                                  0, 0, 0, 0, 0, null) == 0
