"""The entry point that allocates nothing: fnn_gemm_a8w8_static keeps the workspace of the split-K kernel in
an array of the library's own instead of taking one from the caller.  Checked against fnn_gemm_a8w8_ws_tiled
(caller-provided workspace), bit for bit, on two calls in a row, the second on a smaller input."""
import sys

import numpy as np
import pytest
import torch

from flashnn_amd import _lib
from oracle import flashnn_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _inputs(M, N, K, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    a = torch.randint(-128, 128, (M, K), dtype=torch.int8, device=DEV, generator=g)
    b = torch.randint(-128, 128, (N, K), dtype=torch.int8, device=DEV, generator=g)
    ar = (torch.rand(M, device=DEV, generator=g) * 1e-2 + 1e-3).half()
    ac = (torch.rand(N, device=DEV, generator=g) * 1e-2 + 1e-3).float()
    return a, b, ar, ac


def _args(out, a, b, ar, ac):
    M, K = a.shape
    N = b.shape[0]
    return (out.data_ptr(), a.data_ptr(), b.data_ptr(), ar.data_ptr(), ac.data_ptr(), M, N, K, K, K, N,
            _lib.dtype_code(out.dtype), _lib.dtype_code(ar.dtype), _lib.dtype_code(ac.dtype))


def test_static_workspace_entry_matches_the_workspace_entry(hip_lib):
    st = _lib.current_stream(torch.device(DEV))
    ws = torch.zeros(16 << 20, dtype=torch.uint8, device=DEV)
    # (shape, named plan): the library's own choice on a large and then a smaller input, then named splits -
    # the last one smaller again and with more parts than the call before it
    cases = [((384, 1920, 13312), (0, 0, 0)), ((320, 1024, 8192), (0, 0, 0)), ((300, 520, 8192), (256, 192, 3)),
             ((96, 200, 4128), (128, 128, 5)), ((2048, 4096, 4096), (0, 0, 0))]
    for (M, N, K), plan in cases:
        print(f"[gpu-case] static workspace M={M} N={N} K={K} plan={plan}", file=sys.__stderr__, flush=True)
        a, b, ar, ac = _inputs(M, N, K, M + N + K)
        want = torch.full((M, N), 3.0, dtype=torch.bfloat16, device=DEV)
        assert hip_lib.fnn_gemm_a8w8_ws_tiled(*_args(want, a, b, ar, ac), *plan, ws.data_ptr(), ws.numel(), st) == 0
        kernel = _lib.last_kernel()
        got = torch.full((M, N), 5.0, dtype=torch.bfloat16, device=DEV)
        torch.cuda.synchronize()
        held, reserved = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
        assert hip_lib.fnn_gemm_a8w8_static(*_args(got, a, b, ar, ac), *plan, st) == 0, hip_lib.fnn_last_error()
        assert _lib.last_kernel() == kernel and ("split K" in kernel) == (M < 2048)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == held and torch.cuda.memory_reserved() == reserved
        assert torch.equal(got, want)
        rows = slice(0, 4)
        ref = O.gemm_a8w8_epilogue_fp32(O.gemm_a8w8_acc(a[rows].cpu().numpy(), b.cpu().numpy()), O.to_np(ar[rows].cpu()),
                                        ac.cpu().numpy(), O.BF16)
        assert np.array_equal(got[rows].float().cpu().numpy(), ref)


def test_static_workspace_entry_rejects_what_does_not_fit(hip_lib):
    a, b, ar, ac = _inputs(1024, 1920, 13312, 5)
    out = torch.empty(1024, 1920, dtype=torch.bfloat16, device=DEV)
    st = _lib.current_stream(torch.device(DEV))
    rc = hip_lib.fnn_gemm_a8w8_static(*_args(out, a, b, ar, ac), 256, 192, 6, st)
    msg = hip_lib.fnn_last_error()
    assert rc == -2 and b"needs 47190016 bytes" in msg and b"holds 16777216" in msg
    # the same shape with a split that fits, and with the library's own choice
    assert hip_lib.fnn_gemm_a8w8_static(*_args(out, a, b, ar, ac), 256, 192, 2, st) == 0
    want = torch.empty_like(out)
    assert hip_lib.fnn_gemm_a8w8(*_args(want, a, b, ar, ac), st) == 0
    assert torch.equal(out, want)
    assert hip_lib.fnn_gemm_a8w8_static(*_args(out, a, b, ar, ac), 0, 0, 0, st) == 0
    assert torch.equal(out, want)
    # the counters of the library's own workspace can be cleared from outside (after a failed call)
    assert hip_lib.fnn_workspace_init(None, 0, st) == 0, hip_lib.fnn_last_error()
    out.zero_()
    assert hip_lib.fnn_gemm_a8w8_static(*_args(out, a, b, ar, ac), 0, 0, 0, st) == 0
    assert torch.equal(out, want)
