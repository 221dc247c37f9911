"""Launcher functions with the shape of the reference's Triton launchers: the caller
allocates the outputs, the launcher fills them on the current stream.

Each one replaces the reference function named in its docstring and forwards to the C ABI
of libflashnn_hip.so.  The argument checks raise the same exception types with the same
messages as the reference so callers and tests behave identically.
"""
import torch

from . import _lib, tuned_configs
from .kernel_backend import get_autotune_triton_kernels


def hip_dynamic_quantize(out, input, scale):
    """Replaces triton_dynamic_quantize (flashnn/triton_kernels/dynamic_quant.py:73-97)."""
    assert input.is_contiguous(), "input must be contiguous"
    assert input.dim() == 2 and out.shape == input.shape and out.dtype == torch.int8
    assert scale.dtype == torch.float16 and scale.numel() == input.size(0)
    assert out.is_contiguous() and scale.is_contiguous()
    _lib.require_gpu(out, input, scale)
    lib = _lib.load()
    M, K = input.shape
    _lib.check(lib.fnn_dynamic_quant(_lib.ptr(out), _lib.ptr(scale), _lib.ptr(input), M, K,
                                     input.stride(0) if M > 1 else K, out.stride(0) if M > 1 else K,
                                     _lib.dtype_code(input.dtype), _lib.current_stream(input.device)))
    return out, scale


def hip_rmsnorm_dquant_forward(x, weight, eps):
    """Replaces triton_rmsnorm_dquant_forward (flashnn/triton_kernels/rms_norm_dquant.py:80-96)."""
    _lib.require_gpu(x, weight)
    lib = _lib.load()
    y = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    x_arg = _rows(x)
    M, N = x_arg.shape
    # one scale per row, already in the shape the operator returns (a contiguous block of M entries)
    scale = torch.empty(x.shape[:-1], dtype=x.dtype, device=x.device)
    w = _vec(weight, N, "weight")
    _lib.check(lib.fnn_rmsnorm_dquant(_lib.ptr(y), _lib.ptr(scale), _lib.ptr(x_arg), _lib.ptr(w),
                                      float(eps), M, N, N, N, _lib.dtype_code(x.dtype),
                                      _lib.dtype_code(w.dtype), _lib.current_stream(x.device)))
    return y, scale


def _rows(x):
    """x as a contiguous matrix of rows (no view is made of what already is one: a view costs a microsecond)."""
    if x.dim() == 2 and x.is_contiguous():
        return x
    x_arg = x.reshape(-1, x.shape[-1])
    return x_arg if x_arg.is_contiguous() else x_arg.contiguous()


def _vec(t, n, what):
    assert t.numel() == n, f"{what} must have one entry per channel"
    if t.dim() == 1 and t.is_contiguous():
        return t            # only the address is taken: no detached view needed
    t = t.detach().reshape(-1)
    return t if t.is_contiguous() else t.contiguous()


def hip_rmsnorm_forward(x, weight, eps):
    """Replaces triton_rmsnorm_forward (flashnn/triton_kernels/rms_norm.py:68-83)."""
    _lib.require_gpu(x, weight)
    lib = _lib.load()
    y = torch.empty_like(x, memory_format=torch.contiguous_format)
    x_arg = _rows(x)
    M, N = x_arg.shape
    w = _vec(weight, N, "weight")
    _lib.check(lib.fnn_rmsnorm(_lib.ptr(y), _lib.ptr(x_arg), _lib.ptr(w), float(eps), M, N, N, N,
                               _lib.dtype_code(x.dtype), _lib.dtype_code(w.dtype),
                               _lib.current_stream(x.device)))
    return y


def hip_layer_norm_forward(x, weight, bias, eps):
    """Replaces triton_layer_norm_forward (flashnn/triton_kernels/layer_norm.py:84-101)."""
    _lib.require_gpu(x, weight, bias)
    lib = _lib.load()
    y = torch.empty_like(x, memory_format=torch.contiguous_format)
    x_arg = _rows(x)
    M, N = x_arg.shape
    w = _vec(weight, N, "weight")
    b = _vec(bias, N, "bias")
    if b.dtype != w.dtype:
        b = b.to(w.dtype)
    _lib.check(lib.fnn_layernorm(_lib.ptr(y), _lib.ptr(x_arg), _lib.ptr(w), _lib.ptr(b), float(eps), M, N,
                                 N, N, _lib.dtype_code(x.dtype), _lib.dtype_code(w.dtype),
                                 _lib.current_stream(x.device)))
    return y


def hip_layer_norm_dquant_forward(x, weight, bias, eps):
    """Replaces triton_layer_norm_dquant_forward (flashnn/triton_kernels/layer_norm_dquant.py:91-105);
    returns (q int8 like x, scale [rows] in x.dtype) - the normalised tensor the Triton launcher
    also returns is not materialised (its only caller drops it, flashnn/norm.py:107-110)."""
    _lib.require_gpu(x, weight, bias)
    lib = _lib.load()
    x_arg = _rows(x)
    M, N = x_arg.shape
    y = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    scale = torch.empty((M,), dtype=x.dtype, device=x.device)
    w = _vec(weight, N, "weight")
    b = _vec(bias, N, "bias")
    if b.dtype != w.dtype:
        b = b.to(w.dtype)
    _lib.check(lib.fnn_layernorm_dquant(_lib.ptr(y), _lib.ptr(scale), _lib.ptr(x_arg), _lib.ptr(w), _lib.ptr(b),
                                        float(eps), M, N, N, N, _lib.dtype_code(x.dtype),
                                        _lib.dtype_code(w.dtype), _lib.current_stream(x.device)))
    return y, scale


def _flat_scale(t, n, what):
    if t.numel() == n and t.is_contiguous():
        return t            # [n], [n, 1] and [1, n] share one memory layout: no view needed
    if t.dim() != 1:
        t = torch.squeeze(t)
    if t.dim() == 0:
        t = t.reshape(1)
    assert t.dim() == 1 and t.numel() == n, f"{what} must have {n} entries"
    return t if t.is_contiguous() else t.contiguous()


_A8W8_WS_BYTES = {}      # (M, N, K) -> bytes of workspace the library would use for the shape (0: none)
_A8W8_WORKSPACES = {}    # (device index, stream handle) -> zero-initialised workspace tensor


_A8W8_WS_ALLOC = (32 << 20) + 4096      # holds every plan of the library


def _a8w8_workspace(lib, device, stream, M, N, K):
    """The workspace for a shape whose K the library would split over several workgroups per tile, or
    None.  One buffer per device and stream (calls on one stream run in order; calls that overlap in time
    must not share a workspace: a graph captured here and replayed on several streams at once needs the
    C entry point with a workspace per replay), allocated at the first shape that needs one and sized
    for every shape.  It starts zeroed and every call leaves its counters zeroed."""
    need = _A8W8_WS_BYTES.get((M, N, K))
    if need is None:
        need = _A8W8_WS_BYTES[(M, N, K)] = int(lib.fnn_gemm_a8w8_workspace_bytes(M, N, K))
    if need == 0:
        return None
    return _a8w8_workspace_of(device, stream, need)


def _a8w8_workspace_of(device, stream, need):
    """This device's and stream's workspace, at least `need` bytes (and large enough for every plan of the
    library's own)."""
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream)
    ws = _A8W8_WORKSPACES.get(key)
    if ws is None or ws.numel() < need:
        if len(_A8W8_WORKSPACES) >= 16:         # streams come and go: keep the table small
            _A8W8_WORKSPACES.clear()
        ws = _A8W8_WORKSPACES[key] = torch.zeros(max(need, _A8W8_WS_ALLOC), dtype=torch.uint8, device=device)
    return ws


def hip_gemm_a8w8_forward(out, a, b, alpha_row, alpha_col, tile=None):
    """Replaces triton_gemm_a8w8_forward (flashnn/triton_kernels/gemm_a8w8.py:182-221).

    Unlike the Triton launcher the scale type need not equal the output type: fp16, bf16 and
    fp32 scales are accepted in any combination.  `tile` = (rows, columns, waves[, parts of K]) names a
    tile of the MFMA kernel (and a split of K over that many workgroups per tile) and bypasses the
    tuned-configuration lookup (not part of the reference's signature; the results are the same bits for
    every choice)."""
    assert a.dtype == torch.int8 and b.dtype == torch.int8, "Matrix A/B must be int8 type"
    assert a.is_contiguous(), "Matrix A must be contiguous"
    assert out.dtype == torch.float16 or out.dtype == torch.bfloat16, \
        "Output type must be float16 or bfloat16"
    assert a.shape[1] == b.shape[1], "Matrix B must be transposed"
    _lib.require_gpu(out, a, b, alpha_row, alpha_col)
    lib = _lib.load()
    M, K = a.shape
    N = b.shape[0]
    assert out.shape == (M, N) and out.stride(1) == 1
    if b.stride(1) != 1:
        b = b.contiguous()
    ar = _flat_scale(alpha_row, M, "alpha_row")
    ac = _flat_scale(alpha_col, N, "alpha_col")
    args = (_lib.ptr(out), _lib.ptr(a), _lib.ptr(b), _lib.ptr(ar), _lib.ptr(ac),
            M, N, K, a.stride(0) if M > 1 else K, b.stride(0) if N > 1 else K,
            out.stride(0) if M > 1 else N, _lib.dtype_code(out.dtype),
            _lib.dtype_code(ar.dtype), _lib.dtype_code(ac.dtype))
    stream = _lib.current_stream(a.device)
    # shape-keyed tuned tile, named as the reference names the launch (gemm_a8w8.py:199)
    if tile is None:
        tile = tuned_configs.CACHE.shape_tile("gemm_a8w8", M, N, K)
    def run_named(t):
        bm, bn, waves, parts = tuned_configs.as_config(t)
        if bm == 0:
            return run_default()
        if parts > 1:
            ws = _a8w8_workspace_of(a.device, stream, _A8W8_WS_ALLOC)
            rc = lib.fnn_gemm_a8w8_ws_tiled(*args, bm, bn, parts, ws.data_ptr(), ws.numel(), stream)
            if rc != 0:
                _A8W8_WORKSPACES.clear()
            return _lib.check(rc)
        return _lib.check(lib.fnn_gemm_a8w8_tiled(*args, bm, bn, waves, stream))

    def run_default():
        ws = _a8w8_workspace(lib, a.device, stream, M, N, K) if M > 64 else None
        if ws is None:
            _lib.check(lib.fnn_gemm_a8w8(*args, stream))
        else:
            rc = lib.fnn_gemm_a8w8_ws(*args, ws.data_ptr(), ws.numel(), stream)
            if rc != 0:
                # a split call that failed half way may have left counters behind: never reuse the buffer
                _A8W8_WORKSPACES.clear()
            _lib.check(rc)

    if tile is None and get_autotune_triton_kernels():
        tile = tuned_configs.tune(f"gemm_a8w8_{M}_{N}_{K}", tuned_configs.A8W8_CANDIDATES, run_named)
    if tile is None:
        run_default()
    else:
        run_named(tile)
    return out


def hip_gemm_a8w8_int32(a, b, tile=(0, 0, 0)):
    """Raw int32 accumulators of the A8W8 contraction (no reference launcher; parity hook).
    `tile` = (rows, columns, waves) names a tile of the MFMA kernel; (0, 0, 0) leaves the choice to the
    library."""
    assert a.dtype == torch.int8 and b.dtype == torch.int8, "Matrix A/B must be int8 type"
    assert a.is_contiguous() and b.is_contiguous() and a.shape[1] == b.shape[1]
    _lib.require_gpu(a, b)
    lib = _lib.load()
    M, K = a.shape
    N = b.shape[0]
    acc = torch.empty((M, N), dtype=torch.int32, device=a.device)
    _lib.check(lib.fnn_gemm_a8w8_i32_tiled(_lib.ptr(acc), _lib.ptr(a), _lib.ptr(b), M, N, K, K, K, N, *tile,
                                           _lib.current_stream(a.device)))
    return acc


def _weight_only(fn_name, out, act, quant_w, scale_w, bias, zero_points, n_out, tile=None):
    assert quant_w.dtype == torch.int8, "Weight must be int8 type"
    assert act.is_contiguous(), "Activation must be contiguous"
    assert quant_w.is_contiguous(), "Weight must be contiguous"
    assert act.shape[1] == quant_w.shape[1], "Matrix B must be transposed"
    _lib.require_gpu(out, act, quant_w, scale_w, bias, zero_points)
    lib = _lib.load()
    M, K = act.shape
    N = n_out
    assert out.shape == (M, N) and out.stride(1) == 1
    # the common layouts ([N] or [K/g, N], contiguous) pass through without creating views
    if not (scale_w.dim() == 1 or (scale_w.dim() == 2 and scale_w.shape[0] > 1 and scale_w.shape[1] == N)):
        scale_w = scale_w.squeeze()
    if scale_w.dim() <= 1:
        group = 0
        if scale_w.dim() == 0:
            scale_w = scale_w.reshape(-1)
        assert scale_w.numel() == N
    else:
        assert scale_w.dim() == 2 and scale_w.shape[1] == N
        group = int(K / scale_w.shape[0])
        assert group > 0, "k_per_scale should greater than 0"
        assert group * scale_w.shape[0] == K, "K must be a multiple of the scale rows"
    if not scale_w.is_contiguous():
        scale_w = scale_w.contiguous()
    zp = None
    if zero_points is not None:
        zp = zero_points
        if zp.shape != scale_w.shape:
            zp = zp.squeeze().reshape(scale_w.shape)
        if not zp.is_contiguous():
            zp = zp.contiguous()
        if zp.dtype != scale_w.dtype:
            zp = zp.to(scale_w.dtype)   # zero points are small integers: exact in any float type
    if bias is not None:
        if bias.dim() != 1 or not bias.is_contiguous():
            bias = bias.reshape(-1).contiguous()
        assert bias.numel() == N
    args = (_lib.ptr(out), _lib.ptr(act), _lib.ptr(quant_w), _lib.ptr(scale_w), _lib.ptr(bias),
            _lib.ptr(zp), M, N, K, act.stride(0) if M > 1 else K, K,
            out.stride(0) if M > 1 else N, group, _lib.dtype_code(act.dtype),
            _lib.dtype_code(out.dtype), _lib.dtype_code(scale_w.dtype),
            _lib.dtype_code(zp.dtype) if zp is not None else 0,
            _lib.dtype_code(bias.dtype) if bias is not None else 0)
    # scratch for bf16 rows converted to fp16 (so that every weight is rounded as the reference rounds it): taken
    # from torch's caching allocator per call, which hands it to later calls on this stream in stream order
    def run_default():
        need = 0
        if M > 64 and act.dtype == torch.bfloat16:
            need = int(lib.fnn_gemm_weight_only_workspace_bytes(M, N, K, group, _lib.dtype_code(act.dtype),
                                                                _lib.dtype_code(scale_w.dtype)))
        if need:
            ws = torch.empty(need, dtype=torch.uint8, device=act.device)
            _lib.check(getattr(lib, fn_name + "_ws")(*args, ws.data_ptr(), need, _lib.current_stream(act.device)))
        else:
            _lib.check(getattr(lib, fn_name)(*args, _lib.current_stream(act.device)))

    def run_named(t):
        bm, bn = tuned_configs.as_config(t)[:2]
        if bm == 0:
            return run_default()
        return _lib.check(getattr(lib, fn_name + "_tiled")(*args, bm, bn, _lib.current_stream(act.device)))

    # Up to 64 rows the blocks of the few-row kernel can be named: a shape-keyed record, written by a tuning run
    # under the name of the reference's kernel for the call (gemm_a16w8.py:84, :180; gemm_a16w4.py:84, :210) with
    # the shape it is tuned by there (key M, N, K; gemm_a16w8.py:322-336), and the group size where there is one
    if M <= 64:
        prefix = fn_name[4:] + ("_per_channel" if group == 0 else f"_sub_channel_g{group}")
        if tile is None:
            tile = tuned_configs.CACHE.shape_tile(prefix, M, N, K)
        if tile is None and get_autotune_triton_kernels():
            tile = tuned_configs.tune(f"{prefix}_{M}_{N}_{K}", tuned_configs.weight_only_candidates(N // quant_w.shape[0]),
                                      run_named)
    if tile is None:
        run_default()
    else:
        run_named(tile)
    return out


def hip_gemm_a16w8_forward(out, act, quant_w, scale_w, bias=None, zero_points=None, tile=None):
    """Replaces triton_gemm_a16w8_forward (flashnn/triton_kernels/gemm_a16w8.py:275-338).
    `out` need not be zeroed.  `tile` = (rows per pass, channels per workgroup) names the blocks of the few-row
    kernel (up to 64 rows) and bypasses the tuned-configuration lookup (not part of the reference's signature)."""
    return _weight_only("fnn_gemm_a16w8", out, act, quant_w, scale_w, bias, zero_points,
                        quant_w.shape[0], tile)


def hip_gemm_a16w4_forward(out, act, quant_w, scale_w, bias=None, zero_points=None, tile=None):
    """Replaces triton_gemm_a16w4_forward (flashnn/triton_kernels/gemm_a16w4.py:336-406).
    quant_w is [N/2, K] with channel 2j in the low and 2j+1 in the high nibble of row j.  `tile` as in
    hip_gemm_a16w8_forward."""
    return _weight_only("fnn_gemm_a16w4", out, act, quant_w, scale_w, bias, zero_points,
                        quant_w.shape[0] * 2, tile)


class PrepackedInt4:
    """int4 weights with groups of 128 in the library's packed form (see hip_a16w4_prepack): the buffer and
    the shape it stands for."""

    version = 1     # of the packed layout (written out in csrc/gemm_wo_prepacked.hip)

    def __init__(self, buffer, n, k, group):
        self.buffer, self.n, self.k, self.group = buffer, n, k, group


def hip_a16w4_prepack(quant_w, scale_w, zero_points=None):
    """Repack int4 weights in the reference layout (quant_w [N/2, K] int8 as GemmWeightOnly takes them,
    flashnn/quant_gemm.py:174-204; scale_w and zero_points [K/128, N] fp16) into one stream, made for the
    decode of one or a few tokens.  Returns a PrepackedInt4; the originals are not modified and can be freed.  No
    counterpart in the reference, whose launcher reads the layout above as it is (gemm_a16w4.py:336-406)."""
    assert quant_w.dtype == torch.int8 and quant_w.dim() == 2 and quant_w.stride(1) == 1, "Weight must be int8 type"
    assert scale_w.dim() == 2 and scale_w.dtype == torch.float16 and scale_w.is_contiguous(), \
        "the packed form takes fp16 scales per group of 128"
    _lib.require_gpu(quant_w, scale_w, zero_points)
    lib = _lib.load()
    K = quant_w.shape[1]
    N = quant_w.shape[0] * 2
    assert scale_w.shape[1] == N and scale_w.shape[0] * 128 == K, "the packed form takes groups of 128"
    zp = None
    if zero_points is not None:
        zp = zero_points.reshape(scale_w.shape).to(torch.float16).contiguous()
    size = int(lib.fnn_a16w4_prepacked_bytes(N, K, 128))
    if size == 0:
        raise _lib.FlashnnHipError(f"no packed form for N={N} K={K} (needs N % 16 == 0 and K % 1024 == 0)")
    buf = torch.empty(size, dtype=torch.uint8, device=quant_w.device)
    _lib.check(lib.fnn_a16w4_prepack(_lib.ptr(buf), _lib.ptr(quant_w), _lib.ptr(scale_w), _lib.ptr(zp), N, K,
                                     quant_w.stride(0), 128, _lib.dtype_code(scale_w.dtype), _lib.FNN_F16,
                                     _lib.current_stream(quant_w.device)))
    return PrepackedInt4(buf, N, K, 128)


def hip_gemm_a16w4_prepacked_forward(out, act, packed, bias=None):
    """triton_gemm_a16w4_forward (flashnn/triton_kernels/gemm_a16w4.py:336-406) on weights packed by
    hip_a16w4_prepack: any number of activation rows (one row and up to 64 rows are what the packed form
    is fast for)."""
    assert isinstance(packed, PrepackedInt4)
    assert act.is_contiguous(), "Activation must be contiguous"
    assert act.dim() == 2 and act.shape[1] == packed.k, "Matrix B must be transposed"
    _lib.require_gpu(out, act, packed.buffer, bias)
    lib = _lib.load()
    M = act.shape[0]
    assert out.shape == (M, packed.n) and out.stride(1) == 1
    if bias is not None:
        if bias.dim() != 1 or not bias.is_contiguous():
            bias = bias.reshape(-1).contiguous()
        assert bias.numel() == packed.n
    _lib.check(lib.fnn_gemm_a16w4_prepacked(_lib.ptr(out), _lib.ptr(act), _lib.ptr(packed.buffer), _lib.ptr(bias), M,
                                            packed.n, packed.k, act.stride(0) if M > 1 else packed.k,
                                            out.stride(0) if M > 1 else packed.n, packed.group,
                                            _lib.dtype_code(act.dtype), _lib.dtype_code(out.dtype),
                                            _lib.dtype_code(bias.dtype) if bias is not None else 0,
                                            _lib.current_stream(act.device)))
    return out
