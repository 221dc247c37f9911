"""ctypes binding of libflashnn_hip.so (the C ABI declared in include/flashnn_hip.h)."""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libflashnn_hip.so")

FNN_F16, FNN_BF16, FNN_F32 = 0, 1, 2
_DTYPE_CODE = {torch.float16: FNN_F16, torch.bfloat16: FNN_BF16, torch.float32: FNN_F32}
FNN_I8 = 3   # accepted for the zero points of fnn_fused_moe_a16w4 only

_i64, _int, _ptr, _f32, _size = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_float, ctypes.c_size_t

# name -> argument types; every function returns int unless listed in _RESTYPE
_SIGNATURES = {
    "fnn_version": [],
    "fnn_last_error": [],
    "fnn_last_kernel": [],
    "fnn_dynamic_quant": [_ptr, _ptr, _ptr, _i64, _i64, _i64, _i64, _int, _ptr],
    "fnn_rmsnorm_dquant": [_ptr, _ptr, _ptr, _ptr, _f32, _i64, _i64, _i64, _i64, _int, _int, _ptr],
    "fnn_rmsnorm": [_ptr, _ptr, _ptr, _f32, _i64, _i64, _i64, _i64, _int, _int, _ptr],
    "fnn_layernorm": [_ptr, _ptr, _ptr, _ptr, _f32, _i64, _i64, _i64, _i64, _int, _int, _ptr],
    "fnn_layernorm_dquant": [_ptr, _ptr, _ptr, _ptr, _ptr, _f32, _i64, _i64, _i64, _i64, _int, _int, _ptr],
    "fnn_gemm_a8w8": [_ptr] * 5 + [_i64] * 6 + [_int] * 3 + [_ptr],
    "fnn_gemm_a8w8_tiled": [_ptr] * 5 + [_i64] * 6 + [_int] * 6 + [_ptr],
    "fnn_gemm_a8w8_workspace_bytes": [_i64] * 3,
    "fnn_workspace_init": [_ptr, _size, _ptr],
    "fnn_gemm_a8w8_ws": [_ptr] * 5 + [_i64] * 6 + [_int] * 3 + [_ptr, _size, _ptr],
    "fnn_gemm_a8w8_ws_tiled": [_ptr] * 5 + [_i64] * 6 + [_int] * 6 + [_ptr, _size, _ptr],
    "fnn_gemm_a8w8_static": [_ptr] * 5 + [_i64] * 6 + [_int] * 6 + [_ptr],
    "fnn_gemm_a8w8_i32": [_ptr] * 3 + [_i64] * 6 + [_ptr],
    "fnn_gemm_a8w8_i32_tiled": [_ptr] * 3 + [_i64] * 6 + [_int] * 3 + [_ptr],
    "fnn_gemm_a16w8": [_ptr] * 6 + [_i64] * 7 + [_int] * 5 + [_ptr],
    "fnn_gemm_a16w4": [_ptr] * 6 + [_i64] * 7 + [_int] * 5 + [_ptr],
    "fnn_gemm_weight_only_workspace_bytes": [_i64] * 4 + [_int] * 2,
    "fnn_gemm_a16w8_ws": [_ptr] * 6 + [_i64] * 7 + [_int] * 5 + [_ptr, _size, _ptr],
    "fnn_gemm_a16w4_ws": [_ptr] * 6 + [_i64] * 7 + [_int] * 5 + [_ptr, _size, _ptr],
    "fnn_gemm_a16w8_tiled": [_ptr] * 6 + [_i64] * 7 + [_int] * 7 + [_ptr],
    "fnn_gemm_a16w4_tiled": [_ptr] * 6 + [_i64] * 7 + [_int] * 7 + [_ptr],
    "fnn_a16w4_prepacked_bytes": [_i64] * 3,
    "fnn_a16w4_prepack": [_ptr] * 4 + [_i64] * 4 + [_int] * 2 + [_ptr],
    "fnn_gemm_a16w4_prepacked": [_ptr] * 4 + [_i64] * 6 + [_int] * 3 + [_ptr],
    "fnn_fused_moe_a8w8": [_ptr] * 9 + [_i64] * 9 + [_int] * 7 + [_ptr],
    "fnn_fused_moe_a16w4": [_ptr] * 9 + [_i64] * 14 + [_int] * 8 + [_ptr],
}
_RESTYPE = {"fnn_last_error": ctypes.c_char_p, "fnn_last_kernel": ctypes.c_char_p,
            "fnn_gemm_a8w8_workspace_bytes": ctypes.c_size_t, "fnn_a16w4_prepacked_bytes": ctypes.c_size_t,
            "fnn_gemm_weight_only_workspace_bytes": ctypes.c_size_t}

_lib = None


class FlashnnHipError(RuntimeError):
    """A libflashnn_hip.so entry point returned a non-zero status."""


def exported_symbols():
    return sorted(_SIGNATURES)


def load():
    """Load the HIP library; raises if it has not been built (there is no other backend
    to fall back to - the torch path is only used when the caller selects it)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FlashnnHipError(
            f"{LIB_PATH} is missing: build it with `make -C flashnn_amd/csrc` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = _RESTYPE.get(name, ctypes.c_int)
    _lib = lib
    return lib


def dtype_code(dt):
    try:
        return _DTYPE_CODE[dt]
    except KeyError:
        raise TypeError(f"unsupported dtype {dt}") from None


def current_stream(device):
    """Raw hipStream_t of torch's current stream on `device` (an int; 0 is the null stream)."""
    idx = device.index
    if idx is None:
        idx = torch.cuda.current_device()
    return torch._C._cuda_getCurrentRawStream(idx)


def ptr(t):
    """Device address as an int (None -> NULL); ctypes converts it for a void* parameter."""
    return t.data_ptr() if t is not None else None


def check(rc):
    if rc != 0:
        msg = load().fnn_last_error().decode("utf-8", "replace")
        raise FlashnnHipError(f"libflashnn_hip error {rc}: {msg}")


def last_kernel():
    """Name of the kernel the calling thread's last library call launched (fnn_last_kernel)."""
    return load().fnn_last_kernel().decode("ascii", "replace")


def require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise FlashnnHipError(
                "the HIP backend needs tensors on a GPU; call set_use_triton(False) to select "
                "the torch path explicitly")
