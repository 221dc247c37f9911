"""Backend selection, mirroring flashnn/kernel_backend.py:10-69.

The native backend here is "hip" (libflashnn_hip.so) where the reference has "triton".  The
reference's switch names are kept because callers use them: set_use_triton(False) selects the
torch path, True (the default) the native kernels.  The native path never falls back by
itself: if the library is missing or a tensor is not on a GPU the call raises.
"""
import os

import torch
import torch.nn

autotune_triton_kernels = os.getenv("autotune_triton_kernels", False)
use_triton = os.getenv("USE_TRITON_KERNELS", True)


def get_autotune_triton_kernels():
    return autotune_triton_kernels


def set_autotune_triton_kernels(v: bool):
    """True: the first launch of a shape times the candidate tiles of the A8W8 MFMA kernel and records
    the best in the tuned-configuration file (flashnn_amd/tuned_configs.py); False (the default): recorded
    configurations are used, other shapes take the library's static choice."""
    global autotune_triton_kernels
    autotune_triton_kernels = v


def get_use_triton():
    return use_triton


def set_use_triton(v: bool):
    global use_triton
    use_triton = v


def is_hip():
    return torch.version.hip is not None


THREADS_PER_WARP = 64


class BackendKernel(torch.nn.Module):
    """A kernel with one implementation per backend, `_{backend}_impl`.

    Backends are tried in order ["hip", "torch"]; "hip" is skipped only when the caller has
    switched it off with set_use_triton(False) (flashnn/kernel_backend.py:62-69).
    """

    def __init__(self):
        super().__init__()
        self.backends = ["hip", "torch"]

    def _hip_impl(self, *args, **kwargs):
        raise NotImplementedError

    def _torch_impl(self, *args, **kwargs):
        raise NotImplementedError

    def forward(self, *args, **kwargs):
        for backend in self.backends:
            if backend == "hip" and not get_use_triton():
                continue
            method = getattr(self, f"_{backend}_impl")
            if method.__func__ != getattr(BackendKernel, f"_{backend}_impl"):
                return method(*args, **kwargs)
        raise ValueError("No valid backend found.")
