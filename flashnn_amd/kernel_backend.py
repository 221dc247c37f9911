"""Backend selection with the interface of flashnn/kernel_backend.py:10-69.

The native backend here is "hip" (libflashnn_hip.so) where the reference has "triton".  The reference's
switch names are kept because callers use them: set_use_triton(False) selects the torch formulas, True (the
default) the native kernels.  The native path never falls back by itself: if the library is missing or a
tensor is not on a GPU the call raises.
"""
import os

import torch.nn


def _env_switch(name, default):
    """An environment variable as a switch: unset -> default; "", "0", "false", "off", "no" -> False; any
    other text -> True.  (The reference takes any non-empty text as True, flashnn/kernel_backend.py:10-11;
    "0" switching a flag on helps nobody.)"""
    text = os.environ.get(name)
    if text is None:
        return default
    return text.strip().lower() not in ("", "0", "false", "off", "no")


class _Switches:
    """The two process-wide flags of the reference's module, in one place."""
    native = _env_switch("USE_TRITON_KERNELS", True)
    autotune = _env_switch("autotune_triton_kernels", False)


def get_autotune_triton_kernels():
    return _Switches.autotune


def set_autotune_triton_kernels(v: bool):
    """True: the first launch of a shape times the candidate tiles of the A8W8 MFMA kernel and records
    the best in the tuned-configuration file (flashnn_amd/tuned_configs.py); False (the default): recorded
    configurations are used, other shapes take the library's static choice."""
    _Switches.autotune = bool(v)


def get_use_triton():
    return _Switches.native


def set_use_triton(v: bool):
    _Switches.native = bool(v)


class BackendKernel(torch.nn.Module):
    """An operator with a native implementation, `_hip_impl`, and a torch one, `_torch_impl`; a subclass
    defines one or both.  forward() runs the native one unless set_use_triton(False) is in force or the
    subclass has none, then the torch one; with neither it raises ValueError("No valid backend found."),
    as flashnn/kernel_backend.py:62-69 does.  An error inside the chosen implementation propagates: there
    is no second attempt on the other backend."""

    def _hip_impl(self, *args, **kwargs):
        raise NotImplementedError

    def _torch_impl(self, *args, **kwargs):
        raise NotImplementedError

    def _implements(self, name):
        return getattr(type(self), name) is not getattr(BackendKernel, name)

    def forward(self, *args, **kwargs):
        if _Switches.native and self._implements("_hip_impl"):
            return self._hip_impl(*args, **kwargs)
        if self._implements("_torch_impl"):
            return self._torch_impl(*args, **kwargs)
        raise ValueError("No valid backend found.")
