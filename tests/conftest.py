import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def hip_lib():
    from flashnn_amd import _lib
    return _lib.load()


@pytest.fixture(scope="session")
def oracle_c():
    """The C restatement of the integer GEMM (oracle/int8_gemm.c), built on demand."""
    import ctypes
    import subprocess
    d = os.path.join(ROOT, "oracle")
    so = os.path.join(d, "liboracle_int8.so")
    if not os.path.exists(so):
        subprocess.check_call(["make", "-C", d])
    lib = ctypes.CDLL(so)
    i64, p = ctypes.c_int64, ctypes.c_void_p
    lib.fnn_oracle_int8_gemm.argtypes = [p, p, p, i64, i64, i64, i64, i64, i64]
    lib.fnn_oracle_int8_gemm.restype = None
    lib.fnn_oracle_a8w8_epilogue.argtypes = [p, p, p, p, i64, i64]
    lib.fnn_oracle_a8w8_epilogue.restype = None
    return lib


def pytest_terminal_summary(terminalreporter):
    """Weight-only cases in which some outputs left rtol/atol 1e-2 of the reference-rounding oracle (they
    passed because each such output is closer to the float64 value than the oracle's): name and count."""
    mod = sys.modules.get("test_gpu_parity") or sys.modules.get("tests.test_gpu_parity")
    breaches = getattr(mod, "WO_BREACHES", None)
    if breaches:
        terminalreporter.write_line(f"weight-only outputs beyond rtol/atol 1e-2 of the oracle in {len(breaches)} cases "
                                    "(each at least as close to float64 as the oracle):")
        for case, nbad, total in breaches:
            terminalreporter.write_line(f"  {case}: {nbad} of {total}")
