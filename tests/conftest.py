import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (checker only)."""
    from oracle import pyoracle
    pyoracle.lib()
    return pyoracle


class _InternalPlan(__import__("ctypes").Structure):
    """Mirror of mi_internal_plan (csrc/internal.h): kernel-selection overrides, zero = the library's heuristic."""
    _fields_ = [(n, __import__("ctypes").c_int) for n in (
        "a16_waves", "a16_tpw", "a16_rows", "a16_xlds", "a16_no_gemm", "a16_no_decode", "a16_gemm_min_m", "a16_gemm_splits",
        "a16_gemm_tile", "a16_gemm_rows", "i8_tile", "i8_mid_ring", "i8_ring", "dq_waves", "f8_tile", "a16_decode_rows8", "a16_rows32_min_m", "a16_wide_min_m", "a16_wide4_min_m", "a16_rows32_split")]


@pytest.fixture
def plan():
    """plan(a16_gemm_min_m=17, ...) steers the library to a given kernel instance for the rest of the test (the
    library's internal hook, bound by name: it is not part of the C ABI); the heuristics come back afterwards."""
    import ctypes
    import importlib
    L = importlib.import_module("tpu-mlir_amd.clib").lib()
    L.mi_internal_set_plan.argtypes = [ctypes.c_void_p]
    L.mi_internal_set_plan.restype = None

    def set_plan(**fields):
        rec = _InternalPlan(**fields)
        L.mi_internal_set_plan(ctypes.byref(rec))

    yield set_plan
    L.mi_internal_set_plan(None)
