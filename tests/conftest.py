import ctypes
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _have_gpu() -> bool:
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _have_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def cref():
    """The integer-only C restatement of the codec (oracle/q40_ref.c), built on demand."""
    path = os.path.join(ROOT, "oracle", "libq40ref.so")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    lib = ctypes.CDLL(path)
    lib.q40_ref_mul.restype = ctypes.c_uint16
    lib.q40_ref_mul.argtypes = [ctypes.c_int, ctypes.c_uint16]
    lib.q40_ref_scale.restype = ctypes.c_uint16
    lib.q40_ref_scale.argtypes = [ctypes.c_uint16]
    lib.q40_ref_code.restype = ctypes.c_int
    lib.q40_ref_code.argtypes = [ctypes.c_uint16, ctypes.c_uint16]
    lib.q40_ref_dequant_table.argtypes = [ctypes.c_void_p]
    lib.q40_ref_dequantize.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_long, ctypes.c_void_p]
    lib.q40_ref_quantize.argtypes = [ctypes.c_void_p, ctypes.c_long, ctypes.c_void_p, ctypes.c_void_p]
    return lib
