import ctypes
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def c_oracle():
    """The C restatement of the oracle, built on demand (CPU only)."""
    path = os.path.join(ROOT, "oracle", "libmxfp8_oracle.so")
    if not os.path.exists(path):
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True, capture_output=True)
    lib = ctypes.CDLL(path)
    lib.plko_e4m3_decode.restype = ctypes.c_float
    lib.plko_e4m3_decode.argtypes = [ctypes.c_uint8]
    lib.plko_e4m3_encode.restype = ctypes.c_uint8
    lib.plko_e4m3_encode.argtypes = [ctypes.c_float]
    lib.plko_e8m0_decode.restype = ctypes.c_float
    lib.plko_e8m0_decode.argtypes = [ctypes.c_uint8]
    lib.plko_e8m0_from_amax.restype = ctypes.c_uint8
    lib.plko_e8m0_from_amax.argtypes = [ctypes.c_float]
    lib.plko_bf16_round.restype = ctypes.c_float
    lib.plko_bf16_round.argtypes = [ctypes.c_float]
    lib.plko_swiglu.restype = ctypes.c_float
    lib.plko_swiglu.argtypes = [ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_int]
    lib.plko_mx_quantize.restype = None
    lib.plko_mx_quantize.argtypes = [ctypes.c_void_p, ctypes.c_long, ctypes.c_long, ctypes.c_long,
                                     ctypes.c_void_p, ctypes.c_void_p]
    lib.plko_moe_forward.restype = None
    lib.plko_moe_forward.argtypes = [ctypes.c_void_p] * 10 + [ctypes.c_int] + [ctypes.c_long] * 4 + \
        [ctypes.c_float, ctypes.c_int] + [ctypes.c_void_p] * 3
    return lib
