import ctypes
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
ORACLE_DIR = os.path.join(ROOT, "oracle")
GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def c_oracle():
    """ctypes handle of oracle/liboracle.so (built on demand with plain gcc)."""
    so = os.path.join(ORACLE_DIR, "liboracle.so")
    src = os.path.join(ORACLE_DIR, "dmm_oracle.c")
    if not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "liboracle.so"])
    lib = ctypes.CDLL(so)
    P, I64 = ctypes.c_void_p, ctypes.c_int64
    lib.dmm_oracle_decode_f16.argtypes = [P, P, P, I64]
    lib.dmm_oracle_decode_i8.argtypes = [P, P, P, I64]
    lib.dmm_oracle_decode_swar.argtypes = [P, P, P, I64]
    lib.dmm_oracle_matmul_f16.argtypes = [P, P, ctypes.c_float, P, I64, I64, I64]
    lib.dmm_oracle_decode_matmul_i32.argtypes = [P, P, P, P, I64, I64, I64]
    lib.dmm_oracle_f2h.argtypes = [ctypes.c_float]
    lib.dmm_oracle_f2h.restype = ctypes.c_uint16
    lib.dmm_oracle_h2f.argtypes = [ctypes.c_uint16]
    lib.dmm_oracle_h2f.restype = ctypes.c_float
    return lib


def ptr(a):
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(ctypes.c_void_p)


@pytest.fixture(scope="session")
def all_codes():
    return np.arange(65536, dtype=np.uint16)


def quarter_grid(seed):
    """Seeded half [256,8] grid of odd quarter-units {0.25 .. 2.75}, like the benchmark's."""
    rng = np.random.default_rng(seed)
    vals = np.array([0.25, 0.75, 1.25, 1.75, 2.25, 2.75], dtype=np.float16)
    return vals[rng.integers(0, 6, size=(256, 8))]
