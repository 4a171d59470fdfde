import ctypes
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def ck_ref():
    """oracle/_ref/libck_ref.so: host code of the reference's vendored ck_tile, compiled in place."""
    path = os.path.join(ROOT, "oracle", "_ref", "libck_ref.so")
    if not os.path.exists(path):
        pytest.skip("oracle/_ref/libck_ref.so not built (needs /root/reference; run make -C oracle/ref_build)")
    lib = ctypes.CDLL(path)
    lib.ck_ref_moe_sorting.restype = ctypes.c_int
    lib.ck_ref_pack.restype = ctypes.c_uint8
    return lib


def ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def ck_sort(lib, topk_ids, topk_w, E, unit, mask=None):
    ids = np.ascontiguousarray(topk_ids, dtype=np.int32)
    w = np.ascontiguousarray(topk_w, dtype=np.float32)
    T, k = ids.shape
    cap = (T * k + E * (unit - 1) + unit - 1) // unit * unit + unit
    so = np.zeros(cap, np.int32)
    sw = np.zeros(cap, np.float32)
    se = np.zeros(cap // unit + 1, np.int32)
    m = None if mask is None else np.ascontiguousarray(mask, dtype=np.int32)
    n = lib.ck_ref_moe_sorting(ptr(ids), ptr(w), T, k, E, unit, None if m is None else ptr(m),
                               ptr(so), ptr(sw), ptr(se), cap)
    return so[:n].view(np.uint32), sw[:n], se[: n // unit].view(np.uint32), n
