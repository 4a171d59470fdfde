"""CPU checks of the boundary: the shared library loads and exports every symbol that
include/pyhip_moe.h declares, the ctypes table covers exactly those symbols, and the argument
checks reject bad input without touching a GPU."""
import ctypes
import os
import re

import pytest

from pyhip_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "pyhip_moe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pyhip_moe_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared()
    assert len(names) >= 9
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(_lib.SIGNATURES) == names
    assert lib.pyhip_moe_abi_version() == 9


def test_size_helpers():
    lib = _lib.load()
    assert lib.pyhip_moe_sorting_max_blocks(64, 2, 8, 16) == (128 + 8 * 15 + 15) // 16
    assert lib.pyhip_moe_act_scale_stride(7168) == 224 and lib.pyhip_moe_act_scale_stride(1024) == 32
    assert lib.pyhip_moe_act_scale_stride(2880) == 96
    assert lib.pyhip_moe_sorting_workspace_bytes(16, 8, 256) >= 0
    assert lib.pyhip_moe_schedule_words(256) == 513


def test_argument_errors_are_reported():
    lib = _lib.load()
    rc = lib.pyhip_moe_sorting(None, None, 4, 2, 8, 16, None, None, None, None, None, None, None, None, 0, None, 0, None)
    assert rc == 1
    with pytest.raises(_lib.PyhipError, match="null pointer"):
        _lib.check(rc, "moe_sorting")
    one = ctypes.c_void_p(16)
    rc = lib.pyhip_moe_act_quant_mxfp4(one, 40, 4, 40, one, one, None, None)
    assert rc == 1 and b"multiple of 32" in lib.pyhip_moe_last_error()
    # the sort that carries the input quantisation checks the quantiser's arguments before anything is launched
    rc = lib.pyhip_moe_sorting_quant(one, one, 4, 2, 8, 16, None, None, one, one, one, one, None, one, 256,
                                     one, 1024, 4, 1000, one, one, None)
    assert rc == 1 and b"multiple of 32" in lib.pyhip_moe_last_error()
    rc = lib.pyhip_moe_sorting_quant(one, one, 4, 2, 8, 16, None, None, one, one, one, one, None, one, 256,
                                     None, 1024, 4, 1024, one, one, None)
    assert rc == 1 and b"null pointer" in lib.pyhip_moe_last_error()
    rc = lib.pyhip_moe_gemm1_mxfp4(one, one, one, one, None, one, one, one, None, one, None, None, 4, 2, 8, 1000, 512, 0, 0, 16, 4, 0, 0.0, None)
    assert rc == 1 and b"multiple of 512" in lib.pyhip_moe_last_error()
    rc = lib.pyhip_moe_gemm2_mxfp4(one, one, one, one, None, one, one, one, one, None, one, 4, 2, 8, 1024, 512, 0, 0, 48, 4, None)
    assert rc == 1 and b"block_m" in lib.pyhip_moe_last_error()
    # pads are a part of the size they pad
    rc = lib.pyhip_moe_gemm1_mxfp4(one, one, one, one, None, one, one, one, None, one, None, None, 4, 2, 8, 1024, 512, 1024, 0, 16, 4, 0, 0.0, None)
    assert rc == 1 and b"hidden_pad" in lib.pyhip_moe_last_error()
    rc = lib.pyhip_moe_gemm2_mxfp4(one, one, one, one, None, one, one, one, one, None, one, 4, 2, 8, 1024, 512, 0, -1, 16, 4, None)
    assert rc == 1 and b"inter_pad" in lib.pyhip_moe_last_error()
    # the tile with both operands through LDS only exists with the sort's schedule
    rc = lib.pyhip_moe_gemm1_mxfp4_lds(one, one, one, one, None, one, one, one, None, one, None, None, 4, 2, 8, 1024, 1024, 4, 0, 0.0, None)
    assert rc == 1 and b"schedule missing" in lib.pyhip_moe_last_error()


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libpyhip_moe.so")
    with pytest.raises(_lib.PyhipError, match="no fallback"):
        _lib.load()


def test_code_objects_hold_the_kernels():
    """pyhip_amd/co/*.co (built next to the library) are loadable gfx950 code objects that export the kernels under the
    names pyhip_amd/co_module.py computes"""
    from pyhip_amd import co_module as co
    gemm = [co.gemm_kernel_name(s, mt, 0, nt).encode() for s in (1, 2) for mt in (1, 2, 4, 8, 10, 12, 16, 18) for nt in (False, True)]
    gemm += [co.gemm_kernel_name(1, mt, 1, nt).encode() for mt in (1, 8, 18) for nt in (False, True)]      # clamped SwiGLU
    gemm += [co.gemm_kernel_name(2, mt, 0, nt, True).encode() for mt in (1, 8) for nt in (False, True)]     # atomic epilogue
    gemm += [co.gemm_kernel_name(3, mt, 0, nt).encode() for mt in (1, 8, 18) for nt in (False, True)]       # last-arriver reduction
    gemm += [b"moe_arrive_init_kernel"]
    for name, wanted in (("moe_quant", [b"moe_act_quant_mxfp4_kernel"]),
                         ("moe_reduce", [co.reduce_kernel_name(f, r).encode() for f in (0, 1) for r in (0, 1)]),
                         ("moe_gemm_mxfp4", gemm),
                         # the other sources: every kernel family is there (their template instances are mangled C++
                         # names; the family name is part of each)
                         ("moe_sort", [b"moe_sort_small_kernel", b"moe_sort_hist_kernel", b"moe_sort_scan_kernel",
                                       b"moe_sort_scatter_kernel"]),
                         ("moe_router", [b"moe_router_kernel"]),
                         ("moe_gemm_w4a16", [b"moe_gemm_w4a16_kernel"]),
                         ("moe_gemm_mxfp4_wide", [b"moe_gemm_mxfp4_wide_kernel"])):
        path = os.path.join(co.CO_DIR, name + ".co")
        assert os.path.exists(path), path + " missing: run python -m pyhip_amd.build"
        blob = open(path, "rb").read()
        assert blob[:4] == b"\x7fELF" and b"gfx950" in blob
        for w in wanted:
            assert (w + b"\x00" in blob) if w.startswith(b"_Z") or name == "moe_quant" else (w in blob), w
