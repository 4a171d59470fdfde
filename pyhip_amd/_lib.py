"""ctypes binding of ``libpyhip_moe.so`` (the C ABI declared in ``include/pyhip_moe.h``).

There is no CPU fallback: if the library is missing, loading raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpyhip_moe.so")

_c = ctypes
_P, _I, _L, _F = _c.c_void_p, _c.c_int, _c.c_int64, _c.c_float

#: symbol -> (restype, argtypes); the single source the loader and the export test share
SIGNATURES = {
    "pyhip_moe_abi_version": (_I, []),
    "pyhip_moe_last_error": (_c.c_char_p, []),
    "pyhip_moe_topk_softmax": (_I, [_P, _I, _I, _I, _I, _P, _P, _P]),
    "pyhip_moe_topk_grouped_sigmoid": (_I, [_P, _I, _I, _I, _I, _I, _I, _P, _P, _P]),
    "pyhip_moe_sorting_max_blocks": (_L, [_L, _I, _I, _I]),
    "pyhip_moe_sorting_workspace_bytes": (_L, [_L, _I, _I]),
    "pyhip_moe_schedule_words": (_L, [_I]),
    "pyhip_moe_sorting": (_I, [_P, _P, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _L, _P, _L, _P]),
    "pyhip_moe_pick_block_m": (_I, [_L, _I, _I, _I, _I]),
    "pyhip_moe_pick_w4a16": (_I, [_L, _I, _I, _I]),
    "pyhip_moe_zero_fill": (_I, [_P, _L, _P]),
    "pyhip_moe_forward_workspace_bytes": (_L, [_L, _I, _I, _I, _I, _I, _I]),
    "pyhip_moe_forward": (_I, [_P, _L, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I,
                               _I, _F, _P, _L, _P]),
    "pyhip_moe_route_sorting": (_I, [_P, _I, _I, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _L, _P, _L, _L, _I,
                                     _P, _P, _P]),
    "pyhip_moe_forward_routed": (_I, [_P, _L, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I,
                                      _I, _I, _I, _I, _I, _I, _I, _I, _F, _P, _L, _P]),
    "pyhip_moe_forward_static_capacity": (_L, []),
    "pyhip_moe_forward_static": (_I, [_P, _L, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I,
                                      _I, _F, _P]),
    "pyhip_moe_sorting_quant": (_I, [_P, _P, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _L, _P, _L, _L, _I, _P, _P, _P]),
    "pyhip_moe_act_scale_stride": (_L, [_I]),
    "pyhip_moe_act_quant_mxfp4": (_I, [_P, _L, _L, _I, _P, _P, _P, _P]),
    "pyhip_moe_gemm1_mxfp4": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _L, _I, _F, _P]),
    "pyhip_moe_gemm2_mxfp4": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _L, _P]),
    "pyhip_moe_gemm1_mxfp4_lds": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _L, _I, _F, _P]),
    "pyhip_moe_gemm2_mxfp4_lds": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _L, _P]),
    "pyhip_moe_gemm2_mxfp4_atomic": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _L, _P]),
    "pyhip_moe_gemm2_mxfp4_reduce": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I,
                                          _I, _I, _I, _I, _I, _I, _L, _P]),
    "pyhip_moe_gemm1_w4a16": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _L, _I, _I, _F, _P]),
    "pyhip_moe_gemm2_w4a16": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _L, _I, _P]),
    "pyhip_moe_gemm1_w4a16_token": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _P]),
    "pyhip_moe_gemm2_w4a16_token": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "pyhip_moe_probe_mfma_stream": (_I, [_I, _I, _P, _L, _P, _I, _P, _P]),
    "pyhip_moe_topk_reduce": (_I, [_P, _P, _L, _I, _I, _I, _P, _P]),
    "pyhip_moe_topk_reduce_routed": (_I, [_P, _P, _L, _I, _I, _I, _P, _I, _P, _P, _P]),
}

_lib = None


class PyhipError(RuntimeError):
    pass


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise PyhipError(
                "%s is missing: build it with `python -m pyhip_amd.build` (needs hipcc); "
                "there is no fallback path" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def check(rc, what=""):
    if rc != 0:
        msg = load().pyhip_moe_last_error().decode("utf-8", "replace")
        raise PyhipError("%s failed (code %d): %s" % (what or "pyhip_moe call", rc, msg))


def dptr(t):
    """device pointer of a torch tensor (or None)"""
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def current_stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
