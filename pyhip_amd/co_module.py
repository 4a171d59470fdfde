"""Launching this library's kernels from their code objects (``pyhip_amd/co/*.co``) with nothing but ctypes and the
HIP runtime: ``hipModuleLoad`` -> ``hipModuleGetFunction`` -> ``hipModuleLaunchKernel`` with the arguments packed into
one C struct, the convention of the reference's loader (src/core/hiptools.py:10-100: ``kernel([gx, gy, gz],
[bx, by, bz], *args)``; tensors become ``data_ptr()``, ints C ints, floats C floats).

``libpyhip_moe.so`` is the product path: its host side picks the kernel instance, sizes the grid and checks the
arguments.  This module is for callers that already own a module loader and want the kernels only; the argument
structs they have to fill are mirrored below (``GemmArgs``, ``QuantArgs``, ``ReduceRouting``).
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
CO_DIR = os.path.join(_HERE, "co")

_P, _I, _F, _L = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_longlong


class GemmArgs(ctypes.Structure):
    """argument of moe_gemm_mxfp4_kernel<STAGE, MT, ACT, NT, ATOMIC> (pyhip_amd/csrc/moe_gemm_mxfp4.hip)"""
    _fields_ = [("a_q", _P), ("a_s", _P), ("w", _P), ("w_s", _P), ("bias", _P), ("sorted_ids", _P), ("sorted_w", _P),
                ("sorted_e", _P), ("num_valid", _P), ("sched", _P), ("out", _P), ("out_q", _P), ("out_s", _P),
                ("OSK", _I), ("limit", _F), ("T", _I), ("topk", _I), ("K", _I), ("N", _I), ("SK", _I), ("SC", _I),
                ("n_blk", _I), ("n_tiles", _I), ("a_rows", _I), ("E", _I),
                # STAGE 3 (down GEMM with the last-arriver reduction) only
                ("arrive", _P), ("topk_ids", _P), ("expert_mask", _P), ("final_out", _P), ("final_f32", _I),
                ("experts_all", _I),
                # zero padding at the end of the weight matrices: rows (per half in stage 1) and columns left unfetched
                ("n_pad", _I), ("k_pad", _I)]


class QuantArgs(ctypes.Structure):
    """argument of moe_act_quant_mxfp4_kernel (pyhip_amd/csrc/quant_device.h)"""
    _fields_ = [("x", _P), ("ldx", _L), ("q", _P), ("s", _P), ("rows", _L), ("K", _I), ("SK", _I), ("rows_limit", _P)]


class ReduceRouting(ctypes.Structure):
    """last argument of moe_topk_reduce_kernel<OUT_F32, ROUTED> (pyhip_amd/csrc/moe_reduce.hip)"""
    _fields_ = [("topk_ids", _P), ("expert_mask", _P), ("num_local_tok", _P), ("experts", _I)]


def gemm_kernel_name(stage, mt, act=0, nt=False, atomic=False):
    return "_Z21moe_gemm_mxfp4_kernelILi%dELi%dELi%dELb%dELb%dEEv8GemmArgs" % (stage, mt, act, int(nt), int(atomic))


def reduce_kernel_name(out_f32, routed):
    return "_Z22moe_topk_reduce_kernelILb%dELb%dEEvPK15HIP_vector_typeIjLj4EEPvxiiPKj13ReduceRouting" % (int(out_f32), int(routed))


class HipError(RuntimeError):
    pass


_hip = None


def _runtime():
    global _hip
    if _hip is None:
        _hip = ctypes.CDLL("libamdhip64.so")
        _hip.hipGetErrorString.restype = ctypes.c_char_p
    return _hip


def _check(err, what):
    if err != 0:
        raise HipError("%s: %s" % (what, _runtime().hipGetErrorString(err).decode()))


def _as_c(a):
    """a launch argument as a ctypes value: tensors -> device pointer, int -> C int, float -> C float, None -> NULL"""
    if a is None:
        return _P(None)
    if isinstance(a, (ctypes.Structure, ctypes._SimpleCData)):
        return a
    if hasattr(a, "data_ptr"):
        return _P(a.data_ptr())
    if isinstance(a, bool):
        return _I(int(a))
    if isinstance(a, int):
        return _I(a)
    if isinstance(a, float):
        return _F(a)
    raise TypeError("cannot pass %r to a kernel" % (a,))


class Kernel:
    def __init__(self, module, name):
        self.name = name
        self.func = _P()
        _check(_runtime().hipModuleGetFunction(ctypes.byref(self.func), module.handle, name.encode()),
               "hipModuleGetFunction(%s)" % name)

    def __call__(self, grid, block, *args, shared=0, stream=None):
        """enqueue on ``stream`` (a raw hipStream_t value; default: torch's current stream)"""
        vals = [_as_c(a) for a in args]

        class Packed(ctypes.Structure):
            _fields_ = [("a%d" % i, type(v)) for i, v in enumerate(vals)]
        packed = Packed(*vals)
        size = ctypes.c_size_t(ctypes.sizeof(packed))
        # HIP_LAUNCH_PARAM_BUFFER_POINTER (1), buffer, HIP_LAUNCH_PARAM_BUFFER_SIZE (2), &size, HIP_LAUNCH_PARAM_END (3)
        extra = (_P * 5)(_P(1), ctypes.cast(ctypes.byref(packed), _P), _P(2), ctypes.cast(ctypes.byref(size), _P), _P(3))
        if stream is None:
            import torch
            stream = torch.cuda.current_stream().cuda_stream
        g, b = (list(grid) + [1, 1])[:3], (list(block) + [1, 1])[:3]
        _check(_runtime().hipModuleLaunchKernel(self.func, g[0], g[1], g[2], b[0], b[1], b[2], int(shared), _P(stream),
                                                None, extra), "hipModuleLaunchKernel(%s)" % self.name)


class Module:
    """one code object of ``pyhip_amd/co`` (e.g. ``Module("moe_gemm_mxfp4")``) or any ``.co`` path"""

    def __init__(self, name_or_path):
        path = name_or_path if os.path.sep in name_or_path else os.path.join(CO_DIR, name_or_path + ".co")
        if not os.path.exists(path):
            raise HipError("%s is missing: build it with `python -m pyhip_amd.build`" % path)
        self.handle = _P()
        _check(_runtime().hipModuleLoad(ctypes.byref(self.handle), path.encode()), "hipModuleLoad(%s)" % path)
        self._kernels = {}

    def kernel(self, name):
        if name not in self._kernels:
            self._kernels[name] = Kernel(self, name)
        return self._kernels[name]
