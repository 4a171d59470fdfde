"""Compile the HIP sources under ``pyhip_amd/csrc`` into ``pyhip_amd/libpyhip_moe.so`` (gfx950).

hipcc cross-compiles without a GPU.  The library is built in-tree so that it travels with the
source tree; nothing is JIT-compiled at call time.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libpyhip_moe.so")
SOURCES = ["capi.hip", "moe_sort.hip", "moe_quant.hip", "moe_gemm_mxfp4.hip", "moe_gemm_mxfp4_wide.hip", "moe_gemm_w4a16.hip", "moe_reduce.hip", "moe_router.hip", "moe_forward.hip", "moe_forward_static.hip", "probe_mfma_stream.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         # the GEMM keeps its accumulators in hand-numbered accumulation registers: the compiler must not park
         # spilled values there
         "-mllvm", "-amdgpu-spill-vgpr-to-agpr=0"]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


CO_DIR = os.path.join(HERE, "co")
# every source that holds kernels is also shipped as a stand-alone code object (see build_co); the rest of SOURCES
# (capi, moe_forward, moe_forward_static) is host code only; the measurement probe stays in the library
CO_SOURCES = ["moe_quant.hip", "moe_reduce.hip", "moe_gemm_mxfp4.hip", "moe_sort.hip", "moe_router.hip",
              "moe_gemm_w4a16.hip", "moe_gemm_mxfp4_wide.hip"]


def build_co(verbose=False, jobs=4):
    """Device-only code objects ``pyhip_amd/co/*.co`` for gfx950: what ``hipModuleLoad`` takes, for callers that launch
    kernels themselves with ``hipModuleLaunchKernel`` and a packed argument struct (``pyhip_amd/co_module.py``; the
    reference's loader works that way, src/core/hiptools.py:54-100)."""
    os.makedirs(CO_DIR, exist_ok=True)
    flags = [f for f in FLAGS if f != "-fPIC"]

    def one(src):
        out = os.path.join(CO_DIR, src.replace(".hip", ".co"))
        return _run([HIPCC, *flags, "--offload-device-only", "--no-gpu-bundle-output", "-c", os.path.join(CSRC, src), "-o", out])

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        outs = list(ex.map(one, CO_SOURCES))
    if verbose:
        for o in outs:
            if o.strip():
                print(o)
    return CO_DIR


def build(verbose=False, jobs=4):
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in SOURCES]

    def one(pair):
        src, obj = pair
        return _run([HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj])

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        outs = list(ex.map(one, zip(SOURCES, objs)))
    outs.append(_run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]))
    if verbose:
        for o in outs:
            if o.strip():
                print(o)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_co(verbose=True))
