"""Build-time property of the MXFP4 GEMM kernels: their accumulators live in accumulation registers that are named
by hand inside inline assembly, invisible to the compiler.  That is only sound while the compiler itself never
allocates an accumulation register in those kernels (it would do so to park ordinary registers under pressure).
The check compiles the kernel source to assembly (no GPU needed) and looks at every instruction outside the
inline-assembly regions."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "pyhip_amd", "csrc", "moe_gemm_mxfp4.hip")


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="needs hipcc")
def test_compiler_never_touches_accumulation_registers_of_fixed_tiles(tmp_path):
    from pyhip_amd import build
    out = tmp_path / "gemm.s"
    cmd = [build.HIPCC] + [f for f in build.FLAGS if f not in ("-fPIC",)] + ["--cuda-device-only", "-S", SRC, "-o", str(out)]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout[-2000:]
    text = out.read_text()
    kernels = re.findall(r"^(_Z21moe_gemm_mxfp4_kernelILi\dELi\d+EEv8GemmArgs):[^\n]*\n(.*?)\.end_amdhsa_kernel", text, re.S | re.M)
    assert len(kernels) == 10, "expected two stages x five tile heights"
    for name, body in kernels:
        inside = False
        hand = {"mfma": 0, "read": 0, "write": 0}
        for line in body.split("\n"):
            if "ASMSTART" in line:
                inside = True
            elif "ASMEND" in line:
                inside = False
            elif inside:
                for key, pat in (("mfma", "v_mfma_scale"), ("read", "v_accvgpr_read"), ("write", "v_accvgpr_write")):
                    hand[key] += pat in line
            else:
                code = line.split(";")[0]
                assert "v_accvgpr" not in code and not re.search(r"\ba\[?\d", code), (name, line)
        assert hand["mfma"] and hand["read"] and hand["write"], (name, hand)
        m = re.search(r"ScratchSize: (\d+)", text[text.index(name):])
        assert m and int(m.group(1)) == 0, (name, "spills")
