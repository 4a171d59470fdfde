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
KERNEL_RE = r"^(_Z21moe_gemm_mxfp4_kernelILi\dELi\d+ELi\dELb[01]ELb[01]EEv8GemmArgs):[^\n]*\n(.*?)\.end_amdhsa_kernel"


WIDE_SRC = os.path.join(ROOT, "pyhip_amd", "csrc", "moe_gemm_mxfp4_wide.hip")
WIDE_KERNEL_RE = r"^(_Z26moe_gemm_mxfp4_wide_kernelILi\dELi\dEEv8GemmArgs):[^\n]*\n(.*?)\.end_amdhsa_kernel"


def _device_asm(tmp_path_factory, src, kernel_re):
    if shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"):
        pytest.skip("needs hipcc")
    from pyhip_amd import build
    out = tmp_path_factory.mktemp("asm") / (os.path.basename(src) + ".s")
    cmd = [build.HIPCC] + [f for f in build.FLAGS if f not in ("-fPIC",)] + ["--cuda-device-only", "-S", src, "-o", str(out)]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout[-2000:]
    text = out.read_text()
    return text, re.findall(kernel_re, text, re.S | re.M)


@pytest.fixture(scope="module")
def four_wave_asm(tmp_path_factory):
    """the device assembly of the four-wave GEMM source, compiled once with the library's own flags"""
    text, kernels = _device_asm(tmp_path_factory, SRC, KERNEL_RE)
    assert len(kernels) == 58, ("expected (gate_up x two activations + down) x eight tile heights x two load policies, "
                                "plus the down GEMM with the atomic epilogue at two tile heights x two load policies "
                                "and with the last-arriver reduction at three")
    return text, kernels


@pytest.fixture(scope="module")
def gemm_asm(tmp_path_factory, four_wave_asm):
    """... plus the eight-wave kernels (gate_up x two activations + down), which name their accumulators, set M0 and
    issue vector-memory instructions by hand in the same way"""
    text, kernels = four_wave_asm
    wide_text, wide = _device_asm(tmp_path_factory, WIDE_SRC, WIDE_KERNEL_RE)
    assert len(wide) == 3
    return text + wide_text, kernels + wide


def test_compiler_never_touches_accumulation_registers_of_fixed_tiles(gemm_asm):
    text, kernels = gemm_asm
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


def test_compiler_never_uses_m0(gemm_asm):
    """The LDS-DMA helpers set M0 by hand inside inline assembly.  M0 is reserved for the compiler (a clobber on it
    is not honoured), so the helpers are only sound while no instruction of the compiler's own reads or writes M0
    in these kernels."""
    _, kernels = gemm_asm
    for name, body in kernels:
        inside, hand = False, 0
        for line in body.split("\n"):
            if "ASMSTART" in line:
                inside = True
            elif "ASMEND" in line:
                inside = False
            else:
                code = line.split(";")[0]
                if inside:
                    hand += bool(re.search(r"\bm0\b", code))
                else:
                    assert not re.search(r"\bm0\b", code), (name, line)
        assert hand, name


def _instructions(body):
    for line in body.split("\n"):
        code = line.split(";")[0].strip()
        if code and not code.startswith(".") and not code.endswith(":"):
            yield code


def test_no_vector_written_scalar_register_is_read_too_early_by_vector_memory(gemm_asm):
    """gfx9 hazard: a vector-memory instruction may read a scalar register only 5 wait states after a vector
    instruction (v_readlane / v_readfirstlane) wrote it.  The compiler pads its own instructions but not the
    hand-written ones inside inline assembly, so the generated code of every GEMM kernel is scanned."""
    _, kernels = gemm_asm
    for name, body in kernels:
        ins = list(_instructions(body))
        for i, line in enumerate(ins):
            m = re.match(r"v_(?:readlane|readfirstlane)_b32 s(\d+),", line)
            if not m:
                continue
            sreg, waited = int(m.group(1)), 0
            for nxt in ins[i + 1:i + 8]:
                if re.match(r"(buffer_|global_|scratch_|flat_)", nxt):
                    used = set()
                    for a, b in re.findall(r"s\[(\d+):(\d+)\]", nxt):
                        used.update(range(int(a), int(b) + 1))
                    used.update(int(a) for a in re.findall(r"\bs(\d+)\b", nxt))
                    assert sreg not in used or waited >= 5, (name, line, nxt, waited)
                nop = re.match(r"s_nop (\d+)", nxt)
                waited += int(nop.group(1)) + 1 if nop else 1
                if waited >= 5:
                    break


def _vgprs(operand_text):
    regs = set()
    for a, b in re.findall(r"\bv\[(\d+):(\d+)\]", operand_text):
        regs.update(range(int(a), int(b) + 1))
    regs.update(int(a) for a in re.findall(r"\bv(\d+)\b", operand_text))
    return regs


def test_compiler_never_copies_a_register_with_a_load_in_flight(four_wave_asm):
    """The weight tiles and weight scales are loaded by inline assembly long before they are used, and only the
    hand-written waits know when they have arrived.  That holds as long as the compiler leaves those registers
    alone: a copy it inserts (live-range splitting, a join between two instances of a loop body) would read a
    register whose load is still in flight.  Check: outside the inline-assembly regions no instruction of a GEMM
    kernel reads or writes a register that an inline-assembly load writes to.  (The eight-wave kernels load nothing
    but their weight scales into registers and copy those on purpose, after the wait that covers them.)"""
    _, kernels = four_wave_asm
    for name, body in kernels:
        # Walk the kernel text: a register is "loaded" from the inline-assembly load that writes it until the
        # compiler's own code overwrites it with something else.  Values loaded that way are consumed by
        # inline-assembly MFMAs only, so no instruction of the compiler may READ a register in that state.
        inside, loaded, seen = False, set(), set()
        for line in body.split("\n"):
            if "ASMSTART" in line:
                inside = True
            elif "ASMEND" in line:
                inside = False
            else:
                code = line.split(";")[0].strip()
                if not code or code.startswith(".") or code.endswith(":"):
                    continue
                if inside:
                    m = re.match(r"buffer_load_dword(?:x4)? (v\[\d+:\d+\]|v\d+), (?!.*\blds\b)", code)
                    if m:
                        loaded |= _vgprs(m.group(1))
                        seen |= _vgprs(m.group(1))
                    m = re.match(r"v_accvgpr_read_b32 (v\d+),", code)      # epilogue: a new value for that register
                    if m:
                        loaded -= _vgprs(m.group(1))
                    # the reducing down GEMM reads out3 rows with a load that is waited for inside its own statement
                    m = re.match(r"global_load_dwordx4 (v\[\d+:\d+\]),", code)
                    if m:
                        loaded -= _vgprs(m.group(1))
                elif code.startswith(("v_", "ds_", "buffer_", "global_", "scratch_", "flat_")):
                    mnemonic, _, operands = code.partition(" ")
                    ops = operands.split(",")
                    stores = "store" in mnemonic or "write" in mnemonic or mnemonic.startswith("v_cmp")
                    written = set() if stores else _vgprs(ops[0])
                    read = _vgprs(operands if stores else ",".join(ops[1:]))
                    assert not (read & loaded), (name, code, sorted(read & loaded))
                    loaded -= written
        assert len(seen) >= 64 + 8, (name, len(seen))        # 16 weight tiles of 4 registers, 8 scale dwords
