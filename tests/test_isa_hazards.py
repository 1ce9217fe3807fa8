"""Static check of the generated gfx950 code of the MFMA kernels (no GPU needed: hipcc cross-compiles).

The kernels issue their direct-to-LDS loads from inline assembly with the base address in scalar registers.  On
gfx9-family hardware a vector memory instruction must not read a scalar register within five wait states of a
vector instruction (v_readfirstlane) writing it; the compiler keeps that distance for its own instructions but does
not look into assembly blocks, and a load that reads a stale base faults the GPU.  The test compiles the file to
assembly and looks at the six instructions in front of every load of an assembly block."""
import os
import re
import shutil
import subprocess
import tempfile

import pytest

from scattermoe_amd import _build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
VMEM = re.compile(r"\b(global_load|buffer_load|global_store|buffer_store)\w*\b")
SBASE = re.compile(r"\bs\[(\d+):(\d+)\]")


def _hazards(text):
    lines = text.split("\n")
    found, loads, inside = [], 0, False
    for i, line in enumerate(lines):
        if "ASMSTART" in line:
            inside = True
            continue
        if "ASMEND" in line:
            inside = False
            continue
        if not (inside and VMEM.search(line)):
            continue
        m = SBASE.search(line)
        if not m:
            continue
        loads += 1
        regs = set(range(int(m.group(1)), int(m.group(2)) + 1))
        k, states = i - 1, 0
        while k >= 0 and states < 6:
            t = lines[k].strip()
            k -= 1
            if not t or t[0] in ";." or t.endswith(":"):
                continue
            nop = re.match(r"s_nop (\d+)", t)
            states += int(nop.group(1)) + 1 if nop else 1
            w = re.match(r"v_readfirstlane_b32 s(\d+)", t)
            if w and int(w.group(1)) in regs and states <= 5:
                found.append((i + 1, t, line.strip()))
                break
    return loads, found


def test_scanner_sees_a_hazard_and_its_fix():
    bad = "\tv_readfirstlane_b32 s2, v20\n\t;;#ASMSTART\n\tglobal_load_dword v1, v2, s[2:3]\n\t;;#ASMEND\n"
    good = "\tv_readfirstlane_b32 s2, v20\n\t;;#ASMSTART\n\ts_nop 4\n\tglobal_load_dword v1, v2, s[2:3]\n\t;;#ASMEND\n"
    assert _hazards(bad)[1] and not _hazards(good)[1]


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="needs hipcc")
def test_no_inline_assembly_load_reads_a_freshly_written_scalar_base():
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "gemm_mfma.s")
        cmd = [_build._hipcc()] + _build.HIPCC_FLAGS + ["-S", "--cuda-device-only", "-o", out,
                                                       os.path.join(_build.CSRC, "gemm_mfma.hip")]
        subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
        loads, found = _hazards(open(out).read())
    assert loads > 100, "no inline-assembly loads found: the scan is looking at the wrong text"
    assert not found, found[:5]
