"""The 64-row prefill loop keeps its accumulators and Q fragments in accumulation registers that it names
by number inside inline assembly (csrc/prefill_acc_regs.h).  Listing them as clobbered makes the kernel
descriptor allocate them, but reserves nothing: a compiler that runs short of vector registers would park
its own values in the same registers between two statements of the loop, and the two would overwrite each
other (wrong outputs, wild addresses).  The kernels are safe exactly as long as the compiler generates no
access to an accumulation register of its own, which this test checks on the device assembly of
csrc/prefill.hip: in every kernel that runs the 64-row loop, every instruction that touches an
accumulation register sits inside an inline-assembly block."""

import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "tt-xla_amd", "csrc")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="needs hipcc to emit the device assembly")
def test_compiler_keeps_out_of_the_fixed_accumulation_registers(tmp_path):
    asm = tmp_path / "prefill.s"
    flags = ["-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
             "-Wno-ignored-attributes", "-S", "--cuda-device-only"]
    done = subprocess.run([HIPCC, *flags, os.path.join(CSRC, "prefill.hip"), "-o", str(asm)],
                          capture_output=True, text=True)
    assert done.returncode == 0, done.stderr[-2000:]
    text = asm.read_text()
    kernels = re.findall(r"^(_ZN4ttpa\S*prefill_kernel\S*):[^\n]*\n(.*?)s_endpgm", text, re.S | re.M)
    assert kernels, "no prefill kernel found in the assembly"
    checked = 0
    for name, body in kernels:
        uses_fixed = False
        own = []
        inside = False
        for line in body.split("\n"):
            s = line.strip()
            if s.startswith(";;#ASMSTART"):
                inside = True
                continue
            if s.startswith(";;#ASMEND"):
                inside = False
                continue
            if not s or s.startswith(";"):
                continue
            touches = re.search(r"\ba\[?\d", s.split(";")[0]) is not None
            if inside and touches:
                uses_fixed = True
            if not inside and touches:
                own.append(s)
        if uses_fixed:
            checked += 1
            assert not own, f"{name}: the compiler uses accumulation registers of its own next to the fixed ones: {own[:5]}"
    assert checked >= 4, f"expected the kernels of the 64-row form, found {checked}"
