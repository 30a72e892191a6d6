"""The machine code of the headline kernel (reduce-copy, fp32 Sum, 2 sources) is pinned: the figures in profiles/ and
the roofline that bench.py reports were measured on exactly this instruction stream, so a change to it has to be
deliberate (and is the moment to take the profile again).  The kernel is compiled to gfx950 assembly with the
library's own flags and its instructions are hashed (labels, comments and directives dropped).

The recorded stream is the one the profiled build had, but for one immediate: the offset of a kernel argument in one
s_load_dword (0x38 there, 0x50 since the argument block carries the scale of the scaled sums)."""
import hashlib
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "dfccl_amd", "csrc")
HIPCC = "/opt/rocm/bin/hipcc"
SYMBOL = "_ZN5dfccl16reduceCopyKernelILi7ELi0ELi2ELb0EEEvNS_6RcArgsE"  # reduceCopyKernel<kF32, kSum, 2, false>
INSTRUCTIONS = 316
SHA256 = "98d0c49c0826beb4dd9139c01f4a11f3b59dff141bd3869b205cde3c2ae40434"

pytestmark = pytest.mark.skipif(not os.path.exists(HIPCC), reason="needs hipcc")


def instruction_stream(asm_path, symbol):
    out, inside = [], False
    for line in open(asm_path):
        if line.startswith(symbol + ":"):
            inside = True
            continue
        if not inside:
            continue
        code = line.split(";")[0].rstrip()
        s = code.strip()
        if not s or s.startswith(".") or s.endswith(":"):
            continue
        out.append(re.sub(r"\.LBB[0-9_]+", "L", re.sub(r"\s+", " ", s)))
        if s.startswith("s_endpgm"):
            break
    return out


def test_headline_kernel_is_the_profiled_one(tmp_path):
    asm = tmp_path / "reduce_copy.s"
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
                           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-S",
                           os.path.join(CSRC, "reduce_copy.hip"), "-o", str(asm)],
                          stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    ins = instruction_stream(str(asm), SYMBOL)
    assert len(ins) == INSTRUCTIONS, len(ins)
    assert hashlib.sha256("\n".join(ins).encode()).hexdigest() == SHA256
    # what the 84 % rest on: one 128-bit non-temporal load per source and one non-temporal store per pack, nothing else
    assert sum(1 for i in ins if i.startswith("global_load_dwordx4") and " nt" in i) >= 2
    assert not any(i.startswith(("scratch_", "buffer_")) for i in ins)
