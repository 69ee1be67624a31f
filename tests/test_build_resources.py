"""Compile-time guard on register spills in the HIP kernels.

Spill code inside a hot loop costs more than the occupancy it buys, so it is
treated as a build error: no kernel may touch scratch memory inside a loop, and
what a kernel spills around its loops (values only needed in a rarely taken
epilogue) must stay below 64 bytes per lane.  hipcc cross-compiles for gfx950
without a GPU."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "bitstack_amd", "csrc")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not available")
@pytest.mark.parametrize("src", ["gemv.hip", "gemv_mx.hip", "gemm.hip", "reconstruct.hip", "strip.hip", "pack.hip", "decode_step.hip"])
def test_no_spill_code_in_loops_and_little_scratch(src, tmp_path):
    asm = tmp_path / "k.s"
    out = subprocess.run([HIPCC] + FLAGS + ["-S", "--cuda-device-only", os.path.join(CSRC, src), "-o", str(asm)],
                         capture_output=True, text=True)
    assert out.returncode == 0, out.stderr[-2000:]
    kernel, in_loop, offenders, scratch = None, False, [], {}
    for line in asm.read_text().splitlines():
        m = re.match(r"^(_Z\w+):", line)
        if m:
            kernel, in_loop = m.group(1), False
        if re.match(r"^\.LBB\d+_\d+:", line) or line.startswith("; %bb."):
            in_loop = "Loop" in line
        if kernel and re.match(r"\s+scratch_(load|store)", line) and in_loop:
            offenders.append((kernel, line.strip()))
        m = re.match(r"\s+\.private_segment_fixed_size:\s+(\d+)", line)
        if m and kernel:
            scratch[kernel] = int(m.group(1))
    assert not offenders, f"spill code inside a loop: {offenders[:4]}"
    sizes = re.findall(r"\.private_segment_fixed_size:\s+(\d+)", asm.read_text())
    assert sizes and max(int(v) for v in sizes) <= 64, f"scratch bytes per lane: {sorted(set(sizes))}"


def test_no_instruction_is_written_as_inline_asm():
    """hipcc's hazard recogniser does not look inside inline asm: a VALU instruction
    written that way next to MFMAs can overwrite registers an in-flight MFMA still
    reads (met with v_and_or_b32: one row tile in four came out wrong once register
    allocation changed).  Only empty asm statements (register pinning) are allowed."""
    offenders = []
    for name in sorted(os.listdir(CSRC)):
        if not name.endswith((".hip", ".h")):
            continue
        text = open(os.path.join(CSRC, name)).read()
        for m in re.finditer(r"\basm\s*(?:volatile)?\s*\(\s*\"([^\"]*)\"", text):
            if m.group(1).strip():
                offenders.append((name, m.group(1)))
    assert not offenders, offenders
