"""Compile-time guard: no HIP kernel of the library may spill registers.

A spilling instantiation of the GEMV kernel once returned wrong rows on the
GPU, so a spill is treated as a build error here (hipcc cross-compiles for
gfx950 without a GPU)."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "bitstack_amd", "csrc")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not available")
@pytest.mark.parametrize("src", ["gemv.hip", "gemm.hip", "reconstruct.hip", "pack.hip"])
def test_no_kernel_spills_or_uses_scratch(src, tmp_path):
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature",
           "-Xclang", "-packed-fp32-ops", "-Rpass-analysis=kernel-resource-usage", "-c",
           os.path.join(CSRC, src), "-o", str(tmp_path / "x.o")]
    out = subprocess.run(cmd, capture_output=True, text=True)
    assert out.returncode == 0, out.stderr[-2000:]
    names = re.findall(r"Function Name: (\S+)", out.stderr)
    vspill = [int(v) for v in re.findall(r"VGPRs Spill: (\d+)", out.stderr)]
    sspill = [int(v) for v in re.findall(r"SGPRs Spill: (\d+)", out.stderr)]
    scratch = [int(v) for v in re.findall(r"ScratchSize \[bytes/lane\]: (\d+)", out.stderr)]
    assert names and len(names) == len(vspill) == len(scratch)
    bad = [(n, v, s, sc) for n, v, s, sc in zip(names, vspill, sspill, scratch) if v or sc]
    assert not bad, f"kernels that spill: {bad}"
