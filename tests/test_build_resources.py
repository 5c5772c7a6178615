"""Register allocation of the built kernels.  A kernel whose private (scratch) memory grows into
kilobytes per lane still computes the right thing, so no parity test notices, but every launch
then pays for a scratch allocation of its own (measured: 1.7 ms instead of 70 us for the
one-launch sampler).  The sampler's phases are non-inlined calls precisely to keep the register
allocator from spilling; this compiles every translation unit of the library and reads the
compiler's own resource report.

The same compile also yields the device assembly, which must hold no packed fp32 arithmetic
(v_pk_add_f32 / v_pk_mul_f32 / v_pk_fma_f32): every translation unit is built with the
packed-fp32-ops target feature switched off."""
import os
import re
import shutil
import subprocess

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "managedllama2_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
LIMIT = 1024  # bytes of scratch per lane


@pytest.mark.skipif(shutil.which(HIPCC) is None, reason="hipcc not found")
@pytest.mark.parametrize("source", sorted(f for f in os.listdir(CSRC) if f.endswith(".hip")))
def test_no_kernel_needs_kilobytes_of_scratch(source, tmp_path):
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-Rpass-analysis=kernel-resource-usage", "--cuda-device-only", "-S", source, "-o",
           str(tmp_path / "out.s")]
    out = subprocess.run(cmd, cwd=CSRC, capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    names = re.findall(r"Function Name: (\S+)", out.stderr)
    scratch = [int(v) for v in re.findall(r"ScratchSize \[bytes/lane\]: (\d+)", out.stderr)]
    assert names and len(names) == len(scratch)
    worst = max(zip(scratch, names))
    assert worst[0] <= LIMIT, "%s uses %d bytes of scratch per lane" % (worst[1], worst[0])
    packed = re.findall(r"^\s*(v_pk_(?:add|mul|fma)_f32)\b", open(tmp_path / "out.s").read(), re.M)
    assert not packed, "%s: %d packed fp32 instructions (%s)" % (source, len(packed), packed[0])
