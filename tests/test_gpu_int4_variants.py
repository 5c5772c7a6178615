"""The int4 mat-vec launcher picks among three kernels: the span kernel (consecutive rows per
wavefront, statically scheduled) where the shape suits it, else one row per item for rows of up to
6144 inputs and blocks of consecutive rows (shared scale and zero-word loads) for longer rows.
The latter two handle every shape, and the environment switches LLAMA2_INT4_NO_SPAN (the choice by
row length), LLAMA2_INT4_NARROW / LLAMA2_INT4_BLOCKS (one kernel for all shapes), read once at
llama2_init, take the span kernel out.  The whole int4 and decode-step parity suite is run once
under each switch in a child process, so that the kernels the launcher does NOT pick for a shape
stay held to the same bounds; and since all three kernels add up a row in the same order, their
results are compared bit for bit as well.
"""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("switch", ["LLAMA2_INT4_NO_SPAN", "LLAMA2_INT4_NARROW", "LLAMA2_INT4_BLOCKS"])
def test_int4_suite_with_one_kernel_for_all_shapes(switch):
    env = dict(os.environ)
    env[switch] = "1"
    files = [os.path.join(ROOT, "tests", f) for f in ("test_gpu_int4.py", "test_gpu_transformer.py")]
    r = subprocess.run([sys.executable, "-u", "-m", "pytest", "-x", "-q", "-m", "gpu", "-p", "no:cacheprovider",
                        "--timeout", "120", "--timeout-method", "thread"] + files,
                       env=env, cwd=ROOT, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, (r.stdout + r.stderr)[-3000:]
    assert " passed" in r.stdout


_CHILD = r"""
import sys
import numpy as np
sys.path.insert(0, %(root)r)
sys.path.insert(0, %(tests)r)
from tests_int4_bits import run_all
np.savez(sys.argv[1], **run_all())
"""


def test_span_kernel_equals_the_other_kernels_bit_for_bit(tmp_path):
    """Plain, residual, fused QKV and SwiGLU at ragged and full shapes: the span kernel's fp16 results
    (this process) against the row-length choice of the other two kernels (child process)."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from tests_int4_bits import run_all
    mine = run_all()
    out = str(tmp_path / "other.npz")
    env = dict(os.environ)
    env["LLAMA2_INT4_NO_SPAN"] = "1"
    code = _CHILD % {"root": ROOT, "tests": os.path.join(ROOT, "tests")}
    r = subprocess.run([sys.executable, "-u", "-c", code, out], env=env, cwd=ROOT, capture_output=True, text=True,
                       timeout=600)
    assert r.returncode == 0, (r.stdout + r.stderr)[-3000:]
    import numpy as np
    other = np.load(out)
    assert set(other.files) == set(mine)
    for k in mine:
        assert np.array_equal(mine[k].view(np.uint16), other[k].view(np.uint16)), k
