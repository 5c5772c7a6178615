"""The int4 mat-vec launcher picks one of two kernels by row length: one row per item for rows of
up to 6144 inputs, blocks of consecutive rows (shared scale and zero-word loads) for longer rows.
Either kernel handles every shape, and the environment switches LLAMA2_INT4_NARROW /
LLAMA2_INT4_BLOCKS (read once at llama2_init) force one of them for all shapes.  The whole int4
and decode-step parity suite is run once under each switch in a child process, so that the
kernel the launcher does NOT pick for a shape stays held to the same bounds.
"""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("switch", ["LLAMA2_INT4_NARROW", "LLAMA2_INT4_BLOCKS"])
def test_int4_suite_with_one_kernel_for_all_shapes(switch):
    env = dict(os.environ)
    env[switch] = "1"
    files = [os.path.join(ROOT, "tests", f) for f in ("test_gpu_int4.py", "test_gpu_transformer.py")]
    r = subprocess.run([sys.executable, "-u", "-m", "pytest", "-x", "-q", "-m", "gpu", "-p", "no:cacheprovider",
                        "--timeout", "120", "--timeout-method", "thread"] + files,
                       env=env, cwd=ROOT, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, (r.stdout + r.stderr)[-3000:]
    assert " passed" in r.stdout
