import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.lib()
    return o


def pytest_terminal_summary(terminalreporter):
    """Worst error of every group of fp64 comparisons in this run, under both error floors."""
    try:
        import gpu_util
    except Exception:
        return
    if not gpu_util.WORST:
        return
    terminalreporter.write_line("worst relative error against the fp64 oracle (floor 2^-8 | floor 2^-10):")
    for what, (e8, e10) in sorted(gpu_util.WORST.items()):
        terminalreporter.write_line("  %-28s %.3e | %.3e" % (what, e8, e10))
