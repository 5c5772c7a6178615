"""Shared helpers of the GPU parity tests: every test talks to the kernels
through the C ABI (ctypes), the way the reference's xUnit tests talk to the
raw kernels through ManagedCuda."""
import numpy as np

from managedllama2_amd import capi, synth
from managedllama2_amd.device import DeviceVariable, QWeight, init

TOL = 2e-3       # max relative error against the fp64 oracle, error floor at 2^-8 of the largest |reference|
WORST = {}       # label -> [worst error with the 2^-8 floor, with the 2^-10 floor]; printed at the end of a run


def up(a):
    return DeviceVariable.from_host(a)


def upq(q):
    return QWeight.from_host(*q)


def sizes(K):
    ws, ss, zs = synth.qweight_sizes(K)
    return zs, ss, ws


def rel_err(y, y_ref, floor_bits=8):
    """|y - y*| / max(|y*|, 2^-floor_bits * max|y*|).  Outputs of a zero-mean dot product
    cross zero, where a pure element-wise relative error is unbounded: an output
    that cancels to 1/1000 of its neighbours still carries the fp32 rounding
    noise of all its (up to 13824) terms.  The floor keeps the bound meaningful
    there; away from zero crossings it is the plain relative error."""
    y = np.asarray(y, np.float64)
    y_ref = np.asarray(y_ref, np.float64)
    floor = np.max(np.abs(y_ref)) * 2.0 ** -floor_bits
    return np.abs(y - y_ref) / np.maximum(np.abs(y_ref), max(floor, 1e-30))


def assert_close(y, y_ref, what="", tol=TOL, tol_fine=None):
    """Both floors are asserted with the same bound unless `tol_fine` is given for the 2^-10 floor
    (the largest value measured over the whole suite there is 1.7e-3, on the softmax)."""
    tol_fine = tol if tol_fine is None else tol_fine
    for bits, bound, slot in ((8, tol, 0), (10, tol_fine, 1)):
        e = rel_err(y, y_ref, bits)
        worst = int(np.argmax(e))
        rec = WORST.setdefault(what.split(" ")[0] if what else "?", [0.0, 0.0])
        rec[slot] = max(rec[slot], float(e[worst]))
        assert e[worst] <= bound, "%s: max rel err %.3e (floor 2^-%d, bound %.1e) at %d (got %r want %r)" % (
            what, e[worst], bits, bound, worst, np.asarray(y).ravel()[worst], np.asarray(y_ref).ravel()[worst])


def ulp_diff(a, b):
    """Distance in fp16 representable steps."""
    def key(h):
        u = h.view(np.uint16).astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7FFF), u)
    return np.abs(key(np.asarray(a, np.float16)) - key(np.asarray(b, np.float16)))


def assert_close_normwise(y, y_ref, what="", tol=TOL):
    y = np.asarray(y, np.float64)
    y_ref = np.asarray(y_ref, np.float64)
    e = np.abs(y - y_ref) / np.max(np.abs(y_ref))
    worst = int(np.argmax(e))
    assert e[worst] <= tol, "%s: max norm-wise err %.3e at %d (got %r want %r)" % (
        what, e[worst], worst, y.ravel()[worst], y_ref.ravel()[worst])
