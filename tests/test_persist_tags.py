"""Hand-over tags of the persistent decode step (csrc/decode_persist.hip): a word of a hand-over
buffer carries tag16(serial * (L + 2) + l) of the (step, layer) that wrote it, tag16(t) = t % 65535 + 1,
and a consumer takes a word whose tag is the one it expects.  `serial` is advanced by exactly one before
every persistent step and by nothing else, so what a consumer may find in a word besides the expected
value is the word's PREVIOUS write (an earlier layer of the same step, or the last layer of the step
before): the scheme is sound iff those two tags always differ, through every wrap of the 16-bit tag
and of the 32-bit serial product.  (With a serial that other kernels advanced as well, a delta that is a
multiple of 3855 made them equal for 32 layers: 34 * 3855 = 2 * 65535.)"""
import numpy as np
import pytest


def tag16(t):
    return (t % 65535) + 1


@pytest.mark.parametrize("L", [1, 2, 3, 32, 40, 80, 255])
def test_successive_writes_of_a_word_never_share_a_tag(L):
    serial = np.arange(1, 200_000, dtype=np.uint64)
    base = (serial * np.uint64(L + 2)) & np.uint64(0xFFFFFFFF)  # 32-bit product, as on the device
    prev_base = np.concatenate([[np.uint64(0)], base[:-1]])
    for last in (L - 1, L):  # buffers written at layers 0 .. L - 1, and the layer input also at L (classifier)
        # first write of a step against the last write of the step before
        a = tag16((base + np.uint64(0)) & np.uint64(0xFFFFFFFF))
        b = tag16((prev_base + np.uint64(last)) & np.uint64(0xFFFFFFFF))
        assert not np.any(a[1:] == b[1:])
    for l in range(1, L + 1):  # layer l against layer l - 1 of the same step
        a = tag16((base + np.uint64(l)) & np.uint64(0xFFFFFFFF))
        b = tag16((base + np.uint64(l - 1)) & np.uint64(0xFFFFFFFF))
        assert not np.any(a == b)


def test_a_shared_serial_would_collide():
    """The failure this guards against: with 32 layers and a serial delta of 3855 between two persistent
    steps, the first layer's tag equals the tag the same word got 3855 steps earlier."""
    L = 32
    s0, delta = 7, 3855
    assert tag16((s0 + delta) * (L + 2)) == tag16(s0 * (L + 2))
