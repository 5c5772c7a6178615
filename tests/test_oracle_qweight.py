"""Pins the oracle's int4 pack/unpack against the reference's own golden
vector (test/QWeightTestData.cs, test/QWeightTests.cs:29-48) and its
round-trip cases (test/QWeightTests.cs:9-27)."""
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "qweight_golden.json")


@pytest.fixture(scope="module")
def golden():
    d = json.load(open(GOLDEN))
    d["scales"] = np.array(d["scales_f32_bits"], np.uint32).view(np.float32)
    d["checks"] = np.array(d["checks_f32_bits"], np.uint32).view(np.float32)
    d["W"] = np.array(d["weights"], np.uint32)
    return d


def test_golden_zero_word(golden):
    # test/QWeightTests.cs:34-38
    combined = 0
    for z, v in enumerate(golden["zeros"]):
        combined |= (v & 0xF) << (4 * z)
    assert combined == golden["zero_word"]


def test_golden_scales_are_fp16(golden):
    s = golden["scales"]
    assert np.array_equal(s.astype(np.float16).astype(np.float32), s)


def test_unpack_reproduces_golden(oracle, golden):
    # test/QWeightTests.cs:40-47: Unpack() must equal checks.ToHalf() exactly
    Z = np.array([golden["zero_word"]], np.uint32)
    S = golden["scales"].astype(np.float16)
    got = oracle.ref_qweight_unpack(golden["W"], Z, S)
    want = golden["checks"].astype(np.float16)
    assert got.size == 1024
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_row_layout_agrees_with_golden(oracle, golden):
    # one row of K=1024: the per-row layout and the flat one coincide
    Z = np.array([golden["zero_word"]], np.uint32)
    S = golden["scales"].astype(np.float16)
    rows = oracle.ref_qweight_unpack_rows(golden["W"], Z, S, 1024, 1)
    want = golden["checks"].astype(np.float16)
    assert np.array_equal(rows.ravel().view(np.uint16), want.view(np.uint16))
    d = oracle.f64_dequant_rows(golden["W"], Z, S, 1024, 1).ravel()
    # the fp64 closed form, rounded once, gives the same fp16 values
    assert np.array_equal(d.astype(np.float16).view(np.uint16), want.view(np.uint16))
    # and is exactly (w - z) * s with the golden's nibbles
    k = np.arange(1024)
    w = (golden["W"][k // 8] >> (4 * (k % 8)).astype(np.uint32)) & 0xF
    z = np.array(golden["zeros"])[k // 128]
    assert np.array_equal(d, (w.astype(np.int64) - z) * golden["scales"].astype(np.float64)[k // 128])


ROUND_TRIP = [  # test/QWeightTests.cs:9-18: (min, max-exclusive, multiplier, scale, zero)
    (0, 15, 1.0, 1.0, 0), (-1, 14, 1.0, 1.0, 1), (-14, 1, 1.0, 1.0, 14), (-7, 8, 1.0, 1.0, 7),
    (0, 15, 10.0, 10.0, 0), (0, 15, 0.1, 0.1, 0),
]


@pytest.mark.parametrize("lo,hi,mul,scale,zero", ROUND_TRIP)
def test_pack_unpack_round_trip(oracle, lo, hi, mul, scale, zero):
    rng = np.random.default_rng(31415)
    ints = rng.integers(lo, hi, 1024)
    if mul == 0.1:
        vals = (ints // 10).astype(np.float16)  # C#: integer x / 10
        # with scale 0.1 the values are 0 or 1; quantised 0 or 10
    else:
        vals = (ints * mul).astype(np.float16)
    W, Z, S = oracle.ref_qweight_pack(vals, np.full(8, scale, np.float32), np.full(8, zero, np.uint32))
    back = oracle.ref_qweight_unpack(W, Z, S)
    if mul == 0.1:
        # (Half)0.1 is not 0.1: 10 * half(0.1) rounds to 1 in fp16, exactly as in C#
        assert np.array_equal(back, vals)
    else:
        assert np.array_equal(back, vals)


def test_pack_layout_is_lsb_first(oracle):
    vals = np.zeros(1024, np.float16)
    vals[:8] = [1, 2, 3, 4, 5, 6, 7, 8]
    W, Z, S = oracle.ref_qweight_pack(vals, np.ones(8, np.float32), np.zeros(8, np.uint32))
    assert W[0] == 0x87654321
    assert not W[1:].any() and Z[0] == 0


def test_half_conversions_match_numpy(oracle):
    lib = oracle.lib()
    rng = np.random.default_rng(1)
    f = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 100,
                        rng.standard_normal(20000).astype(np.float32) * 1e-6,
                        np.array([0, -0.0, 65504, 65519.99, 65520, 1e9, 2.0 ** -25, 2.0 ** -24,
                                  5.96e-8, 6.1e-5, 1 + 2.0 ** -11, 1 + 3 * 2.0 ** -11], np.float32)])
    with np.errstate(over="ignore"):  # 65520 and 1e9 round to infinity on purpose
        want = f.astype(np.float16).view(np.uint16)
    got = np.array([lib.oracle_f2h(float(v)) for v in f], np.uint16)
    assert np.array_equal(got, want)
    d = f.astype(np.float64) * (1 + 1e-12)
    with np.errstate(over="ignore"):
        wantd = d.astype(np.float16).view(np.uint16)
    gotd = np.array([lib.oracle_d2h(float(v)) for v in d], np.uint16)
    assert np.array_equal(gotd, wantd)
    allh = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    finite = allh[(allh & 0x7C00) != 0x7C00]
    back = np.array([lib.oracle_h2f(int(v)) for v in finite[::7]], np.float32)
    assert np.array_equal(back, finite[::7].view(np.float16).astype(np.float32))
