"""Pins the oracle's restatement of the converter's repack step
(src/ModelConverter.cs:196-328): AWQ "GEMM" tensors -> the output-major int4
layout the kernels read.

The reference's only check of this code is a SHA-256 of a converted 7B model
that needs the network (test/ConverterTests.cs:18-32, skipped), so the pin is
structural: an integer matrix is packed the way AWQ's packer is published
(qweight[k][c] holds columns 8c + {0,2,4,6,1,3,5,7}[i] in nibble i), repacked by
the oracle, and unpacked by the oracle's golden-pinned dequantiser
(test_oracle_qweight.py); the matrix must come back exactly.  A wrong nibble
order, a missing transpose or a wrong row stride all break that round trip.
"""
import numpy as np
import pytest

from managedllama2_amd import synth

ORDER = [0, 2, 4, 6, 1, 3, 5, 7]


def awq_pack(m):
    """m[rows][cols] of 0..15 -> uint32 [rows][cols/8], AWQ GEMM nibble order."""
    rows, cols = m.shape
    out = np.zeros((rows, cols // 8), np.uint32)
    for i in range(8):
        out |= m[:, ORDER[i]::8].astype(np.uint32) << np.uint32(4 * i)
    return out


@pytest.mark.parametrize("K,N", [(128, 8), (256, 64), (4096, 256), (11008, 64), (5120, 40), (13824, 32)])
def test_awq_tensor_survives_repack_and_unpack(oracle, K, N):
    rng = synth.rng_for(1001, K, N)
    G = K // 128
    m = rng.integers(0, 16, (K, N))
    zm = rng.integers(0, 16, (G, N))
    sm = (0.002 + 0.018 * rng.random((G, N))).astype(np.float16)
    W = oracle.ref_repack_qdata(awq_pack(m), K, N)
    Z = oracle.ref_repack_qdata(awq_pack(zm), G, N)
    S = oracle.ref_repack_scales(sm, G, N)
    ws, ss, zs = oracle.qweight_sizes(K)
    assert W.size == N * ws and Z.size == N * zs and S.size == N * ss
    got = oracle.f64_dequant_rows(W, Z, S, K, N)  # [N][K]
    want = (m - np.repeat(zm, 128, axis=0)).astype(np.float64) * np.repeat(sm, 128, axis=0).astype(np.float64)
    assert np.array_equal(got, want.T)
    assert np.array_equal(S.reshape(N, G), sm.T)


def test_spill_over_nibbles_of_a_ragged_height(oracle):
    """height % 8 != 0 (zero points of K = 11008: 86 groups): the last word of an output row is
    completed with the first rows of the NEXT column, zero behind the last column
    (src/ModelConverter.cs:283-311: `packed` is column-major and 4 words longer than the data)."""
    rng = synth.rng_for(1002)
    H, Wd = 86, 24
    zm = rng.integers(0, 16, (H, Wd))
    out = oracle.ref_repack_qdata(awq_pack(zm), H, Wd).reshape(Wd, 11)
    flat = np.concatenate([zm.T.ravel(), np.zeros(8, np.int64)])  # column-major + the zero tail
    for x in range(Wd):
        for yb in range(11):
            word = int(out[x, yb])
            for i in range(8):
                assert (word >> (4 * i)) & 15 == flat[H * x + 8 * yb + i], (x, yb, i)


def test_scales(oracle):
    rng = synth.rng_for(1003)
    sm = rng.random((86, 40)).astype(np.float16)
    assert np.array_equal(oracle.ref_repack_scales(sm, 86, 40).reshape(40, 86), sm.T)
    # Format.v1 (src/ModelConverter.cs:247-262): rows padded to zeros_size*8 = 88 halfs, compacted to 86
    padded = rng.random((40, 88)).astype(np.float16)
    assert np.array_equal(oracle.ref_compact_scales_v1(padded, 86, 40).reshape(40, 86), padded[:, :86])
