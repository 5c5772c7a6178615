"""Seeded synthetic tensors with the distributions the benchmark configurations
name: int4 weights and zero-points uniform 0..15 packed 8 per uint32 (the
reference's per-row layout, src/TransformerWeights.cs:54-69), fp16 scales
uniform in [0.002, 0.02], fp16 activations N(0,1), fp16 embedding/classifier
N(0, 0.02), RMSNorm weights 1.

Everything is drawn from numpy's PCG64 so a (seed, shape) pair names the same
bits on every machine; nothing big is stored.
"""
import numpy as np

BASE_SEED = 31415  # the reference's tests seed System.Random with it (test/Generator.cs:5)


def qweight_sizes(K):
    """(weights_size, scales_size, zeros_size) per output row,
    src/MatVecResidual.cs:17-19."""
    ss = (K + 127) // 128
    return ((K + 31) // 32) * 4, ss, (ss + 7) // 8


def rng_for(*stream):
    return np.random.Generator(np.random.PCG64([BASE_SEED, *stream]))


def _raw_u32(rng, n):
    """n uniform 32-bit words straight from the bit generator (an order of
    magnitude faster than Generator.integers for gigabytes of nibbles)."""
    return rng.bit_generator.random_raw((n + 1) // 2).view(np.uint32)[:n].copy()


def random_qweight(rng, K, N):
    """One int4 tensor with N output rows of K inputs -> (W, Z, S) flat arrays."""
    ws, ss, zs = qweight_sizes(K)
    W = _raw_u32(rng, N * ws)
    Z = _raw_u32(rng, N * zs)
    S = (0.002 + 0.018 * rng.random(N * ss, dtype=np.float32)).astype(np.float16)
    return W, Z, S


def normal_f16(rng, n, std=1.0):
    return (rng.standard_normal(n, dtype=np.float32) * np.float32(std)).astype(np.float16)


def qweight_bytes(K, N):
    ws, ss, zs = qweight_sizes(K)
    return N * (ws * 4 + zs * 4 + ss * 2)


def random_layer(rng, dim, hidden_dim):
    return {
        "q": random_qweight(rng, dim, dim),
        "k": random_qweight(rng, dim, dim),
        "v": random_qweight(rng, dim, dim),
        "o": random_qweight(rng, dim, dim),
        "gate": random_qweight(rng, dim, hidden_dim),
        "up": random_qweight(rng, dim, hidden_dim),
        "down": random_qweight(rng, hidden_dim, dim),
        "rms_att": np.ones(dim, np.float16),
        "rms_ffn": np.ones(dim, np.float16),
    }


def random_model(cfg, seed=0, rms_random=False):
    """cfg: dict(dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size,
    seq_len, rope_theta).  Returns the tensor set of src/TransformerWeights.cs."""
    rng = rng_for(seed, 1)
    dim, vocab = cfg["dim"], cfg["vocab_size"]
    model = {
        "embedding": normal_f16(rng, vocab * dim, 0.02),
        "classifier": normal_f16(rng, vocab * dim, 0.02),
        "rms_final": np.ones(dim, np.float16),
        "layers": [random_layer(rng, dim, cfg["hidden_dim"]) for _ in range(cfg["n_layers"])],
    }
    if rms_random:  # exercise gamma != 1 in tests
        model["rms_final"] = (1.0 + 0.1 * rng.standard_normal(dim)).astype(np.float16)
        for L in model["layers"]:
            L["rms_att"] = (1.0 + 0.1 * rng.standard_normal(dim)).astype(np.float16)
            L["rms_ffn"] = (1.0 + 0.1 * rng.standard_normal(dim)).astype(np.float16)
    return model


LLAMA2_7B = dict(dim=4096, hidden_dim=11008, n_layers=32, n_heads=32, n_kv_heads=32,
                 vocab_size=32000, seq_len=4096, rope_theta=10000.0)
LLAMA2_13B = dict(dim=5120, hidden_dim=13824, n_layers=40, n_heads=40, n_kv_heads=40,
                  vocab_size=32000, seq_len=4096, rope_theta=10000.0)


def layer_matvec_set_bytes(dim, hidden_dim):
    """Algorithmic bytes of one decoder layer's mat-vec set: weights, zeros,
    scales plus fp16 activations in and out of each of the four launches."""
    qkv = 3 * qweight_bytes(dim, dim) + 2 * dim + 3 * 2 * dim
    o = qweight_bytes(dim, dim) + 2 * dim + 2 * dim + 2 * dim  # x in, residual in, out
    swiglu = 2 * qweight_bytes(dim, hidden_dim) + 2 * dim + 2 * hidden_dim
    down = qweight_bytes(hidden_dim, dim) + 2 * hidden_dim + 2 * dim + 2 * dim
    return {"qkv": qkv, "o": o, "swiglu": swiglu, "down": down,
            "total": qkv + o + swiglu + down}
