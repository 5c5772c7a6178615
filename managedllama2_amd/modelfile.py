"""The reference's model file: a 32-byte Config header (src/Config.cs:6-38)
followed by the tensor stream in the order src/TransformerWeights.cs:33-36 and
:84-94 reads it -- embedding, classifier, final RMSNorm weight, then per layer
q, k, v, o, up, gate, down (each: Weight, Zeros, Scales; :61-66), rmsAttention,
rmsFeedForward.  Tensor sizes per row are those of ReadQWeight (:54-59).
"""
import struct

import numpy as np

from .synth import qweight_sizes

HEADER = struct.Struct("<7if")  # dim, hiddenDim, numLayers, numHeads, numKVHeads, vocabSize, seqLength, ropeTheta
FIELDS = ("dim", "hidden_dim", "n_layers", "n_heads", "n_kv_heads", "vocab_size", "seq_len", "rope_theta")
LAYER_ORDER = ("q", "k", "v", "o", "up", "gate", "down")


class ModelFileError(IOError):
    """FileLoadException in the reference."""


def _qweight_shape(cfg, name):
    dim, hidden = cfg["dim"], cfg["hidden_dim"]
    kv_dim = dim * cfg["n_kv_heads"] // cfg["n_heads"]
    rows, cols = {"q": (dim, dim), "k": (dim, kv_dim), "v": (dim, kv_dim), "o": (dim, dim),
                  "up": (dim, hidden), "gate": (dim, hidden), "down": (hidden, dim)}[name]
    ws, ss, zs = qweight_sizes(rows)
    return ws * cols, zs * cols, ss * cols


def expected_size(cfg):
    n = 2 * (2 * cfg["vocab_size"] * cfg["dim"] + cfg["dim"])
    per_layer = 2 * 2 * cfg["dim"]
    for name in LAYER_ORDER:
        w, z, s = _qweight_shape(cfg, name)
        per_layer += 4 * w + 4 * z + 2 * s
    return HEADER.size + n + cfg["n_layers"] * per_layer


def write_model(path, cfg, model):
    with open(path, "wb") as f:
        f.write(HEADER.pack(*[cfg[k] for k in FIELDS]))  # Config.SaveConfig, src/Config.cs:33-38
        for key in ("embedding", "classifier", "rms_final"):
            f.write(np.ascontiguousarray(model[key], np.float16).tobytes())
        for L in model["layers"]:
            for name in LAYER_ORDER:
                W, Z, S = L[name]
                f.write(np.ascontiguousarray(W, np.uint32).tobytes())
                f.write(np.ascontiguousarray(Z, np.uint32).tobytes())
                f.write(np.ascontiguousarray(S, np.float16).tobytes())
            f.write(np.ascontiguousarray(L["rms_att"], np.float16).tobytes())
            f.write(np.ascontiguousarray(L["rms_ffn"], np.float16).tobytes())


def read_config(path):
    with open(path, "rb") as f:
        raw = f.read(HEADER.size)
    if len(raw) != HEADER.size:
        raise ModelFileError("Invalid model config")
    cfg = dict(zip(FIELDS, HEADER.unpack(raw)))
    if cfg["rope_theta"] != 10000.0:  # src/Config.cs:27-28
        raise ModelFileError("Invalid model config")
    # nothing is derived from a header field before all of them are sane (the same limits as the C++ host layer)
    ok = (0 < cfg["dim"] <= 1 << 20 and 0 < cfg["hidden_dim"] <= 1 << 20 and 0 < cfg["n_layers"] <= 1 << 12
          and 0 < cfg["n_heads"] <= cfg["dim"] and cfg["dim"] % cfg["n_heads"] == 0
          and 0 < cfg["n_kv_heads"] <= cfg["n_heads"] and cfg["n_heads"] % cfg["n_kv_heads"] == 0
          and 0 < cfg["vocab_size"] <= 1 << 24 and 0 < cfg["seq_len"] <= 1 << 24)
    if not ok:
        raise ModelFileError("Invalid model config")
    return cfg


def read_model(path):
    """-> (cfg, model) with the tensors memory-mapped (nothing is copied until
    it is uploaded)."""
    cfg = read_config(path)
    data = np.memmap(path, np.uint8, "r")
    remaining = data.size - HEADER.size
    if expected_size(cfg) != data.size:  # src/TransformerWeights.cs:39-40
        raise ModelFileError("Failed to read file. offset: %d != length: %d" % (expected_size(cfg) - HEADER.size, remaining))
    off = HEADER.size

    def take(dtype, count):
        nonlocal off
        n = count * np.dtype(dtype).itemsize
        a = data[off:off + n].view(dtype)
        off += n
        return a

    model = {"embedding": take(np.float16, cfg["vocab_size"] * cfg["dim"]),
             "classifier": take(np.float16, cfg["vocab_size"] * cfg["dim"]),
             "rms_final": take(np.float16, cfg["dim"]), "layers": []}
    for _ in range(cfg["n_layers"]):
        L = {}
        for name in LAYER_ORDER:
            w, z, s = _qweight_shape(cfg, name)
            L[name] = (take(np.uint32, w), take(np.uint32, z), take(np.float16, s))
        L["rms_att"] = take(np.float16, cfg["dim"])
        L["rms_ffn"] = take(np.float16, cfg["dim"])
        model["layers"].append(L)
    assert off == data.size
    return cfg, model
