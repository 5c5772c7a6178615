"""CPU-side tests of the model-file layer (src/Config.cs:21-38,
src/TransformerWeights.cs:20-103): Python reader/writer and the C++ host's
pre-GPU checks, which raise what the reference raises."""
import os
import struct

import numpy as np
import pytest

from managedllama2_amd import hostlib, modelfile, synth

CFG = dict(dim=256, hidden_dim=640, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=300, seq_len=32, rope_theta=10000.0)


@pytest.fixture(scope="module")
def model_path(tmp_path_factory):
    p = str(tmp_path_factory.mktemp("m") / "model.bin")
    modelfile.write_model(p, CFG, synth.random_model(CFG, seed=21, rms_random=True))
    return p


def test_7b_file_size_matches_the_reference():
    assert modelfile.expected_size(synth.LLAMA2_7B) == 3889438752  # size of the converted 7B file
    assert modelfile.HEADER.size == 32


def test_round_trip(model_path):
    cfg, model = modelfile.read_model(model_path)
    assert cfg == CFG
    want = synth.random_model(CFG, seed=21, rms_random=True)
    assert os.path.getsize(model_path) == modelfile.expected_size(CFG)
    assert np.array_equal(model["classifier"], want["classifier"])
    for a, b in zip(model["layers"], want["layers"]):
        for name in modelfile.LAYER_ORDER:
            for x, y in zip(a[name], b[name]):
                assert np.array_equal(x, y)
        assert np.array_equal(a["rms_ffn"], b["rms_ffn"])
    # file order: up before gate (src/TransformerWeights.cs:90-91)
    w_up = want["layers"][0]["up"][0]
    off = 32 + 2 * (2 * CFG["vocab_size"] * CFG["dim"] + CFG["dim"])
    for name in ("q", "k", "v", "o"):
        off += sum(4 * n if i < 2 else 2 * n for i, n in enumerate(modelfile._qweight_shape(CFG, name)))
    raw = np.fromfile(model_path, np.uint32, w_up.size, offset=off)
    assert np.array_equal(raw, w_up)


def test_host_layer_accepts_a_good_file(model_path):
    hostlib.check_model_file(model_path)


def test_bad_rope_theta_is_invalid_model_config(model_path, tmp_path):
    data = bytearray(open(model_path, "rb").read())
    data[28:32] = struct.pack("<f", 500000.0)
    bad = str(tmp_path / "theta.bin")
    open(bad, "wb").write(data)
    with pytest.raises(hostlib.HostError) as e:
        hostlib.check_model_file(bad)
    assert e.value.code == 1 and "Invalid model config" in str(e.value)  # src/Config.cs:27-28
    with pytest.raises(modelfile.ModelFileError):
        modelfile.read_config(bad)


def test_truncated_and_oversized_files_fail_to_read(model_path, tmp_path):
    data = open(model_path, "rb").read()
    for name, blob in (("short.bin", data[:-10]), ("long.bin", data + b"\0" * 6)):
        bad = str(tmp_path / name)
        open(bad, "wb").write(blob)
        with pytest.raises(hostlib.HostError) as e:
            hostlib.check_model_file(bad)
        assert e.value.code == 1 and "Failed to read file" in str(e.value)  # src/TransformerWeights.cs:39-40
        with pytest.raises(modelfile.ModelFileError):
            modelfile.read_model(bad)


def test_gqa_is_not_implemented(model_path, tmp_path):
    data = bytearray(open(model_path, "rb").read())
    data[16:20] = struct.pack("<i", 1)  # numKVHeads
    bad = str(tmp_path / "gqa.bin")
    open(bad, "wb").write(data)
    with pytest.raises(hostlib.HostError) as e:
        hostlib.check_model_file(bad)
    assert e.value.code == 2 and "kvDim" in str(e.value)  # src/Transformer.cs:55-56
