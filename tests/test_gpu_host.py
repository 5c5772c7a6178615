"""The C++ host layer (libLlama2::Transformer over the C ABI) on the GPU: a
model file written in the reference's format is loaded through the memory
mapped reader and decoded greedily; the tokens must equal what the ctypes host
produces with the same kernels, for every way of issuing the step."""
import numpy as np
import pytest

from managedllama2_amd import capi, hostlib, modelfile, synth
from managedllama2_amd.transformer import Transformer

pytestmark = pytest.mark.gpu

CFG = dict(dim=512, hidden_dim=1408, n_layers=3, n_heads=4, n_kv_heads=4, vocab_size=1000, seq_len=64, rope_theta=10000.0)


@pytest.fixture(scope="module")
def model_file(tmp_path_factory):
    p = str(tmp_path_factory.mktemp("m") / "model.bin")
    model = synth.random_model(CFG, seed=31, rms_random=True)
    modelfile.write_model(p, CFG, model)
    return p, model


@pytest.mark.parametrize("host_mode,py_mode", [(hostlib.HOST_LOOP, None), (hostlib.MODULES, capi.DECODE_MODULES),
                                               (hostlib.FUSED_GRAPH, capi.DECODE_FUSED | capi.DECODE_GRAPH)])
def test_cpp_transformer_generates_the_same_tokens(model_file, host_mode, py_mode):
    path, model = model_file
    prompt = [int(t) for t in synth.rng_for(501).integers(3, CFG["vocab_size"], 6)]
    t = hostlib.Transformer(path, host_mode, stop_on_special=False)
    got = t.Generate(prompt, 30)
    logits = t.logits(CFG["vocab_size"])
    assert t.seq_len == CFG["seq_len"]
    t.close()
    ref = Transformer(dict(CFG), model, mode=py_mode)
    want = list(ref.Generate(prompt, 30, stop_on_special=False))
    assert got == want and len(got) == 30 and got[:5] == prompt[1:]
    assert np.array_equal(logits.view(np.uint16), ref.runstate.logits.to_host().view(np.uint16))
    ref.close()


def test_loading_from_file_equals_loading_from_arrays(model_file):
    path, model = model_file
    cfg, mapped = modelfile.read_model(path)
    a = Transformer(dict(cfg), mapped, mode=capi.DECODE_MODULES)
    b = Transformer(dict(CFG), model, mode=capi.DECODE_MODULES)
    prompt = [5, 9, 11]
    assert list(a.Generate(prompt, 12, stop_on_special=False)) == list(b.Generate(prompt, 12, stop_on_special=False))
    a.close()
    b.close()


def test_stop_on_special_token(model_file):
    # Transformer.Generate stops at a token < 3 (src/Transformer.cs:106): a prompt containing one ends the run there
    path, _ = model_file
    t = hostlib.Transformer(path, hostlib.MODULES, stop_on_special=True)
    assert t.Generate([7, 8, 2, 9, 10], 10) == [8]
    t.close()
