"""GPU parity of the converter's repack kernels (llama2_repack_qdata,
llama2_repack_scales, llama2_compact_scales_v1) against the oracle's
line-for-line restatement of src/ModelConverter.cs:277-328 -- bit-exact, the
spill-over nibbles of ragged heights included -- and the converted model end to
end: an AWQ-format checkpoint of a small model converts to a file whose greedy
decode equals that of the model built directly in the target layout."""
import numpy as np
import pytest

from managedllama2_amd import capi, hostlib, modelconvert, modelfile, synth
from managedllama2_amd.transformer import Transformer
from gpu_util import up

pytestmark = pytest.mark.gpu

ORDER = [0, 2, 4, 6, 1, 3, 5, 7]


def awq_pack(m):
    rows, cols = m.shape
    out = np.zeros((rows, cols // 8), np.uint32)
    for i in range(8):
        out |= m[:, ORDER[i]::8].astype(np.uint32) << np.uint32(4 * i)
    return out


def repack(q_in, height, width):
    d_in = up(np.ascontiguousarray(q_in, np.uint32).ravel())
    d_out = up(np.full(width * ((height + 7) // 8), 0xDEADBEEF, np.uint32))
    capi.call("llama2_repack_qdata", d_out.ptr, d_in.ptr, height, width)
    return d_out.to_host()


@pytest.mark.parametrize("height,width", [
    (4096, 4096), (4096, 11008), (11008, 4096), (5120, 5120), (13824, 5120),  # the 7B / 13B weight tensors
    (32, 4096), (86, 4096), (86, 11008), (40, 5120), (108, 5120),              # their zero-point tensors
    (8, 8), (64, 64), (72, 264), (256, 8), (1, 8), (7, 16), (9, 24), (1000, 40)])
def test_repack_qdata_bit_exact(oracle, height, width):
    rng = synth.rng_for(1101, height, width)
    q_in = rng.integers(0, 2 ** 32, height * width // 8, dtype=np.uint64).astype(np.uint32)
    got = repack(q_in, height, width)
    want = oracle.ref_repack_qdata(q_in, height, width)
    assert np.array_equal(got, want)


def test_repack_then_dequantise_recovers_the_matrix(oracle):
    rng = synth.rng_for(1102)
    K, N = 11008, 256
    G = K // 128
    m, zm = rng.integers(0, 16, (K, N)), rng.integers(0, 16, (G, N))
    sm = (0.002 + 0.018 * rng.random((G, N))).astype(np.float16)
    W, Z, S = modelconvert.RepackQWeight(awq_pack(m), awq_pack(zm), sm, K, N)
    got = oracle.f64_dequant_rows(W, Z, S, K, N)
    want = (m - np.repeat(zm, 128, axis=0)).astype(np.float64) * np.repeat(sm, 128, axis=0).astype(np.float64)
    assert np.array_equal(got, want.T)


@pytest.mark.parametrize("meta_height,width", [(32, 4096), (86, 4096), (32, 11008), (108, 5120), (1, 8), (65, 129)])
def test_scales(oracle, meta_height, width):
    rng = synth.rng_for(1103, meta_height, width)
    s = rng.random(meta_height * width).astype(np.float16)
    d_in, d_out = up(s), up(np.zeros(s.size, np.float16))
    capi.call("llama2_repack_scales", d_out.ptr, d_in.ptr, meta_height, width)
    assert np.array_equal(d_out.to_host().view(np.uint16), oracle.ref_repack_scales(s, meta_height, width).view(np.uint16))
    padded = rng.random(width * ((meta_height + 7) // 8) * 8).astype(np.float16)
    d_in, d_out = up(padded), up(np.zeros(meta_height * width, np.float16))
    capi.call("llama2_compact_scales_v1", d_out.ptr, d_in.ptr, meta_height, width)
    assert np.array_equal(d_out.to_host().view(np.uint16),
                          oracle.ref_compact_scales_v1(padded, meta_height, width).view(np.uint16))


def test_rejects():
    a, b = up(np.zeros(64, np.uint32)), up(np.zeros(64, np.uint32))
    assert capi.raw("llama2_repack_qdata", a.ptr, b.ptr, 8, 12) == capi.ERR_INVALID_ARGUMENT  # width % 8
    assert capi.raw("llama2_repack_qdata", a.ptr, a.ptr, 8, 8) == capi.ERR_INVALID_ARGUMENT   # in place
    assert capi.raw("llama2_repack_qdata", a.ptr, None, 8, 8) == capi.ERR_INVALID_ARGUMENT
    assert capi.raw("llama2_repack_scales", a.ptr, a.ptr, 4, 4) == capi.ERR_INVALID_ARGUMENT
    assert capi.raw("llama2_compact_scales_v1", a.ptr, b.ptr, 0, 4) == capi.ERR_INVALID_ARGUMENT


CFG = dict(dim=512, hidden_dim=1408, n_layers=2, n_heads=4, n_kv_heads=4, vocab_size=1000, seq_len=32, rope_theta=10000.0)


def awq_checkpoint(cfg, rng):
    """A random AWQ (GEMM format) state dictionary and the same model in the target layout."""
    state = {"model.embed_tokens.weight": synth.normal_f16(rng, cfg["vocab_size"] * cfg["dim"], 0.02),
             "lm_head.weight": synth.normal_f16(rng, cfg["vocab_size"] * cfg["dim"], 0.02),
             "model.norm.weight": np.ones(cfg["dim"], np.float16)}
    for i in range(cfg["n_layers"]):
        name = "model.layers.%d" % i
        for tensor, _, K, N in modelconvert._layer_tensors(cfg):
            G = (K + 127) // 128
            state["%s.%s.qweight" % (name, tensor)] = awq_pack(rng.integers(0, 16, (K, N)))
            state["%s.%s.qzeros" % (name, tensor)] = awq_pack(rng.integers(0, 16, (G, N)))
            state["%s.%s.scales" % (name, tensor)] = (0.002 + 0.018 * rng.random((G, N))).astype(np.float16)
        state[name + ".input_layernorm.weight"] = (0.5 + rng.random(cfg["dim"])).astype(np.float16)
        state[name + ".post_attention_layernorm.weight"] = (0.5 + rng.random(cfg["dim"])).astype(np.float16)
    return state


def test_converted_model_decodes_like_the_directly_built_one(oracle, tmp_path):
    rng = synth.rng_for(1104)
    state = awq_checkpoint(CFG, rng)
    path = str(tmp_path / "model.bin")
    modelconvert.Convert(path, CFG, state)
    cfg, model = modelfile.read_model(path)
    assert cfg == CFG
    # the same tensors through the oracle's repack
    for i, L in enumerate(model["layers"]):
        for tensor, key, K, N in modelconvert._layer_tensors(CFG):
            G = (K + 127) // 128
            base = "model.layers.%d.%s" % (i, tensor)
            W, Z, S = L[key]
            assert np.array_equal(W, oracle.ref_repack_qdata(state[base + ".qweight"], K, N))
            assert np.array_equal(Z, oracle.ref_repack_qdata(state[base + ".qzeros"], G, N))
            assert np.array_equal(S.view(np.uint16), oracle.ref_repack_scales(state[base + ".scales"], G, N).view(np.uint16))
    # up and gate are written in that order (src/ModelConverter.cs:165-166) and read back the same way
    prompt = [5, 77, 300]
    t = Transformer(dict(cfg), model, mode=capi.DECODE_FUSED | capi.DECODE_GRAPH)
    toks = list(t.Generate(prompt, 12, stop_on_special=False))
    logits = t.runstate.logits.to_host().astype(np.float64)
    t.close()
    hm = oracle.HostModel(cfg, model)
    hm.tokens[:3] = prompt
    for pos in range(12):
        want = hm.forward(pos, pos + 1).astype(np.float64)
        if pos + 1 >= 3:
            hm.tokens[pos + 1] = toks[pos]
    assert np.max(np.abs(logits - want)) <= 1e-2 * np.max(np.abs(want))


def test_v1_format(oracle):
    rng = synth.rng_for(1105)
    K, N = 11008, 64
    W, Z, S = synth.random_qweight(rng, K, N)
    ws, ss, zs = synth.qweight_sizes(K)
    padded = np.zeros((N, zs * 8), np.float16)
    padded[:, :ss] = S.reshape(N, ss)
    W2, Z2, S2 = modelconvert.RepackQWeight(W, Z, padded, K, N, modelconvert.V1)
    assert np.array_equal(W2, W) and np.array_equal(Z2, Z) and np.array_equal(S2.view(np.uint16), S.view(np.uint16))


def test_cpp_host_repack_equals_python(oracle):
    rng = synth.rng_for(1106)
    K, N = 11008, 128
    G = K // 128
    qw, qz = awq_pack(rng.integers(0, 16, (K, N))), awq_pack(rng.integers(0, 16, (G, N)))
    sc = (0.002 + 0.018 * rng.random((G, N))).astype(np.float16)
    W, Z, S = hostlib.repack_qweight(qw, qz, sc, K, N)
    assert np.array_equal(W, oracle.ref_repack_qdata(qw, K, N))
    assert np.array_equal(Z, oracle.ref_repack_qdata(qz, G, N))
    assert np.array_equal(S.view(np.uint16), oracle.ref_repack_scales(sc, G, N).view(np.uint16))
