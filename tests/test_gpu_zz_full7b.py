"""configs[4]: full Llama-2-7B-shape greedy decode with random-init weights --
32 layers, dim 4096, 32 heads, FFN 11008, int4 g128 linear layers, fp16
embedding / classifier over a 32000 vocabulary, 128 seeded prompt tokens
followed by 256 argmax tokens, every step on the device (hipGraph replay).

The CPU oracle cannot replay 383 steps of a 7B model in test time, so it is
teacher-forced at eleven positions (first, second, mid-prompt, last prompt
token, first generated tokens, mid-generation, last) with the GPU's own history
(tokens AND KV-cache rows of the earlier positions): one step of the fp64
oracle is then compared with the GPU's logits for that step, and the GPU's
token must be the bit-exact argmax of its logits and the oracle's argmax or a
near-tie of it.  The number of positions where the two argmaxes coincide is
printed and asserted (measured: 11 of 11; at least 10 required).

Tolerance: both sides round every module output to fp16; a rounding that
falls the other way is amplified by each of the 32 random-weight layers.
Measured norm-wise logit error (max |difference| / max |logit|) at the eleven
positions: 4.3e-3, 6.0e-3, 2.4e-2, 3.3e-2, 2.5e-2, 1.4e-2, 1.2e-2, 3.2e-2,
1.6e-2, 2.1e-2, 1.3e-2 -- it grows with the length of the attended history
and scatters by a factor of two from position to position.  The bound is the
largest measured value plus half: 5e-2.  The strict per-module bounds (2e-3)
are enforced at these same tensor shapes in test_gpu_int4.py, test_gpu_f16.py,
test_gpu_pointwise.py and, two layers deep, in test_gpu_transformer.py.
"""
import numpy as np
import pytest

from managedllama2_amd import capi, synth
from managedllama2_amd.transformer import Transformer
from gpu_util import assert_close_normwise

pytestmark = pytest.mark.gpu

N_PROMPT, N_GEN = 128, 256
DEEP_TOL = 5e-2
MIN_EXACT = 10


def test_full_7b_greedy_decode(oracle):
    cfg = dict(synth.LLAMA2_7B, seq_len=512)
    model = synth.random_model(cfg, seed=41)
    prompt = synth.rng_for(5).integers(3, cfg["vocab_size"], N_PROMPT).astype(np.int32)
    steps = N_PROMPT + N_GEN - 1

    t = Transformer(dict(cfg), model, mode=capi.DECODE_FUSED | capi.DECODE_GRAPH)
    t.runstate.tokens.copy_to_device(prompt)
    capi.call("llama2_decode_run", t._decoder, 0, steps, N_PROMPT)
    tokens = t.runstate.tokens.to_host(N_PROMPT + N_GEN)
    assert np.array_equal(tokens[:N_PROMPT], prompt)
    assert np.all((tokens >= 0) & (tokens < cfg["vocab_size"]))
    assert len(set(tokens[N_PROMPT:].tolist())) > 4  # not stuck on one id

    # the same run again reproduces every token (deterministic kernels, graph replay)
    t.runstate.tokens.copy_to_device(np.concatenate([prompt, np.zeros(N_GEN, np.int32)]))
    capi.call("llama2_decode_run", t._decoder, 0, steps, N_PROMPT)
    assert np.array_equal(t.runstate.tokens.to_host(N_PROMPT + N_GEN), tokens)

    # teacher-forced oracle steps
    oracle.set_threads(16)
    hm = oracle.HostModel(cfg, model)
    hm.tokens[:tokens.size] = tokens
    dim, S, L = cfg["dim"], cfg["seq_len"], cfg["n_layers"]
    kc = t.runstate.keyCache.to_host().reshape(L, S, dim)
    vc = t.runstate.valueCache.to_host().reshape(L, S, dim)
    exact, errs = 0, []
    checked = (0, 1, 64, N_PROMPT - 1, N_PROMPT, N_PROMPT + 1, 200, 255, 256, 320, steps - 1)
    for pos in checked:
        hm.key_cache.reshape(L, S, dim)[:, :pos] = kc[:, :pos]
        hm.value_cache.reshape(L, S, dim)[:, :pos] = vc[:, :pos]
        want = hm.forward(pos, pos + 1).astype(np.float64)
        t.Forward(pos, pos + 1)  # rewrites row `pos` of the caches with the same values
        got = t.runstate.logits.to_host()
        errs.append(float(np.max(np.abs(got.astype(np.float64) - want)) / np.max(np.abs(want))))
        assert_close_normwise(got, want, "7B logits at pos %d" % pos, DEEP_TOL)
        tok = int(np.argmax(got))
        if pos + 1 >= N_PROMPT:
            assert tok == tokens[pos + 1]  # what the device loop sampled at this step
        best = int(np.argmax(want))
        exact += tok == best
        assert want[tok] >= want[best] - DEEP_TOL * np.max(np.abs(want)), (pos, tok, best)
        # the step's new cache rows agree with the oracle's as well
        row = t.runstate.keyCache.to_host(dim, (L - 1) * S * dim + pos * dim).astype(np.float64)
        assert_close_normwise(row, hm.key_cache.reshape(L, S, dim)[L - 1, pos].astype(np.float64), "k row", DEEP_TOL)
    print("7B teacher-forced steps at positions %s: norm-wise logit error %s; GPU argmax == oracle argmax at %d of %d" %
          (list(checked), ["%.2e" % e for e in errs], exact, len(checked)))
    assert exact >= MIN_EXACT, (exact, len(checked))
    t.close()
