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
near-tie of it (within twice the measured logit error).  The number of
positions where the two argmaxes coincide is printed and asserted (measured:
10 of 11; at least 10 required; the odd one is position 382, where the two
candidates are 2.2e-3 of the largest logit apart in the oracle's own logits).

Tolerance.  Both sides round every module output to fp16, and a rounding that
falls the other way on one side travels through all later layers.  How far it
travels is a property of the (random-weight) network at that position, and the
test MEASURES it: the oracle's own step is repeated with its input, the
embedding row, moved to a neighbouring fp16 value in every element -- the size
of one rounding of one module output -- and the norm-wise change of its logits
(max |change| / max |logit|) is the bound for the GPU's logits at that position
(floor 1e-2 where the network is well conditioned).  Measured, position by
position (GPU error | oracle's own change):

    0: 3.9e-3 | 6.4e-3    1: 3.9e-3 | 9.2e-3    64: 4.9e-2 | 1.4e-1   127: 2.2e-2 | 1.3e-1
  128: 1.3e-2 | 7.4e-2  129: 1.3e-2 | 1.9e-2   200: 1.1e-2 | 7.2e-2   255: 1.9e-2 | 5.0e-2
  256: 7.0e-3 | 1.5e-2  320: 7.9e-3 | 8.8e-2   382: 1.9e-2 | 5.2e-2

The GPU's deviation is 0.09 ... 0.69 of what a single one-step move of the input
does to the oracle itself, at every position.

test_logit_error_against_depth measures where that comes from, on these same
weights cut to their first 1, 2, 4, 8, 16 and 32 layers (norm-wise logit error,
one teacher-forced step):

    layers          1        2        4        8        16       32
    position 127    7.0e-4   2.9e-3   3.6e-3   8.1e-3   1.4e-2   2.2e-2
    position 382    4.9e-3   1.6e-3   4.1e-3   8.2e-3   2.3e-2   1.9e-2

About 7e-4 per layer, growing linearly with the depth (independent rounding
differences adding up), not exponentially; it scatters by a factor of two to
three from position to position.  The depth test asserts the one-layer error
(<= 8e-3) and the growth per doubling (<= 4x); 5e-2 bounds its 32-layer figures.
The strict per-module bounds (2e-3) are enforced at these same tensor shapes in
test_gpu_int4.py, test_gpu_f16.py, test_gpu_pointwise.py and, two layers deep,
in test_gpu_transformer.py.
"""
import numpy as np
import pytest

from managedllama2_amd import capi, synth
from managedllama2_amd.transformer import Transformer
from gpu_util import assert_close_normwise

pytestmark = pytest.mark.gpu

N_PROMPT, N_GEN = 128, 256
DEEP_TOL = 5e-2            # 32 layers, positions 127 and 382 of the depth test
WELL_CONDITIONED = 1e-2    # floor of the per-position bound: the end-to-end bound of the small models in test_gpu_transformer.py
MIN_EXACT = 10
DEPTH1_TOL = 8e-3      # one layer deep: embedding .. classifier is a chain of 9 modules held to 2e-3 each
DOUBLING_FACTOR = 4.0  # largest growth of the error from one depth to twice that depth (measured: at most 2.8)


@pytest.fixture(scope="module")
def model7b():
    return synth.random_model(dict(synth.LLAMA2_7B, seq_len=512), seed=41)


def one_step_sensitivity(hm, model, token, pos):
    """How far the fp64 oracle's own logits move (norm-wise) when every element of the step's input, the
    embedding row of `token`, moves to a neighbouring fp16 value (seeded directions): the size of ONE
    rounding of one module output, sent through all the layers.  The caches of the earlier positions stay."""
    row = model["embedding"].reshape(-1, hm.cfg.dim)[token]
    saved = row.copy()
    base = hm.forward(pos, pos + 1).astype(np.float64)
    up = synth.rng_for(1000 + pos).integers(0, 2, row.size).astype(bool)
    row[:] = np.where(up, np.nextafter(saved, np.float16(np.inf)), np.nextafter(saved, np.float16(-np.inf)))
    moved = hm.forward(pos, pos + 1).astype(np.float64)
    row[:] = saved
    return float(np.max(np.abs(moved - base)) / np.max(np.abs(base))), int(np.argmax(moved)) != int(np.argmax(base))


def test_full_7b_greedy_decode(oracle, model7b):
    cfg = dict(synth.LLAMA2_7B, seq_len=512)
    model = model7b
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
    exact, errs, conds, oracle_flips, misses = 0, [], [], 0, []
    checked = (0, 1, 64, N_PROMPT - 1, N_PROMPT, N_PROMPT + 1, 200, 255, 256, 320, steps - 1)
    for pos in checked:
        hm.key_cache.reshape(L, S, dim)[:, :pos] = kc[:, :pos]
        hm.value_cache.reshape(L, S, dim)[:, :pos] = vc[:, :pos]
        cond, flipped = one_step_sensitivity(hm, model, int(tokens[pos]), pos)
        conds.append(cond)
        oracle_flips += flipped
        want = hm.forward(pos, pos + 1).astype(np.float64)
        t.Forward(pos, pos + 1)  # rewrites row `pos` of the caches with the same values
        got = t.runstate.logits.to_host()
        errs.append(float(np.max(np.abs(got.astype(np.float64) - want)) / np.max(np.abs(want))))
        # the bound of this position: what the oracle itself does when its input moves by one fp16 step
        bound = max(cond, WELL_CONDITIONED)
        assert_close_normwise(got, want, "7B logits at pos %d" % pos, bound)
        tok = int(np.argmax(got))
        if pos + 1 >= N_PROMPT:
            assert tok == tokens[pos + 1]  # what the device loop sampled at this step
        best = int(np.argmax(want))
        exact += tok == best
        if tok != best:
            misses.append((pos, float((want[best] - want[tok]) / np.max(np.abs(want)))))
        assert want[tok] >= want[best] - 2.0 * errs[-1] * np.max(np.abs(want)), (pos, tok, best)
        # the step's new cache rows agree with the oracle's as well
        row = t.runstate.keyCache.to_host(dim, (L - 1) * S * dim + pos * dim).astype(np.float64)
        assert_close_normwise(row, hm.key_cache.reshape(L, S, dim)[L - 1, pos].astype(np.float64), "k row", bound)
    print("7B teacher-forced steps at positions %s: norm-wise logit error %s; GPU argmax == oracle argmax at %d of %d" %
          (list(checked), ["%.2e" % e for e in errs], exact, len(checked)))
    print("  the oracle's own logit change when the step's input row moves by one fp16 step per element: %s; "
          "its argmax changes at %d of %d positions" % (["%.2e" % c for c in conds], oracle_flips, len(checked)))
    print("  positions where the two argmaxes differ, with the distance of the two candidates in the oracle's "
          "logits (of the largest logit): %s" % [(p, "%.1e" % g) for p, g in misses])
    assert exact >= MIN_EXACT, (exact, len(checked))
    t.close()


DEPTHS = (1, 2, 4, 8, 16, 32)
DEPTH_POSITIONS = (127, 382)


def test_logit_error_against_depth(oracle, model7b):
    """Where the end-to-end error comes from: the same 7B-shaped weights cut to their first 1, 2, 4, 8, 16
    and 32 layers (embedding, final norm and classifier kept), the fused step against one teacher-forced
    fp64 step at positions 127 and 382.  One layer deep the logits are within a small multiple of the
    per-module bound; the error then grows about linearly with the depth (fp16 roundings between
    modules that fall differently on the two sides add up), never by more than DOUBLING_FACTOR from
    one depth to twice that depth; the 32-layer figure is what test_full_7b_greedy_decode's bound covers."""
    prompt = synth.rng_for(5).integers(3, synth.LLAMA2_7B["vocab_size"], N_PROMPT).astype(np.int32)
    oracle.set_threads(16)
    table = {}
    for depth in DEPTHS:
        cfg = dict(synth.LLAMA2_7B, seq_len=512, n_layers=depth)
        model = dict(model7b, layers=model7b["layers"][:depth])
        t = Transformer(dict(cfg), model, mode=capi.DECODE_FUSED | capi.DECODE_GRAPH)
        t.runstate.tokens.copy_to_device(prompt)
        capi.call("llama2_decode_run", t._decoder, 0, max(DEPTH_POSITIONS) + 1, N_PROMPT)
        tokens = t.runstate.tokens.to_host(max(DEPTH_POSITIONS) + 2)
        hm = oracle.HostModel(cfg, model)
        hm.tokens[:tokens.size] = tokens
        dim, S, L = cfg["dim"], cfg["seq_len"], depth
        kc = t.runstate.keyCache.to_host().reshape(L, S, dim)
        vc = t.runstate.valueCache.to_host().reshape(L, S, dim)
        for pos in DEPTH_POSITIONS:
            hm.key_cache.reshape(L, S, dim)[:, :pos] = kc[:, :pos]
            hm.value_cache.reshape(L, S, dim)[:, :pos] = vc[:, :pos]
            want = hm.forward(pos, pos + 1).astype(np.float64)
            t.Forward(pos, pos + 1)
            got = t.runstate.logits.to_host().astype(np.float64)
            table[(depth, pos)] = float(np.max(np.abs(got - want)) / np.max(np.abs(want)))
        t.close()
    print("norm-wise logit error of the fused step against the fp64 step, by depth:")
    for pos in DEPTH_POSITIONS:
        print("  position %3d: " % pos + "  ".join("L=%d %.2e" % (d, table[(d, pos)]) for d in DEPTHS))
    for pos in DEPTH_POSITIONS:
        assert table[(1, pos)] <= DEPTH1_TOL, (pos, table[(1, pos)])
        for a, b in zip(DEPTHS, DEPTHS[1:]):
            # amplification per doubling, with the one-layer bound as a floor for the ratio's denominator
            assert table[(b, pos)] <= DOUBLING_FACTOR * max(table[(a, pos)], DEPTH1_TOL / 4), (pos, a, b, table)
        assert table[(32, pos)] <= DEEP_TOL
