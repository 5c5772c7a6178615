"""GPU parity of the persistent decode step (LLAMA2_DECODE_PERSISTENT): the
whole of Transformer.Forward (src/Transformer.cs:158-190) in one launch, the
vectors between the modules handed from workgroup to workgroup as tagged words.

It applies the arithmetic of the launch sequence LLAMA2_DECODE_FUSED operation
for operation, so the two must agree BIT FOR BIT (logits, KV-cache rows, token
ids); against the CPU oracle it is held to the same bounds as the other modes.
"""
import ctypes as C

import numpy as np
import pytest

from managedllama2_amd import capi, synth
from managedllama2_amd.transformer import Transformer
from gpu_util import assert_close_normwise, up, upq, sizes
from test_gpu_transformer import HS128, SMALL, run_and_check

pytestmark = pytest.mark.gpu

FUSED = capi.DECODE_FUSED
PERSIST = capi.DECODE_FUSED | capi.DECODE_PERSISTENT
PERSIST_GRAPH = PERSIST | capi.DECODE_GRAPH


def check_ok(t):
    capi.call("llama2_decode_check", t._decoder)


def bits(a):
    return np.asarray(a).view(np.uint16)


@pytest.mark.parametrize("mode", [PERSIST, PERSIST_GRAPH])
def test_persistent_step_against_oracle(oracle, mode):
    model = synth.random_model(HS128, seed=8, rms_random=True)
    exact, gen, _ = run_and_check(oracle, HS128, model, mode, n_prompt=4, steps=24, seed=404)
    assert exact >= len(gen) - 1


def test_persistent_step_small_heads(oracle):
    """dim 256 = two heads: most workgroups have no row in any phase."""
    model = synth.random_model(SMALL, seed=5, rms_random=True)
    exact, gen, _ = run_and_check(oracle, SMALL, model, PERSIST, n_prompt=5, steps=20, seed=401)
    assert exact >= len(gen) - 1


def test_persistent_equals_fused_bit_for_bit():
    """150 teacher-forced positions (two attention blocks from position 128 on):
    logits after every 10th step and the whole K and V cache."""
    model = synth.random_model(HS128, seed=8, rms_random=True)
    prompt = synth.rng_for(405).integers(3, HS128["vocab_size"], 150).astype(np.int32)
    outs = []
    for mode in (FUSED, PERSIST, PERSIST_GRAPH):
        t = Transformer(dict(HS128), model, mode=mode)
        t.runstate.tokens.copy_to_device(prompt)
        logits = []
        for pos in range(140):
            t.Forward(pos, pos + 1)
            if pos % 10 == 9 or pos >= 126:
                logits.append(t.runstate.logits.to_host())
        check_ok(t)
        outs.append((np.stack(logits), t.runstate.keyCache.to_host(), t.runstate.valueCache.to_host()))
        t.close()
    for other in outs[1:]:
        for a, b, what in zip(outs[0], other, ("logits", "key cache", "value cache")):
            assert np.array_equal(bits(a), bits(b)), "%s differ between the launch sequence and the persistent step" % what


@pytest.mark.parametrize("pos", [127, 128, 511, 512, 1100, 3071, 3072, 3100])
def test_persistent_step_with_long_history(oracle, pos):
    """1, 2, 4, 5, 9 and 24 attention blocks of 128 rows; from 3072 rows on the decoder falls
    back to the launch sequence for the step.  Up to 1024 attended rows the launch sequence uses
    128-row blocks as well and the two agree bit for bit; beyond, the launch sequence merges
    256-row blocks (a different, equally valid grouping of the same sums), and the comparison is
    norm-wise at the per-module tolerance."""
    cfg = dict(HS128, seq_len=max(1200, pos + 40))
    dim, L, S = cfg["dim"], cfg["n_layers"], cfg["seq_len"]
    model = synth.random_model(cfg, seed=11, rms_random=True)
    rng = synth.rng_for(408, pos)
    kc = synth.normal_f16(rng, L * S * dim)
    vc = synth.normal_f16(rng, L * S * dim)
    token = np.array([17], np.int32)
    outs = []
    for mode in (FUSED, PERSIST, PERSIST_GRAPH):
        t = Transformer(dict(cfg), model, mode=mode)
        t.runstate.keyCache.copy_to_device(kc)
        t.runstate.valueCache.copy_to_device(vc)
        t.runstate.tokens.copy_to_device(token, pos)
        t.Forward(pos, pos + 1)
        check_ok(t)
        row = t.runstate.keyCache.to_host(dim, (L - 1) * S * dim + pos * dim)
        vrow = t.runstate.valueCache.to_host(dim, (L - 1) * S * dim + pos * dim)
        outs.append((t.runstate.logits.to_host(), row, vrow))
        t.close()
    same_blocks = pos + 1 <= 1024 or pos + 1 > 3072
    for a, b, what in zip(outs[1], outs[2], ("logits", "k row", "v row")):  # persistent: eager == graph replay
        assert np.array_equal(bits(a), bits(b)), "%s at pos %d" % (what, pos)
    for a, b, what in zip(outs[0], outs[1], ("logits", "k row", "v row")):
        if same_blocks:
            assert np.array_equal(bits(a), bits(b)), "%s at pos %d" % (what, pos)
        else:
            err = np.max(np.abs(a.astype(np.float64) - b.astype(np.float64))) / np.max(np.abs(a.astype(np.float64)))
            assert err <= 2e-3, "%s at pos %d: %.2e" % (what, pos, err)
    if pos in (128, 3071):
        hm = oracle.HostModel(cfg, model)
        hm.key_cache[:], hm.value_cache[:] = kc, vc
        hm.tokens[pos] = token[0]
        want = hm.forward(pos, pos + 1).astype(np.float64)
        assert_close_normwise(outs[1][0], want, "logits at pos %d" % pos, 1e-2)


@pytest.mark.parametrize("mode", [PERSIST, PERSIST_GRAPH])
def test_persistent_device_resident_loop(mode):
    """llama2_decode_run: 260 steps without the host, crossing from one to two
    and three attention blocks; tokens equal the launch sequence's."""
    cfg = dict(HS128, seq_len=300)
    model = synth.random_model(cfg, seed=12)
    prompt = synth.rng_for(406).integers(3, cfg["vocab_size"], 7).astype(np.int32)
    toks = []
    for m in (FUSED | capi.DECODE_GRAPH, mode):
        t = Transformer(dict(cfg), model, mode=m)
        t.runstate.tokens.copy_to_device(prompt)
        capi.call("llama2_decode_run", t._decoder, 0, 260, len(prompt))
        check_ok(t)
        toks.append(t.runstate.tokens.to_host(261))
        t.close()
    assert np.array_equal(toks[0], toks[1])
    assert np.array_equal(toks[0][:7], prompt)


def test_persistent_7b_shaped_layers(oracle):
    """The Llama-2-7B kernel variant (dim 4096, hidden 11008, 32 heads) on two
    layers: bit-identical to the launch sequence, and within the oracle bound."""
    cfg = dict(synth.LLAMA2_7B, n_layers=2, seq_len=160)
    model = synth.random_model(cfg, seed=7)
    prompt = synth.rng_for(407).integers(3, cfg["vocab_size"], 140).astype(np.int32)
    outs = []
    for mode in (FUSED, PERSIST_GRAPH):
        t = Transformer(dict(cfg), model, mode=mode)
        t.runstate.tokens.copy_to_device(prompt)
        logits = []
        for pos in range(135):
            t.Forward(pos, pos + 1)
            if pos in (0, 1, 63, 127, 128, 134):
                logits.append(t.runstate.logits.to_host())
        check_ok(t)
        outs.append((np.stack(logits), t.runstate.keyCache.to_host(135 * 4096, 160 * 4096)))
        t.close()
    assert np.array_equal(bits(outs[0][0]), bits(outs[1][0]))
    assert np.array_equal(bits(outs[0][1]), bits(outs[1][1]))
    exact, gen, _ = run_and_check(oracle, dict(cfg, seq_len=32), model, PERSIST, n_prompt=3, steps=6, seed=403)
    assert exact >= len(gen) - 1


def module_chain(model, cfg, x):
    """The mat-vec set of every layer through the module entry points, the o-projection fed with q."""
    dim, hidden = cfg["dim"], cfg["hidden_dim"]
    zs, ss, ws = sizes(dim)
    hzs, hss, hws = sizes(hidden)
    dx, xb, q, k, v = up(x), up(np.zeros(dim, np.float16)), up(np.zeros(dim, np.float16)), up(np.zeros(dim, np.float16)), up(np.zeros(dim, np.float16))
    h = up(np.zeros(hidden, np.float16))
    for L in model["layers"]:
        g1, g2 = up(L["rms_att"]), up(L["rms_ffn"])
        wq, wk, wv, wo, wg, wu, wd = (upq(L[n]) for n in ("q", "k", "v", "o", "gate", "up", "down"))
        capi.call("llama2_rmsnorm", xb.ptr, dx.ptr, g1.ptr, dim, 1e-5)
        capi.call("llama2_qkv_mat_vec", q.ptr, k.ptr, v.ptr, xb.ptr, wq.Weight.ptr, wq.Zeros.ptr, wq.Scales.ptr,
                  wk.Weight.ptr, wk.Zeros.ptr, wk.Scales.ptr, wv.Weight.ptr, wv.Zeros.ptr, wv.Scales.ptr, dim, dim, zs, ss, ws)
        capi.call("llama2_mat_vec_residual_int4", dx.ptr, q.ptr, wo.Weight.ptr, wo.Zeros.ptr, wo.Scales.ptr, dim, dim, zs, ss, ws)
        capi.call("llama2_rmsnorm", xb.ptr, dx.ptr, g2.ptr, dim, 1e-5)
        capi.call("llama2_mat_vec_swiglu", h.ptr, xb.ptr, wg.Weight.ptr, wg.Zeros.ptr, wg.Scales.ptr, wu.Weight.ptr,
                  wu.Zeros.ptr, wu.Scales.ptr, dim, hidden, zs, ss, ws)
        capi.call("llama2_mat_vec_residual_int4", dx.ptr, h.ptr, wd.Weight.ptr, wd.Zeros.ptr, wd.Scales.ptr, hidden, dim, hzs, hss, hws)
        capi.call("llama2_sync")
    return dx.to_host()


@pytest.mark.parametrize("cfg", [dict(HS128), dict(synth.LLAMA2_7B, n_layers=3, seq_len=16)],
                         ids=["small", "7b-shaped"])
def test_matvec_chain_equals_module_sequence(cfg):
    """llama2_decode_matvec_chain -- the int4 mat-vec family as the persistent
    step runs it -- against the module launches on the same input, bit for bit,
    twice in a row (the hand-over tags move on between launches)."""
    model = synth.random_model(cfg, seed=21, rms_random=True)
    x = synth.normal_f16(synth.rng_for(409), cfg["dim"])
    want = module_chain(model, cfg, x)
    t = Transformer(dict(cfg), model, mode=PERSIST)
    dx, out = up(x), up(np.zeros(cfg["dim"], np.float16))
    for _ in range(2):
        capi.call("llama2_memset", out.ptr, 0, cfg["dim"] * 2)
        capi.call("llama2_decode_matvec_chain", t._decoder, dx.ptr, out.ptr)
        check_ok(t)
        assert np.array_equal(bits(out.to_host()), bits(want))
    t.close()


def test_wait_limit_failure_is_reported_not_hung():
    """A wait limit of zero polls makes every wait inside the step give up at its
    first unsuccessful read (forced from the host: no kernel hangs or faults): the
    step still runs to its end, and llama2_decode_check reports it.  Restoring the
    limit clears the flag and the decoder works again."""
    cfg = dict(HS128, seq_len=64)
    model = synth.random_model(cfg, seed=12)
    t = Transformer(dict(cfg), model, mode=PERSIST)
    t.runstate.tokens.copy_to_device(np.array([5, 6, 7], np.int32))
    t.Forward(0, 1)
    check_ok(t)
    good = t.runstate.logits.to_host()
    capi.call("llama2_decode_set_wait_limit", t._decoder, 0)
    t.Forward(0, 1)
    rc = capi.raw("llama2_decode_check", t._decoder)
    # with no patience at all some wait almost surely fails; if by luck none did, the result is still right
    if rc == capi.OK:
        assert np.array_equal(bits(t.runstate.logits.to_host()), bits(good))
    else:
        assert rc == capi.ERR_STEP_FAILED and "gave up" in capi.last_error()
        # the flag is sticky: the entry points that hand a token to the host report it too
        import ctypes
        token = ctypes.c_int()
        assert capi.raw("llama2_decode_sample", t._decoder, 1, 1, ctypes.byref(token)) == capi.ERR_STEP_FAILED
    capi.call("llama2_decode_set_wait_limit", t._decoder, 1 << 21)
    t.Forward(0, 1)
    check_ok(t)
    assert np.array_equal(bits(t.runstate.logits.to_host()), bits(good))
    t.close()


def test_persistent_rejects_shapes_without_a_kernel():
    cfg = dict(synth.LLAMA2_13B, n_layers=1, seq_len=16, vocab_size=512)
    model = synth.random_model(cfg, seed=3)
    with pytest.raises(capi.Llama2Error) as e:
        Transformer(dict(cfg), model, mode=PERSIST)
    assert e.value.code == capi.ERR_UNSUPPORTED
