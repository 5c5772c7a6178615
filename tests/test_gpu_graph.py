"""Stream capture of module calls into a hipGraph (llama2_graph_begin_capture / end_capture /
launch / destroy; no counterpart in the reference, which pays one cuLaunchKernel per module call,
src/Module.cs:21-22).  Every graph is replayed several times with eager work and synchronisation
between the replays, and every replay is compared with the eager result."""
import ctypes as C

import numpy as np
import pytest

from managedllama2_amd import capi, synth
from managedllama2_amd.device import DeviceVariable
from managedllama2_amd.transformer import Transformer

pytestmark = pytest.mark.gpu

CFG = dict(dim=512, hidden_dim=1408, n_layers=2, n_heads=4, n_kv_heads=4, vocab_size=1000, seq_len=600,
           rope_theta=10000.0)
FUSED = capi.DECODE_FUSED
FUSED_GRAPH = capi.DECODE_FUSED | capi.DECODE_GRAPH


def capture(fn):
    g = C.c_void_p()
    capi.call("llama2_graph_begin_capture")
    try:
        fn()
    finally:
        capi.call("llama2_graph_end_capture", C.byref(g))
    return g


def with_history(model, mode, pos, seed):
    """A Transformer whose caches hold `pos` random rows and whose token at `pos` is set."""
    rng = synth.rng_for(seed)
    n = CFG["n_layers"] * CFG["seq_len"] * CFG["dim"]
    t = Transformer(dict(CFG), model, mode=mode)
    t.runstate.keyCache.copy_to_device(synth.normal_f16(rng, n))
    t.runstate.valueCache.copy_to_device(synth.normal_f16(rng, n))
    t.runstate.tokens.copy_to_device(np.array([17], np.int32), pos)
    return t


@pytest.mark.parametrize("pos", [5, 300])
def test_captured_module_sequence(pos):
    """Transformer.Forward issued module by module from the host (10 launches per layer), captured once."""
    model = synth.random_model(CFG, seed=51)
    t = with_history(model, None, pos, 501)
    t.Forward(pos, pos + 1)  # eager: also creates the scratch of llama2_vec_mat for this shape
    want = t.runstate.logits.to_host()
    g = capture(lambda: t.Forward(pos, pos + 1))
    for rep in range(3):
        capi.call("llama2_memset", t.runstate.logits.ptr, 0, t.runstate.logits.size * 2)  # eager work in between
        capi.call("llama2_memset", t.runstate.x.ptr, 0, t.runstate.x.size * 2)
        capi.call("llama2_graph_launch", g)
        got = t.runstate.logits.to_host()  # synchronises
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), rep
    capi.call("llama2_graph_destroy", g)
    t.close()


@pytest.mark.parametrize("mode", [capi.DECODE_MODULES, FUSED, FUSED_GRAPH])
@pytest.mark.parametrize("pos", [5, 300])
def test_captured_decoder_step(mode, pos):
    """llama2_decode_forward inside the caller's capture: the decoder launches its kernels into that graph
    (with the attention grid of the whole context) instead of replaying its own."""
    model = synth.random_model(CFG, seed=52)
    t = with_history(model, mode, pos, 502)
    t.Forward(pos, pos + 1)
    want = t.runstate.logits.to_host()
    g = capture(lambda: t.Forward(pos, pos + 1))
    for rep in range(3):
        capi.call("llama2_memset", t.runstate.logits.ptr, 0, t.runstate.logits.size * 2)
        capi.call("llama2_graph_launch", g)
        got = t.runstate.logits.to_host()
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), rep
        t.Forward(pos, pos + 1)  # the decoder's own path still works between the replays
        assert np.array_equal(t.runstate.logits.to_host().view(np.uint16), want.view(np.uint16))
    capi.call("llama2_graph_destroy", g)
    t.close()


def test_captured_device_loop_continues_where_the_state_is():
    """Greedy steps of the device-resident loop captured by the caller: the position lives on the device, so
    one captured step replays at whatever position the state holds."""
    model = synth.random_model(CFG, seed=53)
    prompt = [int(v) for v in synth.rng_for(503).integers(3, CFG["vocab_size"], 4)]
    ref = Transformer(dict(CFG), model, mode=FUSED_GRAPH)
    want = list(ref.Generate(prompt, 24, stop_on_special=False))
    ref.close()
    t = Transformer(dict(CFG), model, mode=FUSED)
    t.runstate.tokens.copy_to_device(np.array(prompt, np.int32))
    capi.call("llama2_decode_run", t._decoder, 0, 8, len(prompt))  # eager: positions 0..7
    # a captured llama2_decode_run sets the position it was given, then steps: replay = "2 steps from 8"
    g = capture(lambda: capi.call("llama2_decode_run", t._decoder, 8, 2, len(prompt)))
    capi.call("llama2_graph_launch", g)
    assert list(t.runstate.tokens.to_host(11)[1:]) == want[:10]
    capi.call("llama2_decode_run", t._decoder, 10, 14, len(prompt))
    assert list(t.runstate.tokens.to_host(25)[1:]) == want
    capi.call("llama2_graph_destroy", g)
    t.close()


def test_what_is_refused_during_capture():
    x = DeviceVariable.zeros(np.float16, 64)
    host = np.zeros(64, np.float16)
    p = C.c_void_p()
    g = C.c_void_p()
    assert capi.raw("llama2_graph_end_capture", C.byref(g)) == capi.ERR_INVALID_ARGUMENT  # nothing to end
    capi.call("llama2_graph_begin_capture")
    try:
        for name, args in (("llama2_malloc", (C.byref(p), 256)), ("llama2_sync", ()),
                           ("llama2_memcpy_d2h", (host.ctypes.data, x.ptr, 0, 128)),
                           ("llama2_graph_begin_capture", ()), ("llama2_graph_launch", (x.ptr,))):
            assert capi.raw(name, *args) == capi.ERR_INVALID_ARGUMENT, name
            assert "capture" in capi.last_error(), name
        capi.call("llama2_memset", x.ptr, 0x11, 128)  # a fill kernel, not a memset node: recorded, not run
    finally:
        capi.call("llama2_graph_end_capture", C.byref(g))
    capi.call("llama2_sync")  # allowed again
    assert not x.to_host().view(np.uint8).any()
    for rep in range(2):
        capi.call("llama2_graph_launch", g)
        assert np.array_equal(x.to_host().view(np.uint8), np.full(128, 0x11, np.uint8))
        capi.call("llama2_memset", x.ptr, 0, 128)
    capi.call("llama2_graph_destroy", g)


def test_calls_from_another_host_thread():
    """The managed host builds its Transformer inside a worker task (examples/WebAPI/Program.cs:47-49): a
    thread other than the one that called llama2_init must be able to use the library (one thread at a time)."""
    import threading
    model = synth.random_model(dict(CFG, seq_len=64), seed=54)
    prompt = [5, 9, 11]
    want = list(Transformer(dict(CFG, seq_len=64), model, mode=FUSED_GRAPH).Generate(prompt, 12, stop_on_special=False))
    got, errors = [], []

    def worker():
        try:
            t = Transformer(dict(CFG, seq_len=64), model, mode=FUSED_GRAPH)
            got.extend(t.Generate(prompt, 12, stop_on_special=False))
            t.close()
        except Exception as e:  # surfaced in the main thread below
            errors.append(e)

    th = threading.Thread(target=worker)
    th.start()
    th.join(120)
    assert not th.is_alive() and not errors, errors
    assert got == want


def test_sessions_on_concurrent_host_threads():
    """One Transformer per connection on thread-pool threads (examples/WebSocket/Program.cs:85): the entry
    points take turns under the library's lock, so concurrent sessions produce what each produces alone,
    including decoders created (which captures graphs) while another session is decoding."""
    import threading
    cfg = dict(CFG, seq_len=96)
    model = synth.random_model(cfg, seed=55)
    prompts = [[5, 9, 11], [7, 8], [100, 200, 300, 400], [3, 4, 5]]
    want = []
    for p in prompts:
        t = Transformer(dict(cfg), model, mode=FUSED_GRAPH)
        want.append(list(t.Generate(p, 40, stop_on_special=False)))
        t.close()
    got, errors = [None] * len(prompts), []

    def worker(i):
        try:
            for _ in range(3):  # create / decode / destroy repeatedly while the others run
                t = Transformer(dict(cfg), model, mode=FUSED_GRAPH if i % 2 == 0 else FUSED)
                got[i] = list(t.Generate(prompts[i], 40, stop_on_special=False))
                t.close()
        except Exception as e:
            errors.append((i, e))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(prompts))]
    for th in threads:
        th.start()
    for th in threads:
        th.join(180)
    assert not any(th.is_alive() for th in threads) and not errors, errors
    assert got == want
