"""ctypes binding of libllama2_hip.so -- the same C ABI a C# host binds with
P/Invoke (include/llama2_hip.h).  There is no CPU fallback: if the library
has not been built, or a call fails, this raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libllama2_hip.so")

OK = 0
ERR_INVALID_ARGUMENT = -1
ERR_NOT_INITIALIZED = -2
ERR_UNSUPPORTED = -3
ERR_NO_DEVICE = -4
ERR_STEP_FAILED = -5
MAX_SOFTMAX_SIZE = 8192
MAX_SAMPLER_SIZE = 65536

DECODE_MODULES = 0
DECODE_FUSED = 1
DECODE_GRAPH = 2
DECODE_PERSISTENT = 4

vp = C.c_void_p
i = C.c_int
f = C.c_float
sz = C.c_size_t


class Llama2Error(RuntimeError):
    """Raised on any non-zero status; mirrors ManagedCuda's CudaException
    (thrown synchronously on launch/alloc failure)."""

    def __init__(self, code, message):
        super().__init__("llama2_hip error %d: %s" % (code, message))
        self.code = code


class Config(C.Structure):
    """src/Config.cs:6-19"""
    _fields_ = [("dim", i), ("hidden_dim", i), ("n_layers", i), ("n_heads", i), ("n_kv_heads", i),
                ("vocab_size", i), ("seq_len", i), ("rope_theta", f)]


class QWeight(C.Structure):
    """src/QWeight.cs:5-10"""
    _fields_ = [("weight", vp), ("zeros", vp), ("scales", vp)]


class LayerWeights(C.Structure):
    """src/PerLayerWeight.cs:5-16"""
    _fields_ = [("query", QWeight), ("key", QWeight), ("value", QWeight), ("output", QWeight),
                ("gate", QWeight), ("up", QWeight), ("down", QWeight),
                ("rms_attention", vp), ("rms_feed_forward", vp)]


class TransformerWeights(C.Structure):
    """src/TransformerWeights.cs:8-14"""
    _fields_ = [("token_embedding_table", vp), ("classifier_weights", vp), ("rms_final_weight", vp),
                ("layers", C.POINTER(LayerWeights))]


class RunState(C.Structure):
    """src/RunState.cs:7-25"""
    _fields_ = [("x", vp), ("xb", vp), ("h", vp), ("q", vp), ("attention", vp), ("logits", vp),
                ("key_cache", vp), ("value_cache", vp), ("tokens", vp), ("indices", vp)]


_SIGNATURES = {
    "llama2_init": [i],
    "llama2_shutdown": [],
    "llama2_malloc": [C.POINTER(vp), sz],
    "llama2_free": [vp],
    "llama2_memcpy_h2d": [vp, sz, vp, sz],
    "llama2_memcpy_d2h": [vp, vp, sz, sz],
    "llama2_memcpy_d2d": [vp, vp, sz],
    "llama2_memset": [vp, i, sz],
    "llama2_mem_info": [C.POINTER(sz), C.POINTER(sz)],
    "llama2_sync": [],
    "llama2_graph_begin_capture": [],
    "llama2_graph_end_capture": [C.POINTER(vp)],
    "llama2_graph_launch": [vp],
    "llama2_graph_destroy": [vp],
    "llama2_event_create": [C.POINTER(vp)],
    "llama2_event_record": [vp],
    "llama2_event_elapsed_ms": [vp, vp, C.POINTER(f)],
    "llama2_event_destroy": [vp],
    "llama2_mat_vec_residual_int4": [vp, vp, vp, vp, vp, i, i, i, i, i],
    "llama2_mat_vec_int4": [vp, vp, vp, vp, vp, i, i, i, i, i],
    "llama2_qkv_mat_vec": [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i, i, i, i, i],
    "llama2_mat_vec_swiglu": [vp, vp, vp, vp, vp, vp, vp, vp, i, i, i, i, i],
    "llama2_mat_vec": [vp, vp, vp, i, i],
    "llama2_mat_vec_strided": [vp, vp, vp, i, i, i, i, i, i, f, i],
    "llama2_vec_mat": [vp, vp, vp, i, i, i, i, i, i],
    "llama2_vec_mat_static": [vp, vp, vp, i, i, i, i, i, i],
    "llama2_multi_head_attention": [vp, vp, vp, vp, i, i, i, f, i],
    "llama2_rope_multi_head_attention": [vp, vp, vp, vp, i, i, i, f, i, i, f],
    "llama2_rmsnorm": [vp, vp, vp, i, f],
    "llama2_rope": [vp, vp, i, i, i, f, i],
    "llama2_softmax": [vp, i, i],
    "llama2_argmax": [vp, i, vp, i, i],
    "llama2_embedding": [vp, vp, i, vp, i],
    "llama2_softmax_logits": [vp, i, f, vp],
    "llama2_sort": [vp, vp, i],
    "llama2_cumulative_sum": [vp, i],
    "llama2_sample_top_p": [vp, vp, i, f, vp, i],
    "llama2_sample": [vp, vp, i, f, f, f, vp, i],
    "llama2_repack_qdata": [vp, vp, i, i],
    "llama2_repack_scales": [vp, vp, i, i],
    "llama2_compact_scales_v1": [vp, vp, i, i],
    "llama2_decode_create": [C.POINTER(vp), C.POINTER(Config), C.POINTER(TransformerWeights),
                             C.POINTER(RunState), i],
    "llama2_decode_forward": [vp, i, i],
    "llama2_decode_sample": [vp, i, i, C.POINTER(i)],
    "llama2_decode_sample_top_p": [vp, i, i, f, f, f, C.POINTER(i)],
    "llama2_decode_run": [vp, i, i, i],
    "llama2_decode_run_sampled": [vp, i, i, i, f, f, C.c_ulonglong],
    "llama2_decode_check": [vp],
    "llama2_decode_set_wait_limit": [vp, i],
    "llama2_decode_matvec_chain": [vp, vp, vp],
    "llama2_decode_destroy": [vp],
}
# exported, not status-returning
_OTHER = {"llama2_last_error": (C.c_char_p, []), "llama2_stream": (vp, []),
          "llama2_sampler_coin": (f, [C.c_ulonglong, i])}

EXPORTS = sorted(list(_SIGNATURES) + list(_OTHER))

_lib = None


def load():
    """dlopen the library and type every entry point.  Does not touch the GPU."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise Llama2Error(ERR_NO_DEVICE, "%s is not built (run `python -c 'import __graft_entry__ as g; "
                              "g.build()'` or `make -C managedllama2_amd/csrc`)" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = i
        for name, (restype, argtypes) in _OTHER.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = restype
        _lib = lib
    return _lib


def last_error():
    return load().llama2_last_error().decode("utf-8", "replace")


def check(status):
    if status != OK:
        raise Llama2Error(status, last_error())


def call(name, *args):
    """Invoke an entry point and raise Llama2Error on a non-zero status."""
    check(getattr(load(), name)(*args))


def raw(name, *args):
    """Invoke an entry point and return its status (for error-path tests)."""
    return getattr(load(), name)(*args)
