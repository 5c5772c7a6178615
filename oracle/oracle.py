"""ctypes front-end of the CPU oracle (oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
CPU-baseline leg of the benchmark.  The shipped library never touches it.

All arrays are numpy: fp16 tensors as ``np.float16`` (passed as raw uint16
bits), packed int4 words as ``np.uint32``.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# LLAMA2_ORACLE_LIB names another build of oracle.c (the sanitizer build of tests/test_oracle_sanitize.py)
_LIB_PATH = os.environ.get("LLAMA2_ORACLE_LIB") or os.path.join(_HERE, "liboracle.so")


def build(force=False):
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", os.path.basename(_LIB_PATH)])
    return _LIB_PATH


_lib = None

u16p = C.POINTER(C.c_uint16)
u32p = C.POINTER(C.c_uint32)
f32p = C.POINTER(C.c_float)
f64p = C.POINTER(C.c_double)
i32p = C.POINTER(C.c_int)


class Config(C.Structure):
    """src/Config.cs:6-19 -- 7 x int32 + 1 x float32 = 32 bytes."""
    _fields_ = [("dim", C.c_int), ("hidden_dim", C.c_int), ("n_layers", C.c_int),
                ("n_heads", C.c_int), ("n_kv_heads", C.c_int), ("vocab_size", C.c_int),
                ("seq_len", C.c_int), ("rope_theta", C.c_float)]


class QWeightPtr(C.Structure):
    _fields_ = [("W", u32p), ("Z", u32p), ("S", u16p)]


class LayerPtr(C.Structure):
    _fields_ = [("q", QWeightPtr), ("k", QWeightPtr), ("v", QWeightPtr), ("o", QWeightPtr),
                ("gate", QWeightPtr), ("up", QWeightPtr), ("down", QWeightPtr),
                ("rms_att", u16p), ("rms_ffn", u16p)]


class WeightsPtr(C.Structure):
    _fields_ = [("embedding", u16p), ("classifier", u16p), ("rms_final", u16p),
                ("layers", C.POINTER(LayerPtr))]


class RunStatePtr(C.Structure):
    _fields_ = [("x", u16p), ("xb", u16p), ("h", u16p), ("q", u16p), ("att", u16p),
                ("logits", u16p), ("key_cache", u16p), ("value_cache", u16p), ("tokens", i32p)]


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.oracle_h2f.restype = C.c_float
        _lib.oracle_h2f.argtypes = [C.c_uint16]
        _lib.oracle_f2h.restype = C.c_uint16
        _lib.oracle_f2h.argtypes = [C.c_float]
        _lib.oracle_d2h.restype = C.c_uint16
        _lib.oracle_d2h.argtypes = [C.c_double]
        _lib.ref_argmax.restype = C.c_int
        _lib.ref_sample_top_p.restype = C.c_int
        _lib.ref_sample.restype = C.c_int
        _lib.oracle_coin.restype = C.c_float
        _lib.oracle_coin.argtypes = [C.c_uint64, C.c_int]
    return _lib


def _h(a):  # fp16 array -> uint16 pointer
    assert a.dtype == np.float16 and a.flags.c_contiguous
    return a.ctypes.data_as(u16p)


def _u(a):
    assert a.dtype == np.uint32 and a.flags.c_contiguous
    return a.ctypes.data_as(u32p)


def _d(a):
    assert a.dtype == np.float64 and a.flags.c_contiguous
    return a.ctypes.data_as(f64p)


def set_threads(n):
    lib().oracle_set_threads(C.c_int(n))


def qweight_sizes(K):
    """(weights_size, scales_size, zeros_size) per output row."""
    ss = (K + 127) // 128
    return ((K + 31) // 32) * 4, ss, (ss + 7) // 8


# ---- HostQWeight (flat layout) ------------------------------------------------
def ref_qweight_unpack(W, Z, S):
    out = np.empty(W.size * 8, np.float16)
    lib().ref_qweight_unpack(_u(W), _u(Z), _h(S), C.c_int(W.size), _h(out))
    return out


def ref_qweight_pack(data, scales, zeros):
    """data fp16[n], scales float32[n/128], zeros uint32[n/128] -> (W, Z, S)."""
    n = data.size
    n_words = n // 8
    W = np.zeros(n_words, np.uint32)
    Z = np.zeros(max(n_words // 128, 1), np.uint32)
    S = np.zeros(n_words // 16, np.float16)
    scales = np.ascontiguousarray(scales, np.float32)
    zeros = np.ascontiguousarray(zeros, np.uint32)
    lib().ref_qweight_pack(_h(np.ascontiguousarray(data)), C.c_int(n), scales.ctypes.data_as(f32p),
                           _u(zeros), C.c_int(zeros.size), _u(W), _u(Z), _h(S))
    return W, Z, S


# ---- row-padded layout ----------------------------------------------------------
def ref_qweight_unpack_rows(W, Z, S, K, N):
    out = np.empty((N, K), np.float16)
    lib().ref_qweight_unpack_rows(_u(W), _u(Z), _h(S), C.c_int(K), C.c_int(N), _h(out))
    return out


def f64_dequant_rows(W, Z, S, K, N):
    out = np.empty((N, K), np.float64)
    lib().f64_dequant_rows(_u(W), _u(Z), _h(S), C.c_int(K), C.c_int(N), _d(out))
    return out


# ---- reference C# CPU path ------------------------------------------------------
def ref_matvec(w, x, n, d):
    out = np.empty(d, np.float16)
    lib().ref_matvec(_h(w), _h(x), C.c_int(n), C.c_int(d), _h(out))
    return out


def ref_matvec_int4(x, W, Z, S, K, N):
    out = np.empty(N, np.float16)
    lib().ref_matvec_int4(_h(out), _h(x), _u(W), _u(Z), _h(S), C.c_int(K), C.c_int(N))
    return out


def ref_matvec_residual_int4(res, x, W, Z, S, K, N):
    out = np.array(res, np.float16, copy=True)
    lib().ref_matvec_residual_int4(_h(out), _h(x), _u(W), _u(Z), _h(S), C.c_int(K), C.c_int(N))
    return out


def ref_matvec_swiglu(x, g, u, K, N):
    out = np.empty(N, np.float16)
    lib().ref_matvec_swiglu(_h(out), _h(x), _u(g[0]), _u(g[1]), _h(g[2]), _u(u[0]), _u(u[1]),
                            _h(u[2]), C.c_int(K), C.c_int(N))
    return out


def ref_matvec_strided(q, k, dim, n_heads, n_kv_heads, seq_len):
    att = np.zeros(n_heads * seq_len, np.float16)
    lib().ref_matvec_strided(_h(att), _h(q), _h(k), C.c_int(dim), C.c_int(n_heads),
                             C.c_int(n_kv_heads), C.c_int(seq_len))
    return att


def ref_vecmat(att, v, dim, n_heads, n_kv_heads, seq_len):
    out = np.zeros(dim, np.float16)
    lib().ref_vecmat(_h(out), _h(att), _h(v), C.c_int(dim), C.c_int(n_heads), C.c_int(n_kv_heads),
                     C.c_int(seq_len))
    return out


def ref_softmax(x):
    out = np.array(x, np.float16, copy=True)
    lib().ref_softmax(_h(out), C.c_int(out.size))
    return out


def ref_rmsnorm(x, gamma, eps=1e-5, square_in_half=True):
    out = np.empty(x.size, np.float16)
    lib().ref_rmsnorm(_h(out), _h(x), _h(gamma), C.c_int(x.size), C.c_float(eps),
                      C.c_int(1 if square_in_half else 0))
    return out


def ref_rope(q, k_row, dim, n_heads, n_kv_heads, pos, theta=10000.0):
    q = np.array(q, np.float16, copy=True)
    k = np.array(k_row, np.float16, copy=True)
    lib().ref_rope(_h(q), _h(k), C.c_int(dim), C.c_int(n_heads), C.c_int(n_kv_heads), C.c_int(pos),
                   C.c_float(theta))
    return q, k


def ref_argmax(logits):
    return int(lib().ref_argmax(_h(logits), C.c_int(logits.size)))


def ref_embedding(table, dim, tokens, pos):
    x = np.empty(dim, np.float16)
    tokens = np.ascontiguousarray(tokens, np.int32)
    lib().ref_embedding(_h(x), _h(table), C.c_int(dim), tokens.ctypes.data_as(i32p), C.c_int(pos))
    return x


# ---- stochastic sampler (src/Sampler.cs:48-67) ------------------------------------------
def _i(a):
    assert a.dtype == np.int32 and a.flags.c_contiguous
    return a.ctypes.data_as(i32p)


def ref_softmax_logits(logits, temperature):
    """-> (probabilities fp16, indices int32)"""
    out = np.array(logits, np.float16, copy=True)
    indices = np.empty(out.size, np.int32)
    lib().ref_softmax_logits(_h(out), C.c_int(out.size), C.c_float(temperature), _i(indices))
    return out, indices


def ref_sort(keys, values):
    k = np.array(keys, np.float16, copy=True)
    v = np.array(values, np.int32, copy=True)
    lib().ref_sort(_h(k), _i(v), C.c_int(k.size))
    return k, v


def ref_cumulative_sum(values):
    out = np.array(values, np.float16, copy=True)
    lib().ref_cumulative_sum(_h(out), C.c_int(out.size))
    return out


def ref_sample_top_p(cdf, indices, threshold):
    cdf = np.ascontiguousarray(cdf, np.float16)
    indices = np.ascontiguousarray(indices, np.int32)
    return int(lib().ref_sample_top_p(_h(cdf), _i(indices), C.c_int(cdf.size), C.c_float(threshold)))


def ref_sample(logits, temperature, top_p, coin, generate_token=True):
    """Sampler.Sample on a copy of the logits -> token (-1 when nothing is generated)."""
    work = np.array(logits, np.float16, copy=True)
    indices = np.zeros(work.size, np.int32)
    return int(lib().ref_sample(_h(work), _i(indices), C.c_int(work.size), C.c_float(temperature),
                                C.c_float(top_p), C.c_float(coin), C.c_int(1 if generate_token else 0)))


def coin(seed, pos):
    return float(lib().oracle_coin(C.c_uint64(seed), C.c_int(pos)))


def f64_softmax_logits(logits, temperature):
    out = np.empty(logits.size, np.float64)
    lib().f64_softmax_logits(_d(out), _h(logits), C.c_int(logits.size), C.c_float(temperature))
    return out


def f64_cumulative_sum(values):
    out = np.empty(values.size, np.float64)
    lib().f64_cumulative_sum(_d(out), _h(values), C.c_int(values.size))
    return out


# ---- converter repack (src/ModelConverter.cs:196-328) -----------------------------------
def ref_repack_qdata(q_in, height, width):
    """[height][width/8] AWQ GEMM words -> [width][ceil(height/8)] words."""
    q_in = np.ascontiguousarray(q_in, np.uint32).ravel()
    assert q_in.size == height * width // 8 and width % 8 == 0
    out = np.zeros(width * ((height + 7) // 8), np.uint32)
    lib().ref_repack_qdata(_u(q_in), C.c_int(height), C.c_int(width), _u(out))
    return out


def ref_repack_scales(scales_in, meta_height, width):
    scales_in = np.ascontiguousarray(scales_in, np.float16).ravel()
    out = np.empty(meta_height * width, np.float16)
    lib().ref_repack_scales(_h(scales_in), C.c_int(meta_height), C.c_int(width), _h(out))
    return out


def ref_compact_scales_v1(scales, scales_size, width):
    scales = np.ascontiguousarray(scales, np.float16).ravel()
    out = np.empty(scales_size * width, np.float16)
    lib().ref_compact_scales_v1(_h(scales), C.c_int(scales_size), C.c_int(width), _h(out))
    return out


# ---- fp64 closed forms ------------------------------------------------------------
def f64_matvec_int4(x, W, Z, S, K, N):
    y = np.empty(N, np.float64)
    lib().f64_matvec_int4(_d(y), _h(x), _u(W), _u(Z), _h(S), C.c_int(K), C.c_int(N))
    return y


def f64_matvec_f16(x, M, K, N):
    y = np.empty(N, np.float64)
    lib().f64_matvec_f16(_d(y), _h(x), _h(M), C.c_int(K), C.c_int(N))
    return y


def f64_matvec_strided(q, Km, rows, cols, v_stride, m_col_stride, m_row_stride, o_stride, alpha,
                       n_heads):
    att = np.zeros(n_heads * o_stride, np.float64)
    lib().f64_matvec_strided(_d(att), _h(q), _h(Km), C.c_int(rows), C.c_int(cols),
                             C.c_int(v_stride), C.c_int(m_col_stride), C.c_int(m_row_stride),
                             C.c_int(o_stride), C.c_double(alpha), C.c_int(n_heads))
    return att


def f64_vecmat(att, V, rows, cols, m_col_stride, o_stride, m_row_stride, n_heads):
    out = np.zeros(n_heads * o_stride, np.float64)
    lib().f64_vecmat(_d(out), _h(att), _h(V), C.c_int(rows), C.c_int(cols), C.c_int(m_col_stride),
                     C.c_int(o_stride), C.c_int(m_row_stride), C.c_int(n_heads))
    return out


def f64_softmax(x, size, n_rows):
    out = np.empty(size * n_rows, np.float64)
    lib().f64_softmax(_d(out), _h(x), C.c_int(size), C.c_int(n_rows))
    return out


def f64_rmsnorm(x, gamma, eps=1e-5):
    out = np.empty(x.size, np.float64)
    lib().f64_rmsnorm(_d(out), _h(x), _h(gamma), C.c_int(x.size), C.c_double(eps))
    return out


def f64_rope(q, k_row, n_heads, n_kv_heads, head_size, pos, theta=10000.0):
    qo = np.zeros(q.size, np.float64)
    ko = np.zeros(k_row.size, np.float64)
    lib().f64_rope(_d(qo), _d(ko), _h(q), _h(k_row), C.c_int(n_heads), C.c_int(n_kv_heads),
                   C.c_int(head_size), C.c_int(pos), C.c_double(theta))
    return qo, ko


def round_d2h(a):
    a = np.ascontiguousarray(a, np.float64)
    out = np.empty(a.shape, np.float16)
    lib().oracle_round_d2h(_d(a), _h(out), C.c_size_t(a.size))
    return out


# ---- whole decode step --------------------------------------------------------------
class HostModel:
    """Host-side (numpy) weights + run state laid out as the reference's
    TransformerWeights / RunState, with the pointer structs oracle.c wants."""

    def __init__(self, cfg, weights):
        """cfg: dict with the Config fields; weights: dict as produced by
        managedllama2_amd.synth.random_model()."""
        self.cfg = Config(cfg["dim"], cfg["hidden_dim"], cfg["n_layers"], cfg["n_heads"],
                          cfg["n_kv_heads"], cfg["vocab_size"], cfg["seq_len"], cfg["rope_theta"])
        self.w = weights
        self._layers = (LayerPtr * cfg["n_layers"])()
        for i, L in enumerate(weights["layers"]):
            for name in ("q", "k", "v", "o", "gate", "up", "down"):
                W, Z, S = L[name]
                setattr(self._layers[i], name, QWeightPtr(_u(W), _u(Z), _h(S)))
            self._layers[i].rms_att = _h(L["rms_att"])
            self._layers[i].rms_ffn = _h(L["rms_ffn"])
        self._wp = WeightsPtr(_h(weights["embedding"]), _h(weights["classifier"]),
                              _h(weights["rms_final"]), self._layers)
        dim, kv = cfg["dim"], cfg["dim"] * cfg["n_kv_heads"] // cfg["n_heads"]
        z = lambda n: np.zeros(n, np.float16)
        self.x, self.xb, self.q = z(dim), z(dim), z(dim)
        self.h = z(cfg["hidden_dim"])
        self.att = z(cfg["n_heads"] * max(dim, cfg["seq_len"]))
        self.logits = z(cfg["vocab_size"])
        self.key_cache = z(cfg["n_layers"] * cfg["seq_len"] * kv)
        self.value_cache = z(cfg["n_layers"] * cfg["seq_len"] * kv)
        self.tokens = np.zeros(cfg["seq_len"] + 1, np.int32)
        self._rs = RunStatePtr(_h(self.x), _h(self.xb), _h(self.h), _h(self.q), _h(self.att),
                               _h(self.logits), _h(self.key_cache), _h(self.value_cache),
                               self.tokens.ctypes.data_as(i32p))

    def forward(self, position, next_position):
        lib().f64_forward(C.byref(self.cfg), C.byref(self._wp), C.byref(self._rs),
                          C.c_int(position), C.c_int(next_position))
        return self.logits

    def layer_ptr(self, i):
        return self._layers[i]


def ref_layer_matvec_set(layer_ptr, dim, hidden_dim, xb, x):
    """The reference's C# CPU path (Unpack + Expected loops) for one decoder
    layer's mat-vec set; returns (q, k, v, x_out, h)."""
    q, k, v = (np.empty(dim, np.float16) for _ in range(3))
    h = np.empty(hidden_dim, np.float16)
    xo = np.array(x, np.float16, copy=True)
    lib().ref_layer_matvec_set(C.byref(layer_ptr), C.c_int(dim), C.c_int(hidden_dim), _h(xb),
                               _h(q), _h(k), _h(v), _h(xo), _h(h))
    return q, k, v, xo, h
