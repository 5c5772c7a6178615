"""ctypes binding of libllama2_host.so, the C facade over the C++ host layer
(managedllama2_amd/host/llama2_host.hpp)."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# LLAMA2_HOST_LIB names another build of the facade (the sanitizer build of tests/test_oracle_sanitize.py)
LIB_PATH = os.environ.get("LLAMA2_HOST_LIB") or os.path.join(_HERE, "libllama2_host.so")

HOST_LOOP, MODULES, FUSED, FUSED_GRAPH = -1, 0, 1, 3
_lib = None


class HostError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(message)
        self.code = code  # 1 FileLoadException, 2 NotImplementedException, 3 Llama2Exception


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HostError(4, "%s is not built (make -C managedllama2_amd/host)" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        lib.l2h_last_error.restype = C.c_char_p
        lib.l2h_check_model_file.argtypes = [C.c_char_p]
        lib.l2h_transformer_open.argtypes = [C.c_char_p, C.c_int, C.c_int, C.POINTER(C.c_void_p)]
        lib.l2h_transformer_open_sampled.argtypes = [C.c_char_p, C.c_int, C.c_int, C.c_float, C.c_float,
                                                     C.c_ulonglong, C.POINTER(C.c_void_p)]
        u32p, u16p = C.POINTER(C.c_uint32), C.POINTER(C.c_uint16)
        lib.l2h_repack_qweight.argtypes = [u32p, u32p, u16p, C.c_int, C.c_int, C.c_int, u32p, u32p, u16p]
        lib.l2h_transformer_generate.argtypes = [C.c_void_p, C.POINTER(C.c_int), C.c_int, C.c_int, C.POINTER(C.c_int),
                                                 C.POINTER(C.c_int)]
        lib.l2h_transformer_logits.argtypes = [C.c_void_p, C.POINTER(C.c_uint16), C.c_int]
        lib.l2h_transformer_seq_len.argtypes = [C.c_void_p]
        lib.l2h_transformer_close.argtypes = [C.c_void_p]
        _lib = lib
    return _lib


def _check(rc):
    if rc != 0:
        raise HostError(rc, load().l2h_last_error().decode())


def check_model_file(path):
    _check(load().l2h_check_model_file(path.encode()))


class Transformer:
    """libLlama2::Transformer (ITransformer on token ids)."""

    def __init__(self, model_path, mode=HOST_LOOP, stop_on_special=True, temperature=0.0, top_p=0.9, seed=0):
        self._h = C.c_void_p()
        if temperature == 0.0:
            _check(load().l2h_transformer_open(model_path.encode(), mode, 1 if stop_on_special else 0,
                                               C.byref(self._h)))
        else:
            _check(load().l2h_transformer_open_sampled(model_path.encode(), mode, 1 if stop_on_special else 0,
                                                       temperature, top_p, seed, C.byref(self._h)))

    def Generate(self, prompt_tokens, steps):
        prompt = (C.c_int * len(prompt_tokens))(*[int(t) for t in prompt_tokens])
        out = (C.c_int * max(steps, 1))()
        n = C.c_int()
        _check(load().l2h_transformer_generate(self._h, prompt, len(prompt_tokens), steps, out, C.byref(n)))
        return list(out[:n.value])

    def logits(self, vocab_size):
        out = np.empty(vocab_size, np.float16)
        _check(load().l2h_transformer_logits(self._h, out.ctypes.data_as(C.POINTER(C.c_uint16)), vocab_size))
        return out

    @property
    def seq_len(self):
        return load().l2h_transformer_seq_len(self._h)

    def close(self):
        if self._h:
            _check(load().l2h_transformer_close(self._h))
            self._h = C.c_void_p()


def repack_qweight(qweight, qzeros, scales, height, width, fmt=0):
    """libLlama2::ModelConverter::RepackQWeight (fmt 0 = Format.v0, 1 = Format.v1) -> (Weight, Zeros, Scales)."""
    ss = (height + 127) // 128
    W = np.empty(((height + 7) // 8) * width, np.uint32)
    Z = np.empty(((ss + 7) // 8) * width, np.uint32)
    S = np.empty(ss * width, np.float16)
    qweight = np.ascontiguousarray(qweight, np.uint32).ravel()
    qzeros = np.ascontiguousarray(qzeros, np.uint32).ravel()
    scales = np.ascontiguousarray(scales, np.float16).ravel()
    u32p, u16p = C.POINTER(C.c_uint32), C.POINTER(C.c_uint16)
    _check(load().l2h_repack_qweight(qweight.ctypes.data_as(u32p), qzeros.ctypes.data_as(u32p),
                                     scales.ctypes.data_as(u16p), height, width, fmt, W.ctypes.data_as(u32p),
                                     Z.ctypes.data_as(u32p), S.ctypes.data_as(u16p)))
    return W, Z, S
