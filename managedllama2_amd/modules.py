"""The reference's module API (one class per kernel, src/<Module>.cs) over the
C ABI.  Constructor and Forward signatures follow the C# classes; launch
geometry, which the C# constructors fixed from Config, lives in the library.
"""
from . import capi


def _ceil_div(a, b):
    return (a + (b - 1)) // b


def _sizes(rows):
    scales_size = _ceil_div(rows, 128)
    weights_size = _ceil_div(rows, 32) * 4
    zeros_size = _ceil_div(scales_size, 8)
    return zeros_size, scales_size, weights_size


class Module:
    """src/Module.cs:7-26"""

    def __init__(self, config=None):
        self.config = config
        capi.load()


class MatVec(Module):
    """src/MatVec.cs:6-17"""

    def Forward(self, output, input, matrix, rows, cols):
        capi.call("llama2_mat_vec", output.ptr, input.ptr, matrix.ptr, rows, cols)


class QKVMatVec(Module):
    """src/QKVMatVec.cs:7-33"""

    def __init__(self, config):
        super().__init__(config)
        self.kvDim = config.dim * config.n_kv_heads // config.n_heads

    def Forward(self, queryOutput, keyOutput, valueOutput, input, query, key, value, rows, cols, layerOffset, pos):
        zs, ss, ws = _sizes(rows)
        offset = layerOffset + pos * self.kvDim
        capi.call("llama2_qkv_mat_vec", queryOutput.ptr, keyOutput.offset_pointer(offset),
                  valueOutput.offset_pointer(offset), input.ptr,
                  query.Weight.ptr, query.Zeros.ptr, query.Scales.ptr,
                  key.Weight.ptr, key.Zeros.ptr, key.Scales.ptr,
                  value.Weight.ptr, value.Zeros.ptr, value.Scales.ptr, rows, cols, zs, ss, ws)


class MatVecSwiGLU(Module):
    """src/MatVecSwiGLU.cs:6-25"""

    def Forward(self, output, input, g, u, rows, cols):
        zs, ss, ws = _sizes(rows)
        capi.call("llama2_mat_vec_swiglu", output.ptr, input.ptr, g.Weight.ptr, g.Zeros.ptr, g.Scales.ptr,
                  u.Weight.ptr, u.Zeros.ptr, u.Scales.ptr, rows, cols, zs, ss, ws)


class MatVecResidual(Module):
    """src/MatVecResidual.cs:6-24"""

    def Forward(self, output, input, matrix, rows, cols):
        zs, ss, ws = _sizes(rows)
        capi.call("llama2_mat_vec_residual_int4", output.ptr, input.ptr, matrix.Weight.ptr, matrix.Zeros.ptr,
                  matrix.Scales.ptr, rows, cols, zs, ss, ws)


class MatVecInt4(Module):
    """The plain int4 mat-vec (device function mat_vec_int4,
    native/mat_vec_kernel.cu:166-177); the reference has no module of its own
    for it, QKVMatVec runs three of them."""

    def Forward(self, output, input, matrix, rows, cols):
        zs, ss, ws = _sizes(rows)
        capi.call("llama2_mat_vec_int4", output.ptr, input.ptr, matrix.Weight.ptr, matrix.Zeros.ptr,
                  matrix.Scales.ptr, rows, cols, zs, ss, ws)


class MatVecStrided(Module):
    """src/MatVecStrided.cs:7-20"""

    def Forward(self, attention, query, key, headSize, dim, seqLength, layerOffset, scale):
        capi.call("llama2_mat_vec_strided", attention.ptr, query.ptr, key.offset_pointer(layerOffset), headSize,
                  seqLength, headSize, headSize, dim, seqLength, scale, self.config.n_heads)


class VecMat(Module):
    """src/VecMat.cs:7-20"""

    def Forward(self, output, value, attention, headSize, dim, seqLength, layerOffset):
        capi.call("llama2_vec_mat", output.ptr, attention.ptr, value.offset_pointer(layerOffset), headSize,
                  seqLength, headSize, headSize, dim, self.config.n_heads)


class RMSNorm(Module):
    """src/RMSNorm.cs:5-15"""

    def Forward(self, output, input, weights, size, eps=1e-5):
        capi.call("llama2_rmsnorm", output.ptr, input.ptr, weights.ptr, size, eps)


class RoPERotation(Module):
    """src/RoPERotation.cs:6-25"""

    def __init__(self, config):
        super().__init__(config)
        self.kvDim = config.dim * config.n_kv_heads // config.n_heads

    def Forward(self, query, key, numKVHeads, headSize, pos, layerOffset, theta):
        offset = layerOffset + pos * self.kvDim
        capi.call("llama2_rope", query.ptr, key.offset_pointer(offset), numKVHeads, headSize, pos, theta,
                  self.config.n_heads)


class Softmax(Module):
    """src/Softmax.cs:5-15"""

    def Forward(self, attention, seqLength):
        capi.call("llama2_softmax", attention.ptr, seqLength, self.config.n_heads)


class Argmax(Module):
    """src/Argmax.cs:5-15"""

    def Forward(self, logits, vocabSize, tokens, nextPos, generateToken):
        capi.call("llama2_argmax", logits.ptr, vocabSize, tokens.ptr, nextPos, 1 if generateToken else 0)


class Embedding(Module):
    """src/Embedding.cs:5-15"""

    def Forward(self, output, table, size, tokens, pos):
        capi.call("llama2_embedding", output.ptr, table.ptr, size, tokens.ptr, pos)


class SoftmaxLogits(Module):
    """src/SoftmaxLogits.cs:5-16"""

    def Forward(self, logits, size, temperature, indices):
        capi.call("llama2_softmax_logits", logits.ptr, size, temperature, indices.ptr)


class Sort(Module):
    """src/Sort.cs:5-16"""

    def Forward(self, logits, indices, size):
        capi.call("llama2_sort", logits.ptr, indices.ptr, size)


class CumulativeSum(Module):
    """src/CumulativeSum.cs:5-16"""

    def Forward(self, logits, size):
        capi.call("llama2_cumulative_sum", logits.ptr, size)


class SampleTopP(Module):
    """src/SampleTopP.cs:5-16"""

    def Forward(self, logits, indices, size, threshold, tokens, nextPos):
        capi.call("llama2_sample_top_p", logits.ptr, indices.ptr, size, threshold, tokens.ptr, nextPos)
