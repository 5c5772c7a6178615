"""Host-side orchestration of the decode path, mirroring src/Transformer.cs,
src/TransformerWeights.cs, src/RunState.cs and src/Sampler.cs over the C ABI.  Text (tokenizer, chat templating) is outside
this path: Generate takes and yields token ids.
"""
import ctypes as C
import math

import numpy as np

from . import capi
from .device import DeviceArena, DeviceVariable, QWeight, init
from .modules import (Argmax, CumulativeSum, Embedding, MatVec, MatVecResidual, MatVecStrided, MatVecSwiGLU,
                      QKVMatVec, RMSNorm, RoPERotation, SampleTopP, Softmax, SoftmaxLogits, Sort, VecMat)


def make_config(d):
    return capi.Config(d["dim"], d["hidden_dim"], d["n_layers"], d["n_heads"], d["n_kv_heads"],
                       d["vocab_size"], d["seq_len"], d["rope_theta"])


class PerLayerWeight:
    """src/PerLayerWeight.cs:5-16"""
    pass


class TransformerWeights:
    """src/TransformerWeights.cs:6-104, fed from host arrays (the dict of
    managedllama2_amd.synth.random_model or of modelfile.read_model)."""

    def __init__(self, config, host):
        self.config = config
        from . import modelfile
        cfg = {k: getattr(config, k) for k in modelfile.FIELDS}
        tensors = 3 + config.n_layers * (7 * 3 + 2)
        self.arena = DeviceArena(modelfile.expected_size(cfg) + tensors * DeviceArena.ALIGN)
        up = self.arena.from_host

        def upq(W, Z, S):
            return QWeight(up(W), up(Z), up(S))

        self.tokenEmbeddingTable = up(host["embedding"])
        self.classifierWeights = up(host["classifier"])
        self.rmsFinalWeight = up(host["rms_final"])
        self.layers = []
        for L in host["layers"]:
            w = PerLayerWeight()
            w.queryWeight = upq(*L["q"])
            w.keyWeight = upq(*L["k"])
            w.valueWeight = upq(*L["v"])
            w.outputWeight = upq(*L["o"])
            w.upWeight = upq(*L["up"])
            w.gateWeight = upq(*L["gate"])
            w.downWeight = upq(*L["down"])
            w.rmsAttentionWeight = up(L["rms_att"])
            w.rmsFeedForwardWeight = up(L["rms_ffn"])
            self.layers.append(w)

    def struct(self):
        arr = (capi.LayerWeights * len(self.layers))()
        for i, w in enumerate(self.layers):
            arr[i] = capi.LayerWeights(w.queryWeight.struct(), w.keyWeight.struct(), w.valueWeight.struct(),
                                       w.outputWeight.struct(), w.gateWeight.struct(), w.upWeight.struct(),
                                       w.downWeight.struct(), w.rmsAttentionWeight.ptr,
                                       w.rmsFeedForwardWeight.ptr)
        self._layer_array = arr  # keep alive
        return capi.TransformerWeights(self.tokenEmbeddingTable.ptr, self.classifierWeights.ptr,
                                       self.rmsFinalWeight.ptr, arr)


class RunState:
    """src/RunState.cs:5-55.  config.seq_len is clamped to what fits in free
    device memory minus an 8 MiB reserve, as CalculateMaxUsableSequence does."""

    def __init__(self, config, kvDim):
        def max_usable_sequence():
            free = C.c_size_t()
            total = C.c_size_t()
            capi.call("llama2_mem_info", C.byref(free), C.byref(total))
            remaining = free.value - 8 * 1024 * 1024
            required = config.n_layers * kvDim * 2 * 2 + 4 + config.vocab_size * 4
            return int(min(remaining // required, config.seq_len))

        half = np.float16
        self.x = DeviceVariable(half, config.dim)
        self.xb = DeviceVariable(half, config.dim)
        self.h = DeviceVariable(half, config.hidden_dim)
        self.q = DeviceVariable(half, config.dim)
        self.attention = DeviceVariable(half, config.n_heads * max(config.dim, config.seq_len))
        self.logits = DeviceVariable(half, config.vocab_size)
        config.seq_len = max_usable_sequence()
        self.keyCache = DeviceVariable.zeros(half, config.n_layers * config.seq_len * kvDim)
        self.valueCache = DeviceVariable.zeros(half, config.n_layers * config.seq_len * kvDim)
        self.tokens = DeviceVariable.zeros(np.int32, config.seq_len + 1)
        self.indices = DeviceVariable(np.int32, config.vocab_size)

    def struct(self):
        return capi.RunState(self.x.ptr, self.xb.ptr, self.h.ptr, self.q.ptr, self.attention.ptr,
                             self.logits.ptr, self.keyCache.ptr, self.valueCache.ptr, self.tokens.ptr,
                             self.indices.ptr)


class Sampler:
    """src/Sampler.cs:5-72.  `random` supplies the coin (a callable returning a
    float in [0, 1)); the reference draws it from an unseeded System.Random."""

    def __init__(self, config, runstate, temperature=0.0, topP=0.9, random=None):
        self.config, self.runstate = config, runstate
        self.temperature, self.topP = float(temperature), float(topP)
        self.random = random if random is not None else np.random.default_rng().random
        self.argmax = Argmax(config)
        self.softmax = SoftmaxLogits(config)
        self.cumulativeSum = CumulativeSum(config)
        self.sampleTopP = SampleTopP(config)
        self.sort = Sort(config)

    def Sample(self, nextPosition, generateToken):
        coin = float(np.float32(self.random()))
        rs, n = self.runstate, self.config.vocab_size
        if self.temperature == 0.0 or not generateToken:
            self.argmax.Forward(rs.logits, n, rs.tokens, nextPosition, generateToken)
        else:
            self.softmax.Forward(rs.logits, n, self.temperature, rs.indices)
            if self.topP <= 0 or self.topP >= 1:
                threshold = coin
            else:
                self.sort.Forward(rs.logits, rs.indices, n)
                threshold = float(np.float32(coin) * np.float32(self.topP))
            self.cumulativeSum.Forward(rs.logits, n)
            self.sampleTopP.Forward(rs.logits, rs.indices, n, threshold, rs.tokens, nextPosition)
        return int(rs.tokens[nextPosition])


class Transformer:
    """src/Transformer.cs:6-191.  `mode` None drives the step module by module
    from the host exactly like the C# Forward; a capi.DECODE_* value hands the
    step to llama2_decode_forward."""

    def __init__(self, config_dict, host_weights, mode=None, device=0, temperature=0.0, topP=0.9, random=None):
        init(device)
        self.config = make_config(config_dict)
        c = self.config
        if c.rope_theta != 10000.0:
            raise capi.Llama2Error(capi.ERR_INVALID_ARGUMENT, "Invalid model config")  # Config.cs:27-28
        self.kvDim = c.dim * c.n_kv_heads // c.n_heads
        if self.kvDim != c.dim:
            raise NotImplementedError("Differing kvDim dimention not currently supported.")  # Transformer.cs:55-56
        self.weights = TransformerWeights(c, host_weights)
        self.runstate = RunState(c, self.kvDim)
        self.sampler = Sampler(c, self.runstate, temperature, topP, random)
        self.embedding = Embedding(c)
        self.rmsNorm = RMSNorm(c)
        self.qkvMatVec = QKVMatVec(c)
        self.rope = RoPERotation(c)
        self.matVecStrided = MatVecStrided(c)
        self.softmax = Softmax(c)
        self.vecMat = VecMat(c)
        self.matVecResidual = MatVecResidual(c)
        self.matVecSwiGLU = MatVecSwiGLU(c)
        self.matVec = MatVec(c)
        self.mode = mode
        self._decoder = None
        if mode is not None:
            self._w_struct = self.weights.struct()
            self._s_struct = self.runstate.struct()
            h = C.c_void_p()
            capi.call("llama2_decode_create", C.byref(h), C.byref(c), C.byref(self._w_struct),
                      C.byref(self._s_struct), mode)
            self._decoder = h

    def close(self):
        if self._decoder is not None:
            capi.call("llama2_decode_destroy", self._decoder)
            self._decoder = None

    def Generate(self, promptTokens, steps, stop_on_special=True):
        """src/Transformer.cs:89-112 on token ids."""
        promptTokens = [int(t) for t in promptTokens]
        self.runstate.tokens.copy_to_device(np.array(promptTokens, np.int32))
        for pos in range(steps):
            nextPos = pos + 1
            self.Forward(pos, nextPos)
            generateToken = nextPos >= len(promptTokens)
            token = self.Sample(nextPos, generateToken) if generateToken else promptTokens[nextPos]
            if stop_on_special and token < 3:
                break
            yield token

    def Sample(self, nextPos, generateToken):
        if self._decoder is not None:
            tok = C.c_int()
            sp = self.sampler
            capi.call("llama2_decode_sample_top_p", self._decoder, nextPos, 1 if generateToken else 0,
                      sp.temperature, sp.topP, float(np.float32(sp.random())), C.byref(tok))
            return tok.value
        return self.sampler.Sample(nextPos, generateToken)

    def MultiHeadAttention(self, output, query, key, value, attention, headSize, dim, seqLength, layerOffset,
                           scale):
        """src/Transformer.cs:150-156"""
        self.matVecStrided.Forward(attention, query, key, headSize, dim, seqLength, layerOffset, scale)
        self.softmax.Forward(attention, seqLength)
        self.vecMat.Forward(output, value, attention, headSize, dim, seqLength, layerOffset)

    def Forward(self, position, nextPosition):
        """src/Transformer.cs:158-190"""
        if self._decoder is not None:
            capi.call("llama2_decode_forward", self._decoder, position, nextPosition)
            return
        c, rs, w = self.config, self.runstate, self.weights
        headSize = c.dim // c.n_heads
        scale = 1.0 / math.sqrt(headSize)
        self.embedding.Forward(rs.x, w.tokenEmbeddingTable, c.dim, rs.tokens, position)
        for i, layer in enumerate(w.layers):
            self.rmsNorm.Forward(rs.xb, rs.x, layer.rmsAttentionWeight, c.dim)
            layerOffset = i * c.seq_len * self.kvDim
            self.qkvMatVec.Forward(rs.q, rs.keyCache, rs.valueCache, rs.xb, layer.queryWeight, layer.keyWeight,
                                   layer.valueWeight, c.dim, c.dim, layerOffset, position)
            self.rope.Forward(rs.q, rs.keyCache, c.n_kv_heads, headSize, position, layerOffset, c.rope_theta)
            self.MultiHeadAttention(rs.xb, rs.q, rs.keyCache, rs.valueCache, rs.attention, headSize, c.dim,
                                    nextPosition, layerOffset, scale)
            self.matVecResidual.Forward(rs.x, rs.xb, layer.outputWeight, c.dim, c.dim)
            self.rmsNorm.Forward(rs.xb, rs.x, layer.rmsFeedForwardWeight, c.dim)
            self.matVecSwiGLU.Forward(rs.h, rs.xb, layer.gateWeight, layer.upWeight, c.dim, c.hidden_dim)
            self.matVecResidual.Forward(rs.x, rs.h, layer.downWeight, c.hidden_dim, c.dim)
        self.rmsNorm.Forward(rs.x, rs.x, w.rmsFinalWeight, c.dim)
        self.matVec.Forward(rs.logits, rs.x, w.classifierWeights, c.dim, c.vocab_size)
