"""The tensor side of src/ModelConverter.cs over the C ABI: RepackQWeightByName
(:196-275) on the GPU and Convert's output order (:127-173).  Reading the
PyTorch checkpoint itself (zip + pickle, :175-188, :330-394) is not part of
this path: Convert takes the tensors as arrays, under the checkpoint's names.
"""
import numpy as np

from . import capi, modelfile
from .device import DeviceVariable, init

GROUP_SIZE = 128
V0, V1 = "v0", "v1"  # ModelConverter.Format (:125): AWQ "GEMM" tensors / tensors already output-major


def _ceil_div(a, b):
    return (a + (b - 1)) // b


def RepackQWeight(qweight, qzeros, scales, height, width, fmt=V0):
    """One int4 tensor: height = inputs (K), width = outputs (N).  Returns the
    (Weight, Zeros, Scales) host arrays in the layout of the model file."""
    init(0)
    scales_size = _ceil_div(height, GROUP_SIZE)
    weights_size = _ceil_div(height, 8)
    zeros_size = _ceil_div(scales_size, 8)
    qweight = np.ascontiguousarray(qweight).view(np.uint32).ravel()
    qzeros = np.ascontiguousarray(qzeros).view(np.uint32).ravel()
    scales = np.ascontiguousarray(scales).view(np.float16).ravel()
    if fmt == V0:
        w8 = _ceil_div(width, 8)
        if qweight.size != w8 * height or qzeros.size != w8 * scales_size or scales.size != scales_size * width:
            raise ValueError("tensor sizes do not match height=%d width=%d (Format.v0)" % (height, width))
        d_in, d_out = DeviceVariable.from_host(qweight), DeviceVariable(np.uint32, weights_size * width)
        capi.call("llama2_repack_qdata", d_out.ptr, d_in.ptr, height, width)
        z_in, z_out = DeviceVariable.from_host(qzeros), DeviceVariable(np.uint32, zeros_size * width)
        capi.call("llama2_repack_qdata", z_out.ptr, z_in.ptr, scales_size, width)
        s_in, s_out = DeviceVariable.from_host(scales), DeviceVariable(np.float16, scales_size * width)
        capi.call("llama2_repack_scales", s_out.ptr, s_in.ptr, scales_size, width)
        return d_out.to_host(), z_out.to_host(), s_out.to_host()
    if fmt == V1:
        if qweight.size != weights_size * width or qzeros.size != zeros_size * width or \
                scales.size != zeros_size * 8 * width:
            raise ValueError("tensor sizes do not match height=%d width=%d (Format.v1)" % (height, width))
        s_in, s_out = DeviceVariable.from_host(scales), DeviceVariable(np.float16, scales_size * width)
        capi.call("llama2_compact_scales_v1", s_out.ptr, s_in.ptr, scales_size, width)
        return qweight.copy(), qzeros.copy(), s_out.to_host()
    raise ValueError("Format is not supported")  # :234, :265


# checkpoint name -> (file key, height, width) in Convert's order (:160-167): q, k, v, o, UP, GATE, down
def _layer_tensors(cfg):
    dim, hidden = cfg["dim"], cfg["hidden_dim"]
    kv_dim = dim * cfg["n_kv_heads"] // cfg["n_heads"]
    return (("self_attn.q_proj", "q", dim, dim), ("self_attn.k_proj", "k", dim, kv_dim),
            ("self_attn.v_proj", "v", dim, kv_dim), ("self_attn.o_proj", "o", dim, dim),
            ("mlp.up_proj", "up", dim, hidden), ("mlp.gate_proj", "gate", dim, hidden),
            ("mlp.down_proj", "down", hidden, dim))


def Convert(output_path, cfg, state, fmt=V0):
    """Writes the model file from a state dictionary {checkpoint tensor name: array}."""
    model = {"embedding": state["model.embed_tokens.weight"], "classifier": state["lm_head.weight"],
             "rms_final": state["model.norm.weight"], "layers": []}
    for i in range(cfg["n_layers"]):
        name = "model.layers.%d" % i
        L = {}
        for tensor, key, height, width in _layer_tensors(cfg):
            L[key] = RepackQWeight(state["%s.%s.qweight" % (name, tensor)], state["%s.%s.qzeros" % (name, tensor)],
                                   state["%s.%s.scales" % (name, tensor)], height, width, fmt)
        L["rms_att"] = state[name + ".input_layernorm.weight"]
        L["rms_ffn"] = state[name + ".post_attention_layernorm.weight"]
        model["layers"].append(L)
    modelfile.write_model(output_path, cfg, model)
