"""Interchange formats of the reference's checkpoint converter
(amct_pytorch/experimental/quantization/DeepSeekV3.2/deploy.py), same function names and arguments, tensors on
the GPU.  weight_dequant, pack_4bit and scale_fp32_to_u64 are one kernel each; int_weight_quant composes them
with the fake-quant kernel; int4_assistance_bias is a row reduction left to torch on the device."""
import torch

from . import _lib, ops


def _launch(fn, *args, dev):
    with torch.cuda.device(dev):
        _lib.check(fn(*args, torch.cuda.current_stream(dev).cuda_stream))


def weight_dequant(weight, scale, block_size=128):
    """deploy.py:48-92: fp8 (E4M3FN) weight [M, N] times its per-block fp32 scale, in the default dtype."""
    if weight.dim() != 2 or scale.dim() != 2:
        raise AssertionError("weight and scale must be 2-D")
    M, N = weight.shape
    assert scale.shape[0] == (M + block_size - 1) // block_size, "Mismatch in scale rows and weight rows."
    assert scale.shape[1] == (N + block_size - 1) // block_size, "Mismatch in scale columns and weight columns."
    dev = ops._dev(weight, scale)
    if weight.dtype != torch.float8_e4m3fn:
        raise RuntimeError("weight_dequant: expected a float8_e4m3fn weight, got {}".format(weight.dtype))
    out_dtype = torch.get_default_dtype()
    out = torch.empty(M, N, dtype=out_dtype, device=dev)
    w8 = weight.contiguous().view(torch.uint8)
    sc = scale.to(torch.float32).contiguous()
    _launch(_lib.load().amct_fp8_block_dequant, w8.data_ptr(), sc.data_ptr(), out.data_ptr(), M, N, block_size,
            ops.dtype_code(out_dtype), dev=dev)
    return out


def scale_fp32_to_u64(weight_scale):
    """deploy.py:95-107: [k, n] fp32 scales -> [k, n] uint64 words with the scale's bits in the low half."""
    dev = ops._dev(weight_scale)
    s = weight_scale.float().contiguous()
    out = torch.empty(s.shape, dtype=torch.uint64, device=dev)
    _launch(_lib.load().amct_scale_f32_to_u64, s.data_ptr(), out.data_ptr(), s.numel(), dev=dev)
    return out


def pack_4bit(x):
    """deploy.py:110-127: int8 [n, k] of int4 values -> int8 [n/2, k], pairs of output channels per byte."""
    assert x.dtype == torch.int8
    dev = ops._dev(x)
    x = x.contiguous()
    n, k = x.shape
    if n % 2:
        raise RuntimeError("pack_4bit: the number of output channels must be even")
    y = torch.empty(n // 2, k, dtype=torch.int8, device=dev)
    _launch(_lib.load().amct_pack_int4_pairs_n, x.data_ptr(), y.data_ptr(), n, k, dev=dev)
    return y


def int4_assistance_bias(weight, weight_scale):
    """deploy.py:149-157: (scale * weight * 8).sum(dim=1) in fp32 (a reduction whose order, and so its last
    bits, belong to the library that runs it)."""
    repeat_times = weight.shape[1] // weight_scale.shape[1]
    expanded_scale = weight_scale.repeat_interleave(repeat_times, dim=1)
    return (expanded_scale * weight * 8).sum(dim=1).float()


def int_weight_quant(tensor, bits=8, weight_clip_factor=None):
    """deploy.py:128-146: per-channel absmax quantisation, clamp [-qmax, qmax]; int4 results are packed and
    come with the widened scales and the assistance bias."""
    assert tensor.dim() == 2
    qmax = 2 ** (bits - 1) - 1
    if weight_clip_factor is not None:
        # the clipped scale is absmax * factor / qmax: staged path through the parameter-given kernel
        abs_max = ops.col_minmax(tensor.t().contiguous(), absolute=True).reshape(-1, 1).to(tensor.dtype)
        scale = abs_max * weight_clip_factor / qmax
        _, codes = ops.quant_with_params(tensor, scale.reshape(-1).float(), None, 0, -qmax, qmax, want_dq=False,
                                         codes_kind=ops.CODES_I8, via_src=tensor.dtype != torch.float32)
    else:
        _, codes, s32, _ = ops.fakequant_int(tensor, bits, True, group=0, want_dq=False, codes_kind=ops.CODES_I8,
                                             scope_rule=ops.SCOPE_ABSMAX, qmin=-qmax, qmax=qmax,
                                             via_src=tensor.dtype != torch.float32)
        scale = s32.reshape(-1, 1).to(tensor.dtype)
    if bits == 4:
        bias = int4_assistance_bias(codes, scale)
        return pack_4bit(codes), scale_fp32_to_u64(scale), bias
    return codes, scale.to(torch.float32), None


# ---- compressed-tensors description of a converted checkpoint ------------------------------------------
# Host-side mirror of experimental/quantization/DeepSeekV3.2/deploy.py:171-238: the `quantization_config` block
# that the converter writes into config.json, so that a checkpoint quantised here is described exactly as one the
# reference converted.  Pure dictionaries; the field names are those of the compressed-tensors format.

_PER_LAYER_UNQUANTISED = ("self_attn.indexer.wk", "self_attn.indexer.weights_proj", "self_attn.kv_b_proj",
                          "self_attn.kv_a_proj_with_mqa", "self_attn.q_a_proj")


def generate_ignore_item(num_layers, num_hidden_layers, first_k_dense_replace):
    """Names of the modules that stay unquantised (deploy.py:171-188): five attention projections of every layer,
    the MoE router of the sparse layers, the two extra heads of the multi-token-prediction layers, `lm_head`."""
    names = []
    for layer in range(num_layers):
        prefix = "model.layers.%d." % layer
        names.extend(prefix + leaf for leaf in _PER_LAYER_UNQUANTISED)
        if layer >= first_k_dense_replace:
            names.append(prefix + "mlp.gate")
        if layer >= num_hidden_layers:
            names.extend((prefix + "eh_proj", prefix + "shared_head.head"))
    names.append("lm_head")
    return names


def generate_w4a8_quant(num_layers, first_k_dense_replace):
    """The expert blocks of the sparse layers, which take the W4A8 scheme (deploy.py:191-196)."""
    return ["model.layers.%d.mlp.experts" % layer for layer in range(first_k_dense_replace, num_layers)]


def _tensor_scheme(num_bits, dynamic, observer, strategy):
    return {"actorder": None, "block_structure": None, "dynamic": dynamic, "group_size": None, "num_bits": num_bits,
            "observer": observer, "observer_kwargs": {}, "strategy": strategy, "symmetric": True, "type": "int"}


def generate_quant_group(a_num_bits=8, w_num_bits=8, targets=None, activation_use_clip=False):
    """One config group (deploy.py:199-211): dynamic per-token symmetric activations, static per-channel symmetric
    weights."""
    return {"input_activations": _tensor_scheme(a_num_bits, True, "memoryless", "token"),
            "activation_use_clip": activation_use_clip,
            "output_activations": None,
            "targets": targets,
            "weights": _tensor_scheme(w_num_bits, False, "minmax", "channel")}


def generate_quant_config(c8, ignores, w4a8=False, clip=False):
    """The whole `quantization_config` (deploy.py:214-238): group_0 = W8A8 on every Linear; with `w4a8` group_1 = W4A8
    on the grouped expert GEMM; with `c8` an fp8 group-128 KV-cache scheme (its two flags are the strings the
    reference writes, not booleans)."""
    groups = {"group_0": generate_quant_group(8, 8, ["Linear"])}
    if w4a8:
        groups["group_1"] = generate_quant_group(8, 4, ["MoEGMM"], activation_use_clip=clip)
    kv = {"num_bits": 8, "type": "float", "strategy": "group", "group_size": 128, "dynamic": "true",
          "symmetric": "true"} if c8 else None
    return {"config_groups": groups, "format": "int-quantized", "global_compression_ratio": 1, "ignore": ignores,
            "kv_cache_scheme": kv, "quant_method": "compressed-tensors", "quantization_status": "compressed"}
