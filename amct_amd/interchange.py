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
