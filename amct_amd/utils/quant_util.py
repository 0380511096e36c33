"""Host-side mirror of amct_pytorch/utils/quant_util.py: same function names, argument meaning,
return shapes/dtypes and error messages; every arithmetic step runs in a HIP kernel.
Layout helpers (pad / reshape) are torch views and copies."""
import math

import torch

from .. import ops
from .vars import INT4, INT8


def pad_zero_by_group(tensor, group_size):
    """amct_pytorch/utils/quant_util.py:23-36."""
    pad = (group_size - (tensor.shape[-1] % group_size)) % group_size
    return torch.nn.functional.pad(tensor, (0, pad), 'constant', 0)


def convert_to_per_group_shape(input_tensor, group_size):
    """[N,K] -> [N, ceil(K/g), g] with right zero padding (quant_util.py:39-53)."""
    padded = pad_zero_by_group(input_tensor, group_size)
    return padded.reshape(padded.shape[0], padded.shape[1] // group_size, group_size)


def _bits(kind):
    return int(kind.replace('int', ''))


def _as_2d(t):
    if t.dim() == 3:                       # already grouped [N,G,g]
        return t.reshape(t.shape[0], -1), t.shape[-1]
    return t, None


def _factor_layout(tensor2d, scale, group_size):
    """Map the reference's broadcastable factor shapes onto the kernels' (group, flat factors)."""
    n = scale.numel()
    rows, cols = tensor2d.shape
    if group_size:
        g = math.ceil(cols / group_size)
        if n != rows * g:
            raise RuntimeError("scale has {} elements, expected {} x {}".format(n, rows, g))
        return group_size
    if n == 1:
        return -1
    if n == rows:
        return 0
    raise RuntimeError("scale.shape should be equal to 1 or cout. current is {}".format(n))


@torch.no_grad()
def convert_dtype(ori_tensor, quant_dtype):
    """round-half-even, saturate, narrow: int8 -> torch.int8, int4 -> torch.int32 (one code per
    element) (quant_util.py:56-73)."""
    if quant_dtype not in (INT8, INT4):
        raise ValueError('Not supported quant_dtype {}'.format(quant_dtype))
    bits = _bits(quant_dtype)
    shape = ori_tensor.shape
    flat = ori_tensor.reshape(-1, shape[-1])
    one = torch.ones(1, dtype=torch.float32, device=ori_tensor.device)
    _, codes = ops.quant_with_params(flat, one, None, -1, -(1 << (bits - 1)), (1 << (bits - 1)) - 1, want_dq=False,
                                     codes_kind=ops.CODES_I8 if bits == 8 else ops.CODES_I32)
    return codes.reshape(shape)


def quant_weight(tensor, wts_type, scale, offset=None, group_size=None):
    """tensor / scale (+ offset) -> integer codes (quant_util.py:76-93).  With group_size the result
    keeps the grouped shape [N, ceil(K/g), g] like the reference (pad columns hold the code of 0)."""
    if wts_type not in (INT8, INT4):
        raise ValueError('Not supported quant_dtype {}'.format(wts_type))
    bits = _bits(wts_type)
    src = tensor
    if group_size:
        src = pad_zero_by_group(tensor, group_size)
    group = _factor_layout(src, scale, group_size)
    _, codes = ops.quant_with_params(src, scale.reshape(-1), None if offset is None else offset.reshape(-1), group,
                                     -(1 << (bits - 1)), (1 << (bits - 1)) - 1, want_dq=False,
                                     codes_kind=ops.CODES_I8 if bits == 8 else ops.CODES_I32)
    if group_size:
        return codes.reshape(codes.shape[0], codes.shape[1] // group_size, group_size)
    return codes


def apply_smooth_weight(smooth_factor, ori_weight):
    """W * smooth, in W's dtype (quant_util.py:96-111)."""
    smooth_factor = smooth_factor.to(device=ori_weight.device, dtype=ori_weight.dtype)
    if list(smooth_factor.shape) != [1, ori_weight.shape[1]]:
        raise RuntimeError("smooth_factor shape should be {} current shape is {}"
                           .format([1, ori_weight.shape[1]], list(smooth_factor.shape)))
    return ops.col_scale(ori_weight, smooth_factor, divide=False)


def check_scale_offset_shape(weight, scale_w, offset_w=None, group_size=None):
    """quant_util.py:114-140."""
    if group_size is None:
        if scale_w.shape[0] == 1:
            return
        if scale_w.shape[0] == weight.shape[0]:
            return
        raise RuntimeError("scale.shape should be equal to 1 or cout. current is {}, "
                           "pls check quant factors from quantize model".format(scale_w.shape[0]))
    if list(scale_w.shape) != [weight.shape[0], math.ceil(weight.shape[1] / group_size), 1]:
        raise RuntimeError(
            "scale.shape should be [{}] current shape is {}, please check quant factors from quantize model.".format(
                (weight.shape[0], math.ceil(weight.shape[1] / group_size), 1), list(scale_w.shape)))
    if offset_w is None:
        return
    if scale_w.shape != offset_w.shape:
        raise RuntimeError("offset_w.shape should be equal to scale_w.shape,"
                           " pls check quant factors from quantize model")


def apply_awq_quantize_weight(weight_tensor, awq_scale, group_size):
    """W / awq_scale (quant_util.py:143-159)."""
    cin = weight_tensor.shape[1]
    if list(awq_scale.shape) != [1, cin]:
        raise RuntimeError("AWQ params scale.shape should be [1, {}] current shape is {}".format(
            cin, list(awq_scale.shape)))
    return ops.col_scale(weight_tensor, awq_scale, divide=True)


def quant_dequant_weight(tensor, quant_params=None, scale=None, offset=None):
    """Fake-quantise with given factors, result in tensor's dtype and shape
    (quant_util.py:162-188)."""
    wts_dtype = quant_params.get('weights_cfg').get('quant_type')
    group_size = quant_params.get('weights_cfg').get('group_size')
    bits = _bits(wts_dtype)
    group = _factor_layout(tensor, scale, group_size)
    dq, _ = ops.quant_with_params(tensor, scale.reshape(-1), None if offset is None else offset.reshape(-1), group,
                                  -(1 << (bits - 1)), (1 << (bits - 1)) - 1)
    return dq
