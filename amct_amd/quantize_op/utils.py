"""Host-side mirror of amct_pytorch/quantize_op/utils.py: min/max by granularity and the
(max, min) -> (scale, offset) closed form, computed by HIP kernels."""
import torch

from .. import ops
from ..utils.quant_util import convert_to_per_group_shape, pad_zero_by_group  # noqa: F401  (re-exported like the reference)

FLT_EPSILON = 1.192092896e-7


def check_scale_offset(scale, offset):
    """amct_pytorch/quantize_op/utils.py:54-72 -- same messages."""
    valid = bool(torch.all(torch.isfinite(scale))) and bool(torch.all(torch.isfinite(1 / scale)))
    if not valid:
        raise RuntimeError("Param scale has invalid value inf, nan or zeros!")
    if offset is not None and not torch.all(torch.isfinite(offset)):
        raise RuntimeError("Param offset has invalid value inf or nan!")


def get_int_quant_scope(data_type, symmetric, abs_max_is_negative=False):
    """2^b - 1 (asymmetric); 2^(b-1) - 1, plus one where the minimum dominates (symmetric)
    (utils.py:158-176)."""
    quant_bits = int(data_type.replace('int', ''))
    if not symmetric:
        return pow(2, quant_bits) - 1
    return abs_max_is_negative + pow(2, quant_bits - 1) - 1


def calculate_scale_offset(data_max, data_min, symmetric, data_type, check=True):
    """(scale fp32, offset int32 | None), shaped like data_max (utils.py:75-108).  Raises the
    reference's RuntimeError when a factor is not finite.  That check reads a flag back from the device, which
    synchronises the stream: check=False skips it for callers inside a loop (the factors are computed the same
    way, a non-finite one is simply not reported) -- validate once afterwards with check_scale_offset."""
    bits = int(data_type.replace('int', ''))
    dev = data_max.device
    if not check:
        return ops.scale_offset(data_max, data_min, bits, bool(symmetric))
    bad = torch.zeros(2, dtype=torch.int32, device=dev)
    scale, offset = ops.scale_offset(data_max, data_min, bits, bool(symmetric), bad=bad[:1])
    if int(bad[0].item()):
        # find which message the reference would give
        check_scale_offset(scale, None)
        raise RuntimeError("Param offset has invalid value inf or nan!")
    return scale, offset


def get_weight_min_max_by_granularity(weight_data, quant_config):
    """(min, max): [N,1] per channel, [1,1] per tensor, [N, ceil(K/g), 1] per group, in the weight's
    dtype (utils.py:111-136)."""
    cfg = quant_config.get('weights_cfg')
    strategy = cfg.get('strategy')
    if strategy == 'channel':
        mn, mx = ops.minmax(weight_data, 0)
        mn, mx = mn.reshape(-1, 1), mx.reshape(-1, 1)
    elif strategy == 'tensor':
        mn, mx = ops.minmax(weight_data, 0)
        mn, _ = ops.minmax(mn.reshape(1, -1), 0)
        _, mx = ops.minmax(mx.reshape(1, -1), 0)
        mn, mx = mn.reshape(1, 1), mx.reshape(1, 1)
    else:
        mn, mx = ops.minmax(weight_data, cfg.get('group_size'))
        mn, mx = mn.unsqueeze(-1), mx.unsqueeze(-1)
    # the extrema are elements of the weight (or 0): the narrowing is exact
    return mn.to(weight_data.dtype), mx.to(weight_data.dtype)


def convert_to_dst_shape(input_tensor, dst_shape):
    """Flatten groups and drop pad columns (utils.py:139-155)."""
    if input_tensor.shape == dst_shape:
        return input_tensor
    return input_tensor.reshape(input_tensor.shape[0],
                                input_tensor.shape[1] * input_tensor.shape[2])[:dst_shape[0], :dst_shape[1]]
