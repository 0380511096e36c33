"""Host-side mirror of the calibration arithmetic of amct_pytorch/quantize_op/smooth_quant_module.py: the
per-channel activation statistics with their running update (:79-91), the smoothing factor (:113-133) and the
per-tensor activation parameters (:170-178).  The reductions over tokens and over output channels run in the
column-statistics kernel; the factor itself is a [1, K] tensor and stays in torch on the device."""
import torch

from .. import ops
from .utils import calculate_scale_offset


def new_channel_stats(weight):
    """(data_max, data_min) as the module initialises them (:58-61): [1, K] of the weight's dtype, -inf / +inf."""
    k = weight.shape[-1]
    data_max = torch.full((1, k), float('-inf'), dtype=weight.dtype, device=weight.device)
    data_min = torch.full((1, k), float('inf'), dtype=weight.dtype, device=weight.device)
    return data_max, data_min


@torch.no_grad()
def update_channel_min_max(inputs, data_max, data_min):
    """One calibration batch (:79-80, :88-91): per input channel amax / amin over all tokens, then
    data_max = batch_max > data_max ? batch_max : data_max and the mirror image for data_min.  Returns the new
    (data_max, data_min), [1, K], in the promoted dtype of inputs and the running tensors like torch.where."""
    x2 = inputs.reshape(-1, inputs.shape[-1])
    out_dtype = torch.promote_types(x2.dtype, data_max.dtype)
    cmax = data_max.reshape(-1).to(torch.float32).contiguous()
    cmin = data_min.reshape(-1).to(torch.float32).contiguous()
    ops.col_minmax(x2, cmax, cmin)
    return cmax.reshape(1, -1).to(out_dtype), cmin.reshape(1, -1).to(out_dtype)


@torch.no_grad()
def calculate_smooth(act_max, weight, smooth_strength):
    """:113-133.  wts_max = |W|.amax(dim=0) from the column kernel; factor = act_max^a / wts_max^(1-a), with
    1 wherever the factor is below eps of its dtype or not finite."""
    wts_max = ops.col_minmax(weight, absolute=True).reshape(1, -1).to(weight.dtype)
    smooth_factor = (act_max ** smooth_strength) / (wts_max ** (1 - smooth_strength))
    zero_mask = smooth_factor < torch.finfo(act_max.dtype).eps
    invalid_mask = ~torch.isfinite(smooth_factor)
    return torch.where(zero_mask | invalid_mask, torch.ones((), dtype=smooth_factor.dtype, device=smooth_factor.device),
                       smooth_factor)


@torch.no_grad()
def smooth_factor_from_stats(data_max, data_min, weight, smooth_strength):
    """:93-95: act_max = max(|data_max|, |data_min|), then calculate_smooth."""
    act_max = torch.max(data_max.abs(), data_min.abs())
    return calculate_smooth(act_max, weight, smooth_strength)


@torch.no_grad()
def per_tensor_params(data_max, data_min, smooth_factor, symmetric, act_type):
    """:170-178: scale_d / offset_d of the smoothed activation from the channel statistics."""
    max_val = (data_max / smooth_factor).max().reshape(-1)
    min_val = (data_min / smooth_factor).min().reshape(-1)
    return calculate_scale_offset(max_val, min_val, symmetric, act_type)
