"""Host-side mirror of the fake-quant half of amct_pytorch/algorithm/awq.py (:30-49, :121-170).
process_weights_for_layers runs one fused kernel per layer and grid point; do_quant / do_dequant
remain available as separate calls with the reference's signatures."""
import torch

from .. import ops
from ..quantize_op.utils import calculate_scale_offset, get_weight_min_max_by_granularity
from ..utils.data_utils import convert_precision  # noqa: F401


def calculate_scale_offset_by_granularity(weight, quant_config):
    """awq.py:121-126."""
    weight_min, weight_max = get_weight_min_max_by_granularity(weight, quant_config)
    cfg = quant_config.get('weights_cfg')
    return calculate_scale_offset(weight_max, weight_min, cfg.get('symmetric'), cfg.get('quant_type'))


def _group_arg(scale, weight, granularity, group_size):
    if granularity == 'group':
        return group_size
    return -1 if scale.numel() == 1 else 0


def do_quant(weight, scale_w, offset_w, weight_granularity, group_size=None):
    """weight / scale (+ offset), narrowed to the weight's dtype, NOT rounded (awq.py:129-149)."""
    group = _group_arg(scale_w, weight, weight_granularity, group_size)
    out, _ = ops.quant_with_params(weight, scale_w.reshape(-1), None if offset_w is None else offset_w.reshape(-1),
                                   group, -128, 127, stage=ops.STAGE_SCALE)
    return out


def do_dequant(weight, scale, offset, weight_granularity, group_size=None):
    """(weight - offset) * scale in the weight's dtype (awq.py:152-170)."""
    group = _group_arg(scale, weight, weight_granularity, group_size)
    out, _ = ops.quant_with_params(weight, scale.reshape(-1), None if offset is None else offset.reshape(-1),
                                   group, -128, 127, stage=ops.STAGE_DEQUANT)
    return out


@torch.no_grad()
def process_weights_for_layers(layers, scale_awq, quant_config):
    """One AWQ grid point on every layer: W*s -> factors -> fake-quant (value narrowed to the weight
    dtype before rounding) -> /s, written back to layer.weight.data (awq.py:30-49).  One kernel
    launch per layer."""
    cfg = quant_config.get('weights_cfg')
    bits = int(cfg.get('quant_type').replace('int', ''))
    strategy = cfg.get('strategy')
    group_size = cfg.get('group_size')
    for layer in layers:
        w = layer.weight.data
        if strategy == 'tensor' or (strategy == 'group' and w.shape[1] % group_size):
            # per-tensor factors need a global reduction; ragged groups need padding: staged path
            ws = ops.col_scale(w, scale_awq.to(w.dtype), divide=False)
            scale, offset = calculate_scale_offset_by_granularity(ws, quant_config)
            group = -1 if strategy == 'tensor' else group_size
            dq, _ = ops.quant_with_params(ws, scale.reshape(-1), None if offset is None else offset.reshape(-1), group,
                                          -(1 << (bits - 1)), (1 << (bits - 1)) - 1, via_src=True)
            layer.weight.data = ops.col_scale(dq, scale_awq.to(w.dtype), divide=True)
            continue
        dq, _, _, _ = ops.fakequant_int(w, bits, bool(cfg.get('symmetric')), group=group_size if strategy == 'group' else 0,
                                        col_scale=scale_awq, col_mode=ops.COL_MUL_THEN_DIV, via_src=True)
        layer.weight.data = dq


def awq_scale_for_ratio(inputs_mean, ratio, dtype):
    """The candidate scale of one grid point (awq.py:85-88): mean|x| ** ratio, clamped, normalised by the
    geometric mean of its extremes in fp64, narrowed to the activation dtype and clamped again."""
    scale_awq = inputs_mean.pow(ratio).clamp(min=1e-4).to(torch.float64).view(1, -1)
    scale_awq = scale_awq / (scale_awq.max() * scale_awq.min()).sqrt()
    return torch.clamp(scale_awq.to(dtype), 1e-4, torch.finfo(dtype).max)


def _first_output(block, inputs, kwargs):
    out = block(inputs, **kwargs)
    return out[0] if isinstance(out, tuple) else out


def _require_finite(inputs, layers):
    if not bool(torch.isfinite(inputs).all()):
        raise RuntimeError("Run AWQ error! Invalid value(nan or inf) in activation!")
    if not all(bool(torch.isfinite(layer.weight.data).all()) for layer in layers):
        raise RuntimeError("Run AWQ error! Invalid value(nan or inf) in weight!")


@torch.no_grad()
def search_scale(inputs, layers, block, quant_config, kwargs=None):
    """AWQ scale search (awq.py:52-105) with everything resident on the device.  Same arguments, return
    value and errors as the reference.  The reference copies the whole state dict of `block` to the host
    once and loads it back after every grid point; only the weights of `layers` change inside the loop
    (process_weights_for_layers, which replaces layer.weight.data by a new tensor and never writes into the
    old one), so here the original weight tensors are simply kept and put back: no copy at all, the
    fake-quant of a grid point is one fused kernel per layer and its loss one pass over the two outputs."""
    _require_finite(inputs, layers)
    kwargs = kwargs or {}
    grids_num = quant_config.get("algorithm").get('awq').get('grids_num')
    target = _first_output(block, inputs, kwargs)
    channel_mean = inputs.abs().contiguous().view(-1, inputs.shape[-1]).mean(0)     # one value per input channel
    originals = [layer.weight.data for layer in layers]
    winner, winner_loss = None, torch.tensor(float('inf'), device=inputs.device)
    try:
        for grid in range(grids_num):
            candidate = awq_scale_for_ratio(channel_mean, grid / grids_num, inputs.dtype)
            process_weights_for_layers(layers, candidate, quant_config)
            loss = ops.awq_loss(target, _first_output(block, inputs, kwargs))
            if not torch.isnan(loss) and loss < winner_loss:
                winner, winner_loss = candidate, loss
            for layer, w in zip(layers, originals):
                layer.weight.data = w
    finally:
        for layer, w in zip(layers, originals):                                     # also after an exception
            layer.weight.data = w
    if winner is None or torch.isinf(winner_loss):
        raise RuntimeError("Run AWQ error! Got invalid loss.")
    return winner


@torch.no_grad()
def apply_scale(scale_awq, ori_module, input_data):
    """awq.py:108-118: fold the chosen scale into the weight and out of the activation, in place."""
    scale = scale_awq.to(ori_module.weight.device)
    ori_module.weight.data.mul_(scale)
    input_data.div_(scale)
