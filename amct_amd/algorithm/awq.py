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
