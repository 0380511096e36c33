"""Integer quantisation oracle (CPU, eager torch) -- test infrastructure only.

Every function restates, op for op and in the same order, what the reference
executes on CPU tensors, because bit-exactness against that eager path is the
parity bar.  The op order matters (fp32 true division, a separate add of the
offset, round-half-even, clamp, ...), the Python around it does not.

Reference lines followed (paths relative to the reference root):

  group_view / ungroup          amct_pytorch/utils/quant_util.py:23-53,
                                amct_pytorch/quantize_op/utils.py:139-155
  sym_scope / scale_offset      amct_pytorch/quantize_op/utils.py:26-108,158-176
  weight_min_max                amct_pytorch/quantize_op/utils.py:111-136
  to_codes / quant_codes        amct_pytorch/utils/quant_util.py:56-93
  fake_quant                    amct_pytorch/utils/quant_util.py:162-188
  awq_fake_quant                amct_pytorch/algorithm/awq.py:129-170 with
                                amct_pytorch/utils/data_utils.py:48-66
  awq_grid_step                 amct_pytorch/algorithm/awq.py:30-49
  smooth_weight / awq_weight    amct_pytorch/utils/quant_util.py:96-111,143-159
  absmax_quant (variant B)      amct_pytorch/experimental/quantization/
                                DeepSeekV3.2/deploy.py:128-146
  token_min_max                 amct_pytorch/quantize_op/minmax_module.py:96-105
  dynamic_token_quant           composition of token_min_max, scale_offset
                                (symmetric) and quant_codes on the live batch;
                                the experimental tree's dynamic form
                                (.../cores/quantization/node.py:39-43,181-204)
                                is restated as dynamic_token_quant_absmax.

Pin status: every function here is pinned by tests/test_oracle_int.py --
hand-computed known answers that are exact in fp32 (power-of-two scales, ties
to even), numpy float32 cross-computation of the IEEE division chain, the
zero-padding rule for ragged groups, and range/idempotence invariants -- and
by tests/golden/int_quant_kat.json, the whole chain computed with exact
fractions and an explicit round-to-nearest-even after every operation (no
floating-point library involved), which both this oracle and the HIP path must
reproduce bit for bit.
"""
import math

import torch

EPS_F32 = 1.192092896e-7          # quantize_op/utils.py:23


def _bits(kind):
    return int(kind.replace('int', ''))


# --------------------------------------------------------------------------
# layout helpers
# --------------------------------------------------------------------------
def group_view(t, g):
    """[N,K] -> [N,ceil(K/g),g]; the tail of the last group is zero-filled and
    those zeros take part in every later min/max (quant_util.py:23-53)."""
    tail = (-t.shape[-1]) % g
    if tail:
        t = torch.nn.functional.pad(t, (0, tail), 'constant', 0)
    return t.reshape(t.shape[0], t.shape[1] // g, g)


def ungroup(t, shape):
    """Inverse of group_view: flatten groups, drop pad columns
    (quantize_op/utils.py:139-155)."""
    if t.shape == shape:
        return t
    return t.reshape(t.shape[0], t.shape[1] * t.shape[2])[:shape[0], :shape[1]]


# --------------------------------------------------------------------------
# min/max -> scale, offset
# --------------------------------------------------------------------------
def sym_scope(kind, neg_dominates):
    """127 (7) normally, 128 (8) where |min| > |max| (utils.py:158-176).
    `neg_dominates` is a bool tensor; bool + int promotes to int64."""
    return neg_dominates + 2 ** (_bits(kind) - 1) - 1


def scale_offset(vmax, vmin, symmetric, kind, check=True):
    """(scale fp32, offset int32|None) from max/min (utils.py:75-108)."""
    vmax = vmax.to(torch.float32)
    vmin = vmin.to(torch.float32)
    nbits = _bits(kind)
    if symmetric:
        neg = vmax.abs() < vmin.abs()
        scope = sym_scope(kind, neg)
        bound = torch.where(vmax.abs() > vmin.abs(), vmax.abs(), vmin.abs())
        scale = bound / scope
        offset = None
    else:
        vmax = torch.clamp(vmax, 0, None)
        vmin = torch.clamp(vmin, None, 0)
        scope = 2 ** nbits - 1
        half = math.ceil(scope / 2)
        scale = (vmax - vmin) / scope
        offset = torch.where(vmax != vmin, -half - vmin / scale,
                             torch.tensor(-half, dtype=vmax.dtype))
    # eps guard (utils.py:26-51)
    tiny = scale < EPS_F32
    if not symmetric:
        offset = torch.where(tiny, torch.tensor(-(2.0 ** (nbits - 1))), offset)
    scale = torch.where(tiny, torch.tensor(1.0), scale)
    if check:
        check_scale_offset(scale, offset)
    scale = scale.to(torch.float32)
    if offset is not None:
        offset = offset.round().to(torch.int32)
    return scale, offset


def check_scale_offset(scale, offset):
    """utils.py:54-72 -- same messages, same exception type."""
    if not torch.all(torch.isfinite(scale)) or not torch.all(torch.isfinite(1 / scale)):
        raise RuntimeError("Param scale has invalid value inf, nan or zeros!")
    if offset is not None and not torch.all(torch.isfinite(offset)):
        raise RuntimeError("Param offset has invalid value inf or nan!")


def weight_min_max(w, strategy, group_size=None):
    """(min, max) per channel [N,1], per tensor [1,1] or per group [N,G,1]
    (utils.py:111-136)."""
    if strategy == 'channel':
        return (w.min(dim=1, keepdim=True).values, w.max(dim=1, keepdim=True).values)
    if strategy == 'tensor':
        return w.min().reshape(1, 1), w.max().reshape(1, 1)
    wg = group_view(w, group_size)
    return (wg.min(dim=-1, keepdim=True).values, wg.max(dim=-1, keepdim=True).values)


def weight_scale_offset(w, strategy, symmetric, kind, group_size=None):
    """awq.py:121-126 / minmax_module.py:69-77."""
    vmin, vmax = weight_min_max(w, strategy, group_size)
    return scale_offset(vmax, vmin, symmetric, kind)


# --------------------------------------------------------------------------
# elementwise quantisation
# --------------------------------------------------------------------------
def to_codes(t, kind):
    """round-half-even, saturate, narrow (quant_util.py:56-73); int4 codes are
    held one per int32."""
    if kind == 'int8':
        return t.round().clamp(-128, 127).to(torch.int8)
    if kind == 'int4':
        return t.round().clamp(-8, 7).to(torch.int32)
    raise ValueError('Not supported quant_dtype {}'.format(kind))


def quant_codes(w, kind, scale, offset=None, group_size=None):
    """w/scale (+offset) -> codes (quant_util.py:76-93).  Output keeps the
    grouped shape [N,G,g] when group_size is given."""
    if group_size:
        w = group_view(w, group_size)
    t = w / scale
    if offset is not None:
        t = t + offset
    return to_codes(t, kind)


def fake_quant(w, kind, scale, offset=None, group_size=None):
    """quantise then dequantise, result in w's dtype (quant_util.py:162-188)."""
    nbits = _bits(kind)
    shape = w.shape
    src = w.dtype
    if group_size:
        w = group_view(w, group_size)
    t = w / scale
    if offset is not None:
        t = t + offset
    t = torch.clamp(torch.round(t), -(2 ** (nbits - 1)), 2 ** (nbits - 1) - 1)
    if offset is not None:
        t = t - offset
    t = t * scale
    return t.reshape(shape[0], -1)[:, :shape[1]].to(src)


def awq_fake_quant(w, kind, scale, offset, strategy, group_size=None):
    """AWQ's own fake-quant: the scaled value is narrowed to the weight dtype
    BEFORE rounding (awq.py:129-149 -> data_utils.py:48-66 -> awq.py:152-170)."""
    nbits = _bits(kind)
    src = w.dtype
    shape = w.shape
    # do_quant
    t = group_view(w, group_size) if strategy == 'group' else w
    t = t / scale
    if offset is not None:
        t += offset
    t = ungroup(t, shape).to(src)
    # convert_precision
    t = torch.clamp(torch.round(t), -(2 ** (nbits - 1)), 2 ** (nbits - 1) - 1)
    # do_dequant
    if strategy == 'group':
        t = group_view(t, group_size)
    if offset is not None:
        t = t - offset
    keep = t.dtype
    t = t * scale
    return ungroup(t, shape).to(keep)


def awq_grid_step(w, awq_scale, kind, strategy, symmetric, group_size=None):
    """One grid point of the AWQ search applied to one weight
    (awq.py:30-49): W*s -> factors -> fake-quant -> /s.  Returns
    (new_weight, scale, offset)."""
    ws = w.mul(awq_scale)
    scale, offset = weight_scale_offset(ws, strategy, symmetric, kind, group_size)
    dq = awq_fake_quant(ws, kind, scale, offset, strategy, group_size)
    return dq / awq_scale, scale, offset


def smooth_weight(smooth, w):
    """quant_util.py:96-111."""
    smooth = smooth.to(dtype=w.dtype)
    if list(smooth.shape) != [1, w.shape[1]]:
        raise RuntimeError("smooth_factor shape should be {} current shape is {}"
                           .format([1, w.shape[1]], list(smooth.shape)))
    return w * smooth


def awq_weight(w, awq_scale):
    """quant_util.py:143-159."""
    if list(awq_scale.shape) != [1, w.shape[1]]:
        raise RuntimeError("AWQ params scale.shape should be [1, {}] current shape is {}".format(
            w.shape[1], list(awq_scale.shape)))
    return w / awq_scale


def absmax_quant(w, bits=8, clip=None):
    """Variant B: s = absmax/qmax, clamp to +-qmax, no eps guard
    (experimental .../deploy.py:128-146, the non-packing branch)."""
    qmax = 2 ** (bits - 1) - 1
    amax = torch.abs(w).max(dim=1, keepdim=True)[0]
    if clip is not None:
        amax = amax * clip
    s = amax / qmax
    q = torch.clamp(torch.round(w / s), -qmax, qmax)
    return q.to(torch.int8), s.to(torch.float32)


# --------------------------------------------------------------------------
# activations
# --------------------------------------------------------------------------
def token_min_max(x):
    """amax/amin over every dim except -2, keepdim (minmax_module.py:96-105).
    For a 2-D [M,K] input this is one (min,max) per row."""
    dims = list(range(x.dim()))
    dims.pop(-2)
    return torch.amin(x, dim=tuple(dims), keepdim=True), torch.amax(x, dim=tuple(dims), keepdim=True)


def dynamic_token_quant(x, smooth_recip=None):
    """Per-token dynamic symmetric int8: optional x*(1/smooth) in x's dtype
    (npu_quantization_linear.py:96-97), row min/max, symmetric scale with the
    127/128 scope rule, codes = clamp(rne(x/s)).  Returns (int8 [M,K], s [M])."""
    if smooth_recip is not None:
        x = x * smooth_recip
    vmin, vmax = x.amin(dim=-1, keepdim=True), x.amax(dim=-1, keepdim=True)
    s, _ = scale_offset(vmax, vmin, True, 'int8')
    return quant_codes(x, 'int8', s), s.reshape(-1)


def dynamic_token_quant_absmax(x, bits=8):
    """The experimental tree's dynamic per-token symmetric form
    (node.py:181-204 with sym_quant :39-43): s = absmax/qmax, s=1 for an
    all-zero row, clamp [-(qmax+1), qmax]."""
    qmax = 2 ** (bits - 1) - 1
    r = x.reshape(-1, x.shape[-1])
    vmax, vmin = r.amax(1, keepdim=True), r.amin(1, keepdim=True)
    z = torch.zeros_like(vmax)
    vmax, vmin = torch.maximum(vmax, z), torch.minimum(vmin, z)
    vmax = torch.maximum(torch.abs(vmin), vmax)
    dead = vmax == 0
    s = vmax / torch.tensor(qmax)
    s[dead] = 1
    q = torch.clamp((r / s).round(), -(qmax + 1), qmax)
    return q.to(torch.int8), s.reshape(-1)


def static_quantize(x, scales, zero_points, axis=-1):
    """The activation-quantise operator as the deploy module calls it
    (npu_quantization_linear.py:98-99, div_mode=False): multiply by the stored
    reciprocal scale, add the offset, round-half-even, saturate to int8.
    `axis=-1`: scales broadcast over the last dim (1 element = per tensor);
    `axis=-2`: one scale per row of the last-but-one dim (per token).
    The operator itself lives in the un-vendored torch_npu package: the
    precision of the multiply-add, the rounding and the saturation inside it
    are PARITY UNPINNED; this states the documented semantics with the
    multiply and the add each done (and rounded) in fp32."""
    if axis == -2:
        shp = [1] * x.dim()
        shp[-2] = -1
        sc = scales.reshape(shp)
        zp = zero_points.reshape(shp) if zero_points is not None else None
    else:
        sc, zp = scales, zero_points
    t = x.float() * sc.float()
    if zp is not None:
        t = t + zp.float()
    return t.round().clamp(-128, 127).to(torch.int8)


def awq_loss(ori_out, quant_out):
    """The loss of one AWQ grid point (amct_pytorch/algorithm/awq.py:96): the difference in the tensors' own
    dtype (one rounding), its fourth power and the mean in fp64 (the reference's fp32 mean is one rounding of
    this sum order-for-order; comparisons against it carry that tolerance).  Pinned by closed forms in the
    tests: a constant difference d gives d^4, a single non-zero difference d gives d^4 / n, the sign of the
    difference does not matter, and a difference that the dtype cannot represent is rounded first."""
    d = (ori_out - quant_out).double()
    return float((d * d * d * d).mean()) if d.numel() else float('nan')


def awq_search_scale(inputs, weights, forward, grids_num, kind, strategy, symmetric, group_size=None):
    """The AWQ scale search (amct_pytorch/algorithm/awq.py:52-105) on plain tensors: `weights` are the
    [N,K] weights of the layers that share the input, `forward(inputs, weights)` evaluates the block.
    Returns (best_scale [1,K], losses per grid point as Python floats).  Test infrastructure only.
    Parity unpinned beyond its parts: the grid step is awq_grid_step (pinned above); the loop, the scale
    formula and the loss are restated from the cited lines and have no independent check."""
    if not torch.isfinite(inputs).all():
        raise RuntimeError("Run AWQ error! Invalid value(nan or inf) in activation!")
    for w in weights:
        if not torch.isfinite(w).all():
            raise RuntimeError("Run AWQ error! Invalid value(nan or inf) in weight!")
    ori_out = forward(inputs, weights)
    min_loss = torch.tensor(float('inf'))
    best_scale = None
    losses = []
    inputs_mean = inputs.abs().contiguous().view(-1, inputs.shape[-1]).mean(0)
    for grid in range(grids_num):
        ratio = grid / grids_num
        scale_awq = inputs_mean.pow(ratio).clamp(min=1e-4).to(torch.float64).view(1, -1)
        scale_awq = scale_awq / (scale_awq.max() * scale_awq.min()).sqrt()
        scale_awq = torch.clamp(scale_awq.to(inputs.dtype), 1e-4, torch.finfo(inputs.dtype).max)
        new_w = [awq_grid_step(w, scale_awq, kind, strategy, symmetric, group_size)[0] for w in weights]
        quant_out = forward(inputs, new_w)
        loss = (ori_out - quant_out).float().pow(4).mean()
        losses.append(float(loss))
        if not torch.isnan(loss) and loss < min_loss:
            min_loss = loss
            best_scale = scale_awq
    if best_scale is None or torch.isinf(min_loss):
        raise RuntimeError("Run AWQ error! Got invalid loss.")
    return best_scale, losses


# --------------------------------------------------------------------------
# SmoothQuant calibration statistics (amct_pytorch/quantize_op/smooth_quant_module.py)
# --------------------------------------------------------------------------
def channel_min_max_update(inputs, data_max, data_min):
    """:79-80, :88-91 -- batch amax / amin per input channel over all tokens, then the running update."""
    batch_max = inputs.reshape(-1, inputs.shape[-1]).amax(dim=0, keepdim=True)
    batch_min = inputs.reshape(-1, inputs.shape[-1]).amin(dim=0, keepdim=True)
    data_max = torch.where(batch_max > data_max, batch_max, data_max)
    data_min = torch.where(batch_min < data_min, batch_min, data_min)
    return data_max, data_min


def smooth_factor(act_max, weight, smooth_strength):
    """:113-133 -- act_max^a / (|W|.amax(dim=0))^(1-a), 1 where below eps or not finite."""
    wts_max = weight.abs().amax(dim=0, keepdim=True)
    f = (act_max ** smooth_strength) / (wts_max ** (1 - smooth_strength))
    bad = (f < torch.finfo(act_max.dtype).eps) | ~torch.isfinite(f)
    return torch.where(bad, torch.tensor(1.0, dtype=f.dtype), f)
