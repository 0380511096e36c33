"""Host-side mirror of the weight optimisation of amct_pytorch/quantize_op/gptq_module.py (:91-155, :161-186)
with the tensors resident on the device.  The column loop of each block is one kernel launch
(amct_gptq_block); ordering, damping, the two Cholesky factorisations and the trailing update are library
calls on the device, as they are library calls in the reference."""
import math

import torch

from .. import _lib, ops
from .utils import calculate_scale_offset, get_weight_min_max_by_granularity


@torch.no_grad()
def update_hessian(hessian, nsamples, input_data, columns):
    """:161-186.  Returns (hessian, nsamples); the matrix stays on the device instead of moving to the host.
    For bf16 / fp16 activations on the device the update runs in place: the returned tensor IS the `hessian` passed in
    (the reference and the fp32 branch below build a new tensor per call) -- pass a clone to keep the earlier value.
    That branch applies 2 / n to the fp32 sum of exact products instead of scaling every element by sqrt(2 / n) first,
    so it matches the reference to fp32 rounding, not bit for bit."""
    if len(input_data.shape) == 2:
        input_data = input_data.unsqueeze(0)
    batch_size = input_data.shape[0]
    rows = input_data.reshape((-1, input_data.shape[-1]))
    if rows.is_cuda and rows.dtype in (torch.bfloat16, torch.float16):
        # the matrix-pipe kernel: one pass over the lower triangle of H, the product of the 16-bit values exact in fp32
        if hessian is None:
            hessian = torch.empty((columns, columns), dtype=torch.float32, device=rows.device)
            beta = 0.0
        else:
            beta = nsamples / (nsamples + batch_size)
        nsamples += batch_size
        hessian = ops.hessian_update(hessian, rows, beta, 2 / nsamples)
    else:
        # fp32 activations keep the fp32 product
        x = rows.t()
        if hessian is None:
            hessian = torch.zeros((columns, columns), device=x.device)
        hessian = hessian * (nsamples / (nsamples + batch_size))
        nsamples += batch_size
        x = math.sqrt(2 / nsamples) * x.float()
        hessian = hessian + x.matmul(x.t())
    if not torch.isfinite(hessian).all():
        raise RuntimeError("hessian matrix has invalid value, inf or nan.")
    return hessian, nsamples


def gptq_block(weight_sorted, i1, i2, hinv, scale_w, offset_w, gidx, qmin, qmax):
    """The column loop of block [i1, i2) in place on weight_sorted [N, columns] fp32; returns err_block."""
    dev = ops._dev(weight_sorted, hinv, scale_w, offset_w, gidx)
    n, columns = weight_sorted.shape
    count = i2 - i1
    err = torch.empty(n, count, dtype=torch.float32, device=dev)
    if scale_w.numel() == 1:
        stride = 0
    else:
        stride = scale_w.numel() // n
    w_ptr = weight_sorted.data_ptr() + i1 * 4
    h_ptr = hinv.data_ptr() + (i1 * hinv.shape[1] + i1) * 4
    with torch.cuda.device(dev):
        _lib.check(_lib.load().amct_gptq_block(
            w_ptr, columns, err.data_ptr(), count, h_ptr, hinv.shape[1], scale_w.data_ptr(),
            None if offset_w is None else offset_w.data_ptr(), stride, gidx.data_ptr(), n, count, qmin, qmax,
            torch.cuda.current_stream(dev).cuda_stream))
    return err


@torch.no_grad()
def get_opt_weight_and_quant_factor(weight, hessian, quant_config, block_size=128, perc_damp=0.01):
    """:91-155.  weight [N, K] (any float dtype), hessian [K, K] fp32 on the same device.  Returns
    (optimised weight in the weight's dtype, scale_w, offset_w)."""
    cfg = quant_config.get('weights_cfg')
    group_size = cfg.get('group_size')
    wts_type = cfg.get('quant_type')
    bits = int(wts_type.replace('int', ''))
    columns = weight.shape[1]
    out_dtype = weight.dtype
    weight = weight.clone().float()
    hessian = hessian.clone()
    dead = torch.diag(hessian) == 0
    hessian[dead, dead] = 1
    weight[:, dead] = 0
    perm = torch.argsort(torch.diag(hessian), descending=True)
    invperm = torch.argsort(perm)
    weight_min, weight_max = get_weight_min_max_by_granularity(weight, quant_config)
    scale_w, offset_w = calculate_scale_offset(weight_max, weight_min, cfg.get('symmetric'), wts_type)
    ws = weight[:, perm].contiguous()
    hs = hessian[perm][:, perm]
    damp = perc_damp * torch.mean(torch.diag(hs))
    diag = torch.arange(columns, device=weight.device)
    hs[diag, diag] += damp
    hs = torch.linalg.cholesky(hs)
    hs = torch.cholesky_inverse(hs)
    hinv = torch.linalg.cholesky(hs, upper=True).contiguous()
    sc = scale_w.reshape(-1).float().contiguous()
    zc = None if offset_w is None else offset_w.reshape(-1).to(torch.int32).contiguous()
    if group_size:
        gidx_all = (perm // group_size).to(torch.int32)
    else:
        gidx_all = torch.zeros(columns, dtype=torch.int32, device=weight.device)
    qmin, qmax = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
    for i1 in range(0, columns, block_size):
        i2 = min(i1 + block_size, columns)
        err_block = gptq_block(ws, i1, i2, hinv, sc, zc, gidx_all[i1:i2].contiguous(), qmin, qmax)
        if i2 < columns:
            ws[:, i2:] -= err_block.matmul(hinv[i1:i2, i2:])
    return ws[:, invperm].to(out_dtype), scale_w, offset_w
