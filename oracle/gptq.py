"""GPTQ weight optimisation oracle (CPU, eager torch) -- test infrastructure only.

Restates amct_pytorch/quantize_op/gptq_module.py:
  block_loop      :128-151  the column loop of one block (quantise column, error, rank-1 update)
  optimize_weight :91-155   the whole routine (dead columns, ordering, damping, Cholesky, blocks)
  update_hessian  :161-186

Pin status: block_loop is elementwise fp32 arithmetic in a fixed order; tests/test_oracle_int.py checks it
against a scalar Python loop on numpy float32 values (one rounding per operation, written out).
optimize_weight and update_hessian go through
library factorisations and GEMMs whose summation order is the library's: parity unpinned, compared by
tolerance only.
"""
import math

import torch

from . import int_quant as iq


def block_loop(weight_block, hinv_block, kind, scale_cols, offset_cols):
    """weight_block [N, count] fp32 (modified in place and returned), hinv_block [count, count],
    scale_cols / offset_cols: lists of [N,1] (or [1,1]) factor tensors, one per column (offset None when
    symmetric).  Returns (weight_block, err_block)."""
    count = weight_block.shape[1]
    err_block = torch.zeros_like(weight_block)
    for i in range(count):
        w = weight_block[:, i]
        d = hinv_block[i, i]
        off = None if offset_cols is None else offset_cols[i]
        w_q = iq.fake_quant(w.reshape(-1, 1), kind, scale_cols[i], off).reshape(-1)
        err = (w - w_q) / d
        weight_block[:, i:] -= err.unsqueeze(1).matmul(hinv_block[i, i:].unsqueeze(0))
        err_block[:, i] = err
    return weight_block, err_block


def update_hessian(hessian, nsamples, input_data, columns):
    if input_data.dim() == 2:
        input_data = input_data.unsqueeze(0)
    batch_size = input_data.shape[0]
    x = input_data.reshape((-1, input_data.shape[-1])).t()
    if hessian is None:
        hessian = torch.zeros((columns, columns))
    hessian = hessian * (nsamples / (nsamples + batch_size))
    nsamples += batch_size
    x = math.sqrt(2 / nsamples) * x.float()
    hessian = hessian + x.matmul(x.t())
    if not torch.isfinite(hessian).all():
        raise RuntimeError("hessian matrix has invalid value, inf or nan.")
    return hessian, nsamples


def optimize_weight(weight, hessian, kind, strategy, symmetric, group_size=None, block_size=128, perc_damp=0.01):
    """Returns (optimised weight in the weight's dtype, scale_w, offset_w)."""
    columns = weight.shape[1]
    out_dtype = weight.dtype
    weight = weight.clone().float()
    hessian = hessian.clone()
    dead = torch.diag(hessian) == 0
    hessian[dead, dead] = 1
    weight[:, dead] = 0
    perm = torch.argsort(torch.diag(hessian), descending=True)
    invperm = torch.argsort(perm)
    scale_w, offset_w = iq.weight_scale_offset(weight, strategy, symmetric, kind, group_size)
    ws = weight[:, perm]
    hs = hessian[perm][:, perm]
    damp = perc_damp * torch.mean(torch.diag(hs))
    diag = torch.arange(columns)
    hs[diag, diag] += damp
    hs = torch.linalg.cholesky(hs)
    hs = torch.cholesky_inverse(hs)
    hinv = torch.linalg.cholesky(hs, upper=True)
    for i1 in range(0, columns, block_size):
        i2 = min(i1 + block_size, columns)
        scale_cols, offset_cols = [], (None if offset_w is None else [])
        for i in range(i2 - i1):
            if strategy == 'group':
                g = int(perm[i1 + i]) // group_size
                scale_cols.append(scale_w.reshape(weight.shape[0], -1)[:, g].unsqueeze(-1))
                if offset_w is not None:
                    offset_cols.append(offset_w.reshape(weight.shape[0], -1)[:, g].unsqueeze(-1))
            else:
                scale_cols.append(scale_w.reshape(-1, 1))
                if offset_w is not None:
                    offset_cols.append(offset_w.reshape(-1, 1))
        block = ws[:, i1:i2]
        _, err_block = block_loop(block, hinv[i1:i2, i1:i2], kind, scale_cols, offset_cols)
        ws[:, i2:] -= err_block.matmul(hinv[i1:i2, i2:])
    return ws[:, invperm].to(out_dtype), scale_w, offset_w
