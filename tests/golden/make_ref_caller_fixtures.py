#!/usr/bin/env python3
"""Writes tests/golden/ref_callers.pt: input/output vectors of the reference's own CPU path.

Runs only where the reference checkout exists (the build container): it imports the reference package from
/root/reference with `torch_npu` replaced by a MagicMock (the package imports that module lazily, inside methods,
and the reference's own tests stub it the same way), feeds seeded tensors through the functions below and stores
inputs and outputs with torch.save (plain tensors, ints, strings; loadable with weights_only=True).  The tests only
ever read the resulting file; nothing of the reference travels with it.

Covered (reference lines):
  * calculate_scale_offset / quant_dequant_weight / quant_weight for {int8,int4} x {sym,asym} x {tensor,channel,group}
    x {fp32,bf16,fp16}                                    quantize_op/utils.py:75-136, utils/quant_util.py:56-93,162-188
  * AWQ's do_quant -> convert_precision -> do_dequant     algorithm/awq.py:129-170, utils/data_utils.py:48-66
  * process_weights_for_layers, search_scale              algorithm/awq.py:30-105
  * SmoothQuant.forward statistics + calculate_smooth     quantize_op/smooth_quant_module.py:64-133
  * GPTQuant.update_hessian / get_opt_weight_and_quant_factor   quantize_op/gptq_module.py:86-186
  * NpuQuantizationLinear / NpuWeightQuantizedLinear registered buffers
                                                          deploy_op/npu_quantization_linear.py:27-130,
                                                          deploy_op/weight_npu_quant_module.py:29-100

Run from the repository root:  python tests/golden/make_ref_caller_fixtures.py
"""
import os
import sys
import tempfile
import types
from unittest.mock import MagicMock

import torch

REF = "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))


def cfg(kind, symmetric, strategy, group=None, algorithm=None, inputs=None, batch_num=1):
    w = {'quant_type': kind, 'symmetric': symmetric, 'strategy': strategy}
    if group:
        w['group_size'] = group
    return {'batch_num': batch_num, 'weights_cfg': w, 'inputs_cfg': inputs or {'enable_quant': False},
            'algorithm': algorithm or {'minmax': {}}}


def gen(seed, *shape, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def main():
    scratch = tempfile.mkdtemp(prefix="amct_ref_")
    os.chdir(scratch)                                   # the package writes a log directory into the cwd
    sys.path.insert(0, REF)
    npu = MagicMock()
    npu.npu.is_available.return_value = False
    npu.npu_convert_weight_to_int4pack.side_effect = lambda t: t     # keep the int32 [K,N] codes as they are
    sys.modules['torch_npu'] = npu
    torch.Tensor.npu = lambda self: self
    torch.set_num_threads(1)                            # one thread: reductions in a fixed order

    from amct_pytorch.quantize_op.utils import calculate_scale_offset, get_weight_min_max_by_granularity
    from amct_pytorch.utils.quant_util import quant_dequant_weight, quant_weight
    from amct_pytorch.utils.data_utils import convert_precision
    from amct_pytorch.algorithm import awq as rawq
    from amct_pytorch.quantize_op.smooth_quant_module import SmoothQuant
    from amct_pytorch.quantize_op.gptq_module import GPTQuant
    from amct_pytorch.deploy_op.npu_quantization_linear import NpuQuantizationLinear
    from amct_pytorch.deploy_op.weight_npu_quant_module import NpuWeightQuantizedLinear

    out = {"torch_version": str(torch.__version__)}

    # ---- the elementwise matrix ---------------------------------------------------------------
    matrix = []
    seed = 100
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        for kind in ('int8', 'int4'):
            for symmetric in (True, False):
                for strategy, group in (('tensor', None), ('channel', None), ('group', 32)):
                    seed += 1
                    w = gen(seed, 12, 80 if strategy == 'group' else 72, scale=0.05, dtype=dtype)
                    w[3] = w[3].abs()                   # a one-sided row: the zero clamp of the asymmetric form
                    w[5, :40] = 0
                    c = cfg(kind, symmetric, strategy, group)
                    mn, mx = get_weight_min_max_by_granularity(w, c)
                    s, z = calculate_scale_offset(mx, mn, symmetric, kind)
                    dq = quant_dequant_weight(w, c, s, z)
                    codes = quant_weight(w, kind, s, z, group)
                    t = rawq.do_quant(w.clone(), s, z, strategy, group)
                    t = convert_precision(t, kind)
                    adq = rawq.do_dequant(t, s, z, strategy, group)
                    matrix.append({"dtype": str(dtype), "kind": kind, "symmetric": symmetric, "strategy": strategy,
                                   "group": group or 0, "w": w, "min": mn, "max": mx, "scale": s,
                                   "offset": z, "dq": dq, "codes": codes, "awq_dq": adq})
    out["matrix"] = matrix

    # ---- one AWQ grid point and the scale search -------------------------------------------------
    searches = []
    for dtype, kind, symmetric, strategy, group, grids in (
            (torch.float32, 'int4', False, 'group', 32, 20), (torch.bfloat16, 'int4', False, 'group', 32, 20),
            (torch.bfloat16, 'int8', True, 'channel', None, 10), (torch.float16, 'int4', True, 'group', 64, 8)):
        seed += 1
        lin = [torch.nn.Linear(64, 32, bias=False), torch.nn.Linear(64, 48, bias=False)]
        for i, l in enumerate(lin):
            l.weight.data = gen(seed * 10 + i, l.out_features, 64, scale=0.05, dtype=dtype)

        class Block(torch.nn.Module):
            def __init__(self):
                super().__init__()
                self.a, self.b = lin

            def forward(self, x):
                return torch.cat([self.a(x), self.b(x)], dim=-1)

        blk = Block()
        x = gen(seed * 10 + 5, 96, 64, dtype=torch.float32)
        x = (x * (1 + 3 * torch.rand(64, generator=torch.Generator().manual_seed(seed)))).to(dtype)
        c = cfg(kind, symmetric, strategy, group, algorithm={'awq': {'grids_num': grids}})
        w0 = [l.weight.data.clone() for l in lin]
        with torch.no_grad():
            best = rawq.search_scale(x, lin, blk, c)
            # the weights after one explicit grid point (ratio 0.5 of the search's formula)
            sc = x.abs().view(-1, 64).mean(0).pow(0.5).clamp(min=1e-4).to(torch.float64).view(1, -1)
            sc = sc / (sc.max() * sc.min()).sqrt()
            sc = torch.clamp(sc.to(dtype), 1e-4, torch.finfo(dtype).max)
            rawq.process_weights_for_layers(lin, sc, c)
            w1 = [l.weight.data.clone() for l in lin]
        searches.append({"dtype": str(dtype), "kind": kind, "symmetric": symmetric, "strategy": strategy,
                         "group": group or 0, "grids": grids, "x": x, "weights": w0, "best_scale": best,
                         "grid_scale": sc, "grid_weights": w1})
    out["awq_search"] = searches

    # ---- SmoothQuant statistics and factor ---------------------------------------------------------
    smooth = []
    for dtype, strength, act_strategy in ((torch.bfloat16, 0.5, 'tensor'), (torch.float16, 0.3, 'tensor'),
                                          (torch.bfloat16, 0.8, 'token')):
        seed += 1
        lin = torch.nn.Linear(64, 32, bias=True)
        lin.weight.data = gen(seed, 32, 64, scale=0.05, dtype=dtype)
        lin.weight.data[:, 7] = 0                       # a dead weight column: 0 ** positive in the denominator
        lin.bias.data = gen(seed + 1000, 32, scale=0.1, dtype=dtype)
        c = cfg('int8', True, 'channel', algorithm={'smoothquant': {'smooth_strength': strength}},
                inputs={'quant_type': 'int8', 'symmetric': act_strategy == 'token', 'strategy': act_strategy},
                batch_num=2)
        m = SmoothQuant(lin, 'lin', c)
        xs = [gen(seed * 7 + i, 16, 64, dtype=dtype) for i in range(2)]
        xs[0][:, 9] = 0
        xs[1][:, 9] = 0                                 # a dead activation channel
        for x in xs:
            m(x)
        smooth.append({"dtype": str(dtype), "strength": strength, "act_strategy": act_strategy,
                       "weight": lin.weight.data.clone(), "bias": lin.bias.data.clone(), "inputs": xs,
                       "data_max": m.data_max, "data_min": m.data_min, "smooth": m.scale, "scale_w": m.scale_w,
                       "offset_w": m.offset_w, "scale_d": m.scale_d, "offset_d": m.offset_d})
        # the deploy module built from this calibrated module
        dep = NpuQuantizationLinear(m)
        smooth[-1]["deploy"] = {k: v.clone() for k, v in dep.state_dict().items()}
        smooth[-1]["deploy_bias"] = None if dep.bias is None else dep.bias.clone()
    out["smoothquant"] = smooth

    # ---- GPTQ ---------------------------------------------------------------------------------------
    gptq = []
    for dtype, kind, symmetric, strategy, group, cols in (
            (torch.float32, 'int4', False, 'group', 32, 160), (torch.bfloat16, 'int8', True, 'channel', None, 192),
            (torch.bfloat16, 'int4', True, 'tensor', None, 160), (torch.float16, 'int4', False, 'group', 64, 192)):
        seed += 1
        lin = torch.nn.Linear(cols, 32, bias=False)
        lin.weight.data = gen(seed, 32, cols, scale=0.05, dtype=dtype)
        c = cfg(kind, symmetric, strategy, group, algorithm={'gptq': {}}, batch_num=2)
        m = GPTQuant(lin, 'lin', c)
        xs = [gen(seed * 11 + i, 2, 56, cols, dtype=dtype) for i in range(2)]
        xs[0][..., 5] = 0
        xs[1][..., 5] = 0                               # a dead column of the Hessian
        w0 = lin.weight.data.clone()
        m.update_hessian(xs[0])
        m.update_hessian(xs[1])
        hess = m.hessian.clone()
        wopt, s, z = m.get_opt_weight_and_quant_factor()
        gptq.append({"dtype": str(dtype), "kind": kind, "symmetric": symmetric, "strategy": strategy,
                     "group": group or 0, "weight": w0, "inputs": xs if not gptq else None, "hessian": hess, "opt_weight": wopt,
                     "scale": s, "offset": z})
    out["gptq"] = gptq

    # ---- weight-only deploy buffers ---------------------------------------------------------------------
    deploy = []
    for dtype, kind, symmetric, strategy, group, with_awq in (
            (torch.bfloat16, 'int4', False, 'group', 32, True), (torch.bfloat16, 'int8', True, 'channel', None, False),
            (torch.float16, 'int8', False, 'group', 32, False), (torch.float16, 'int4', True, 'tensor', None, False),
            (torch.bfloat16, 'int8', False, 'tensor', None, True)):
        seed += 1
        w = gen(seed, 32, 64, scale=0.05, dtype=dtype)
        bias = gen(seed + 500, 32, scale=0.1, dtype=dtype)
        c = cfg(kind, symmetric, strategy, group)
        awq_scale = None
        wq = w
        if with_awq:
            awq_scale = (0.5 + torch.rand(1, 64, generator=torch.Generator().manual_seed(seed))).to(dtype)
            wq = w * awq_scale                          # what apply_scale leaves in the module (awq.py:108-118)
        mn, mx = get_weight_min_max_by_granularity(wq, c)
        s, z = calculate_scale_offset(mx, mn, symmetric, kind)
        qm = types.SimpleNamespace(weight=torch.nn.Parameter(wq.clone(), requires_grad=False),
                                   bias=torch.nn.Parameter(bias.clone(), requires_grad=False), wts_type=kind,
                                   group_size=group, scale_w=s, offset_w=z, scale=None)
        dep = NpuWeightQuantizedLinear(qm)
        deploy.append({"dtype": str(dtype), "kind": kind, "symmetric": symmetric, "strategy": strategy,
                       "group": group or 0, "weight": wq, "bias": bias, "scale_w": s, "offset_w": z,
                       "buffers": {k: v.clone() for k, v in dep.state_dict().items()},
                       "dep_bias": dep.bias.clone(), "dep_group_size": dep.group_size})
    out["weight_only_deploy"] = deploy

    path = os.path.join(HERE, "ref_callers.pt")
    torch.save(out, path)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
