"""The HIP path against vectors written by the reference's own CPU path (tests/golden/ref_callers.pt) and against the
exact-fraction known answers for 16-bit sources, groups and the cast-before-round variant
(tests/golden/int_quant_kat16.json).  Everything goes through the C ABI."""
import pytest
import torch

import types

from amct_amd import ops
from amct_amd.deploy_op import HipQuantizationLinear, HipWeightQuantizedLinear
from amct_amd.algorithm import awq as hawq
from amct_amd.quantize_op import gptq as hgptq
from amct_amd.quantize_op import smooth_quant_stats as hsq
from amct_amd.quantize_op.utils import calculate_scale_offset, get_weight_min_max_by_granularity
from amct_amd.utils.data_utils import convert_precision
from amct_amd.utils.quant_util import quant_dequant_weight, quant_weight
from util import assert_bits_equal, load_int_quant_kat16, load_ref_callers

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ref():
    return load_ref_callers()


def _cfg(c, algorithm=None):
    w = {'quant_type': c["kind"], 'symmetric': c["symmetric"], 'strategy': c["strategy"]}
    if c["group"]:
        w['group_size'] = c["group"]
    return {'batch_num': 1, 'weights_cfg': w, 'inputs_cfg': {'enable_quant': False}, 'algorithm': algorithm or {}}


def test_exact_fraction_fixture_16bit_group_awq(dev):
    cases = load_int_quant_kat16()
    for i, c in enumerate(cases):
        w = c["w"].to(dev)
        tag = "case {} {} int{} sym={} g={}".format(i, c["src"], c["bits"], c["symmetric"], c["group"])
        dq, codes, s, z = ops.fakequant_int(w, c["bits"], c["symmetric"], group=c["group"], codes_kind=ops.CODES_I32)
        assert_bits_equal(s.reshape(-1), c["scale"], tag + " scale")
        if not c["symmetric"]:
            assert torch.equal(z.reshape(-1).cpu(), c["offset"]), tag
        assert torch.equal(codes.cpu(), c["codes"]), tag + " codes"
        assert_bits_equal(dq, c["dq"], tag + " dq")
        adq, _, _, _ = ops.fakequant_int(w, c["bits"], c["symmetric"], group=c["group"], via_src=True)
        assert_bits_equal(adq, c["awq_dq"], tag + " awq dq")


def test_reference_elementwise_matrix(dev, ref):
    """Function level, named and called like the reference's (quantize_op/utils.py, utils/quant_util.py,
    algorithm/awq.py), on the reference's own outputs."""
    for c in ref["matrix"]:
        cfg = _cfg(c)
        w = c["w"].to(dev)
        kind, sym, strat, g = c["kind"], c["symmetric"], c["strategy"], c["group"] or None
        tag = "{} {} sym={} {}".format(c["dtype"], kind, sym, strat)
        mn, mx = get_weight_min_max_by_granularity(w, cfg)
        assert_bits_equal(mn, c["min"], tag + " min")
        assert_bits_equal(mx, c["max"], tag + " max")
        s, z = calculate_scale_offset(mx, mn, sym, kind)
        assert_bits_equal(s, c["scale"], tag + " scale")
        if sym:
            assert z is None
        else:
            assert z.dtype == torch.int32 and torch.equal(z.cpu(), c["offset"]), tag
        assert_bits_equal(quant_dequant_weight(w, cfg, s, z), c["dq"], tag + " dq")
        codes = quant_weight(w, kind, s, z, g)
        assert codes.dtype == c["codes"].dtype and tuple(codes.shape) == tuple(c["codes"].shape), tag
        assert torch.equal(codes.cpu(), c["codes"]), tag + " codes"
        t = hawq.do_quant(w.clone(), s, z, strat, g)
        t = convert_precision(t, kind)
        adq = hawq.do_dequant(t, s, z, strat, g)
        assert_bits_equal(adq, c["awq_dq"], tag + " awq dq")


class _Block(torch.nn.Module):
    def __init__(self, lin):
        super().__init__()
        self.a, self.b = lin

    def forward(self, x):
        return torch.cat([self.a(x), self.b(x)], dim=-1)


def test_reference_awq_grid_point_and_search(dev, ref):
    for c in ref["awq_search"]:
        cfg = _cfg(c, {'awq': {'grids_num': c["grids"]}})
        lin = []
        for w in c["weights"]:
            l = torch.nn.Linear(w.shape[1], w.shape[0], bias=False)
            l.weight.data = w.clone()
            lin.append(l.to(dev))
        blk = _Block(lin).to(dev)
        x = c["x"].to(dev)
        # one explicit grid point: bit for bit
        hawq.process_weights_for_layers(lin, c["grid_scale"].to(dev), cfg)
        for l, w1 in zip(lin, c["grid_weights"]):
            assert_bits_equal(l.weight.data, w1, "grid point weights")
        for l, w in zip(lin, c["weights"]):
            l.weight.data = w.clone().to(dev)
        best = hawq.search_scale(x, lin, blk, cfg)
        want = c["best_scale"]
        assert best.dtype == want.dtype and tuple(best.shape) == tuple(want.shape)
        # the candidate scale goes through pow() on the device: one unit in the last place of the dtype at most.
        # A different winning grid point would differ by far more than that in most channels.
        rel = ((best.cpu().double() - want.double()).abs() / want.double().abs()).max().item()
        assert rel <= 2.0 * torch.finfo(want.dtype).eps, rel
        for l, w in zip(lin, c["weights"]):                        # the weights are put back untouched
            assert_bits_equal(l.weight.data, w, "weights restored")


def test_reference_smoothquant_statistics(dev, ref):
    for c in ref["smoothquant"]:
        w = c["weight"].to(dev)
        dmax, dmin = hsq.new_channel_stats(w)
        for x in c["inputs"]:
            dmax, dmin = hsq.update_channel_min_max(x.to(dev), dmax, dmin)
        assert_bits_equal(dmax, c["data_max"], "data_max")
        assert_bits_equal(dmin, c["data_min"], "data_min")
        f = hsq.smooth_factor_from_stats(dmax, dmin, w, c["strength"])
        want = c["smooth"]
        assert f.dtype == want.dtype and tuple(f.shape) == tuple(want.shape)
        # pow() on the device against the host's: a few units in the last place of the 16-bit dtype
        rel = ((f.cpu().double() - want.double()).abs() / want.double().abs()).max().item()
        assert rel <= 4.0 * torch.finfo(want.dtype).eps, rel
        assert f[0, 9].item() == 1.0


def test_reference_gptq(dev, ref):
    """Cholesky factorisations and the inverse run in the device library here and in the host library in the
    reference: the factors must agree bit for bit, the optimised weight on all but a few percent of the entries,
    and nowhere by more than a few quantisation steps."""
    for idx, c in enumerate(ref["gptq"]):
        cfg = _cfg(c, {'gptq': {}})
        w = c["weight"].detach().to(dev)
        got, s, z = hgptq.get_opt_weight_and_quant_factor(w, c["hessian"].to(dev), cfg)
        assert_bits_equal(s, c["scale"].detach(), "gptq scale")
        if c["symmetric"]:
            assert z is None
        else:
            assert torch.equal(z.cpu(), c["offset"])
        want = c["opt_weight"].detach()
        assert got.dtype == want.dtype and tuple(got.shape) == tuple(want.shape)
        diff = (got.cpu().float() - want.float()).abs()
        step = float(c["scale"].detach().max())
        frac = (diff > 0.51 * step).float().mean().item()
        assert frac <= 0.05, (idx, frac)
        assert float(diff.max()) <= 4.0 * step, (idx, float(diff.max()), step)


def test_reference_weight_only_deploy_buffers(dev, ref):
    """HipWeightQuantizedLinear built from the same calibrated fields as the reference's module: its buffers,
    brought to the reference's layout, equal the registered buffers the reference wrote (the int4 word packing
    itself lives in torch_npu: the fixture holds the unpacked [K, N] int32 codes)."""
    for c in ref["weight_only_deploy"]:
        qm = types.SimpleNamespace(weight=torch.nn.Parameter(c["weight"].to(dev), requires_grad=False),
                                   bias=torch.nn.Parameter(c["bias"].to(dev), requires_grad=False),
                                   wts_type=c["kind"], group_size=c["group"] or None, scale_w=c["scale_w"].to(dev),
                                   offset_w=None if c["offset_w"] is None else c["offset_w"].to(dev), scale=None)
        mod = HipWeightQuantizedLinear(qm)
        want = c["buffers"]
        qw, sw, ow = mod.reference_layout()
        if c["kind"] == 'int4':
            qw = ops.unpack_nibbles_to_i32_kn(mod.quantized_weight)
        assert qw.dtype == want["quantized_weight"].dtype
        assert torch.equal(qw.cpu(), want["quantized_weight"])
        assert_bits_equal(sw, want["scale_w"], "scale_w")
        if "offset_w" in want:
            assert_bits_equal(ow, want["offset_w"], "offset_w")
        else:
            assert ow is None
        assert torch.equal(mod.bias.cpu(), c["dep_bias"].float())
        assert mod.group_size == c["dep_group_size"]


def test_reference_w8a8_deploy_buffers(dev, ref):
    """HipQuantizationLinear from the reference's calibrated SmoothQuant fields against the buffers its
    NpuQuantizationLinear registered."""
    for c in ref["smoothquant"]:
        qm = types.SimpleNamespace(weight=torch.nn.Parameter(c["weight"].to(dev), requires_grad=False),
                                   bias=torch.nn.Parameter(c["bias"].to(dev), requires_grad=False),
                                   act_type='int8', wts_type='int8', scale_w=c["scale_w"].to(dev), offset_w=None,
                                   scale_d=c["scale_d"].to(dev),
                                   offset_d=None if c["offset_d"] is None else c["offset_d"].to(dev),
                                   scale=c["smooth"].to(dev), group_size=None)
        mod = HipQuantizationLinear(qm)
        dep = c["deploy"]
        assert torch.equal(mod.quantized_weight.cpu(), dep["quantized_weight"])
        for k in ("act_scale", "act_offset", "deq_scale", "scale_factor"):
            assert_bits_equal(getattr(mod, k), dep[k], k)
        if "pertoken_scale" in dep:
            assert_bits_equal(mod.pertoken_scale, dep["pertoken_scale"], "pertoken_scale")
        want_b = c["deploy_bias"]
        assert mod.bias.dtype == want_b.dtype and torch.equal(mod.bias.cpu(), want_b)
