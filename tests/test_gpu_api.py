"""The reference-shaped Python API (function, module and operator level) on the GPU against the
oracle's restatement of the reference."""
import types

import pytest
import torch

from amct_amd import ops, torch_hip
from amct_amd.algorithm import awq
from amct_amd.deploy_op import HipQuantizationLinear, HipWeightQuantizedLinear
from amct_amd.quantize_op import utils as qutils
from amct_amd.utils import data_utils, quant_util
from oracle import deploy as od
from oracle import int_quant as iq
from util import assert_bits_equal, check_weight_only

pytestmark = pytest.mark.gpu


def cfg(kind, sym, strategy, group=None):
    w = {'quant_type': kind, 'symmetric': sym, 'strategy': strategy}
    if group:
        w['group_size'] = group
    return {'weights_cfg': w}


@pytest.mark.parametrize("kind", ['int8', 'int4'])
@pytest.mark.parametrize("sym", [True, False])
@pytest.mark.parametrize("strategy,group", [('tensor', None), ('channel', None), ('group', 32)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_weight_only_matrix(dev, kind, sym, strategy, group, dtype):
    """The reference's weight-only test matrix (tests/amct_pytorch/test_minmax.py:56-381):
    {int8,int4} x {tensor,channel,group32} x {sym,asym}, here with numeric checks."""
    torch.manual_seed(0)
    w = torch.randn(64, 80 if strategy == 'group' else 64).to(dtype)
    c = cfg(kind, sym, strategy, group)
    wd = w.to(dev)
    mn, mx = qutils.get_weight_min_max_by_granularity(wd, c)
    omn, omx = iq.weight_min_max(w, strategy, group)
    assert mn.shape == omn.shape and mn.dtype == w.dtype
    assert torch.equal(mn.cpu(), omn) and torch.equal(mx.cpu(), omx)
    s, z = qutils.calculate_scale_offset(mx, mn, sym, kind)
    os_, oz = iq.scale_offset(omx, omn, sym, kind)
    assert s.shape == os_.shape and s.dtype == torch.float32
    assert_bits_equal(s, os_, "scale")
    assert (z is None) == sym                      # offset_w is None iff symmetric
    if not sym:
        assert z.dtype == torch.int32
        assert_bits_equal(z, oz, "offset")
    dq = quant_util.quant_dequant_weight(wd, c, s, z)
    assert_bits_equal(dq, iq.fake_quant(w, kind, os_, oz, group), "quant_dequant_weight")
    codes = quant_util.quant_weight(wd, kind, s, z, group)
    oc = iq.quant_codes(w, kind, os_, oz, group)
    assert codes.dtype == (torch.int8 if kind == 'int8' else torch.int32)      # test_quantize.py:84,101
    assert_bits_equal(codes, oc, "quant_weight")


def test_calculate_scale_offset_raises(dev):
    with pytest.raises(RuntimeError, match="Param scale has invalid value inf, nan or zeros!"):
        qutils.calculate_scale_offset(torch.tensor([[float('inf')]], device=dev), torch.tensor([[0.0]], device=dev), True, 'int8')


def test_convert_helpers(dev):
    t = (torch.randn(7, 33) * 100).to(torch.bfloat16)
    assert_bits_equal(quant_util.convert_dtype(t.to(dev), 'int8'), iq.to_codes(t, 'int8'), "convert_dtype int8")
    assert_bits_equal(quant_util.convert_dtype(t.to(dev), 'int4'), iq.to_codes(t, 'int4'), "convert_dtype int4")
    want = torch.clamp(torch.round(t), -8, 7)
    assert_bits_equal(data_utils.convert_precision(t.to(dev), 'int4'), want, "convert_precision")
    cs = (0.5 + torch.rand(1, 33)).to(torch.bfloat16)
    assert_bits_equal(quant_util.apply_smooth_weight(cs.to(dev), t.to(dev)), iq.smooth_weight(cs, t), "smooth")
    assert_bits_equal(quant_util.apply_awq_quantize_weight(t.to(dev), cs.to(dev), 32), iq.awq_weight(t, cs), "awq div")


def test_gptq_column_calls(dev):
    """The call pattern of amct_pytorch/quantize_op/gptq_module.py:136-148: one [N,1] column at a time."""
    torch.manual_seed(1)
    w = torch.randn(48, 96)
    for strategy, group in (('channel', None), ('group', 32), ('tensor', None)):
        c = cfg('int4', False, strategy, group)
        s, z = iq.weight_scale_offset(w, strategy, False, 'int4', group)
        for col in (0, 37, 95):
            x = w[:, col].reshape(-1, 1)
            if group:
                sc, zc = s[:, col // group], z[:, col // group]          # [N,1]
                sc, zc = sc.unsqueeze(-1), zc.unsqueeze(-1)
                sc, zc = s[:, col // group].unsqueeze(-1), z[:, col // group].unsqueeze(-1)
            else:
                sc, zc = s, z
            want = iq.fake_quant(x, 'int4', sc, zc, group)
            got = quant_util.quant_dequant_weight(x.to(dev), c, sc.to(dev), zc.to(dev))
            assert_bits_equal(got, want, "%s col %d" % (strategy, col))


@pytest.mark.parametrize("strategy,group,sym", [('group', 32, False), ('channel', None, True), ('tensor', None, False),
                                                ('group', 48, False)])
def test_awq_process_weights(dev, strategy, group, sym):
    torch.manual_seed(2)
    c = cfg('int4', sym, strategy, group)
    layers = [torch.nn.Linear(96, 40, bias=False).to(torch.bfloat16) for _ in range(2)]
    scale_awq = (0.5 + torch.rand(1, 96)).to(torch.bfloat16)
    want = [iq.awq_grid_step(l.weight.data, scale_awq, 'int4', strategy, sym, group)[0] for l in layers]
    dl = [torch.nn.Linear(96, 40, bias=False).to(torch.bfloat16).to(dev) for _ in range(2)]
    for a, b in zip(dl, layers):
        a.weight.data.copy_(b.weight.data)
    awq.process_weights_for_layers(dl, scale_awq.to(dev), c)
    for a, w_ in zip(dl, want):
        assert_bits_equal(a.weight.data, w_, "awq grid step %s" % strategy)
    # the staged functions on their own
    w = layers[0].weight.data
    s, z = iq.weight_scale_offset(w, strategy, sym, 'int4', group)
    if group is None or 96 % group == 0:
        t = iq.group_view(w, group) / s if group else w / s
        if z is not None:
            t = t + z
        want_q = iq.ungroup(t, w.shape).to(w.dtype)
        got = awq.do_quant(w.to(dev), s.to(dev), None if z is None else z.to(dev), strategy, group)
        assert_bits_equal(got, want_q, "do_quant")


def module_forward_check(got, x, buf, N, K, g, scale_factor, kind):
    """A weight-only module's forward (any leading dims) against the exact anchor, with the bound of the reading the
    library reports for the flattened call."""
    rows = x.numel() // K
    query = ops.gemm_w4a16_weight_rounded if kind == 'int4' else ops.gemm_w8a16_weight_rounded
    check_weight_only(got.reshape(rows, N), x.reshape(rows, K), buf['codes_nk'].reshape(N, K), buf['scale_w'].t(),
                      None if buf['offset_w'] is None else buf['offset_w'].t().float(), g, buf['bias'], scale_factor,
                      query(rows, N, K, g, x.dtype), what=kind, exact_rel=2e-5)


def quant_module(weight, bias, **kw):
    m = types.SimpleNamespace(weight=torch.nn.Parameter(weight, requires_grad=False), bias=bias, act_type='int8',
                              wts_type='int8', scale_w=None, offset_w=None, scale_d=None, offset_d=None, scale=None,
                              group_size=None)
    for k, v in kw.items():
        setattr(m, k, v)
    return m


@pytest.mark.parametrize("mode", ['tensor_sym', 'tensor_asym', 'token_sym', 'tensor_sym_smooth'])
@pytest.mark.parametrize("with_bias", [False, True])
def test_w8a8_module(dev, mode, with_bias):
    torch.manual_seed(3)
    N, K, M = 96, 128, 24
    w = (torch.randn(N, K) * 0.05).to(torch.bfloat16)
    b = torch.randn(N).to(torch.bfloat16) if with_bias else None
    x = torch.randn(2, M, K).to(torch.bfloat16)
    smooth = (0.5 + torch.rand(1, K)).to(torch.bfloat16) if mode.endswith('smooth') else None
    ws = iq.smooth_weight(smooth, w) if smooth is not None else w
    scale_w, _ = iq.weight_scale_offset(ws, 'channel', True, 'int8')
    xs = x / smooth if smooth is not None else x
    if mode.startswith('tensor'):
        sym = 'asym' not in mode
        scale_d, offset_d = iq.scale_offset(xs.max().reshape(-1), xs.min().reshape(-1), sym, 'int8')
    else:
        mn, mx = iq.token_min_max(xs)
        scale_d, offset_d = iq.scale_offset(mx, mn, True, 'int8')
        scale_d = scale_d.reshape(M, 1)
    buf = od.w8a8_buffers(w, b, scale_w, scale_d, offset_d, smooth)
    want = od.w8a8_forward(buf, x)
    qm = quant_module(w.to(dev), None if b is None else torch.nn.Parameter(b.to(dev), requires_grad=False),
                      scale_w=scale_w.to(dev), scale_d=scale_d.to(dev),
                      offset_d=None if offset_d is None else offset_d.to(dev),
                      scale=None if smooth is None else smooth.to(dev))
    mod = HipQuantizationLinear(qm)
    assert_bits_equal(mod.quantized_weight, buf['quantized_weight'], "quantized_weight")
    assert mod.quantized_weight.shape == (K, N) and mod.quantized_weight.dtype == torch.int8
    assert_bits_equal(mod.act_scale, buf['act_scale'], "act_scale")
    assert_bits_equal(mod.deq_scale, buf['deq_scale'], "deq_scale")
    if buf['bias'] is None:
        assert mod.bias is None
    else:
        assert_bits_equal(mod.bias, buf['bias'], "bias")
    got = mod(x.to(dev))
    assert got.shape == (2, M, N) and got.dtype == torch.bfloat16
    assert_bits_equal(got, want, "forward")
    keys = set(mod.state_dict().keys())
    assert {'act_scale', 'act_offset', 'quantized_weight', 'deq_scale'} <= keys


def test_w8a8_offset_bias_at_k4096_is_the_exact_integer(dev):
    """With an activation offset the module folds -(offset_d @ Wq) into an int32 bias.  The reference evaluates that
    sum with an fp32 matmul (npu_quantization_linear.py:56-59), which stops being exact once
    K * |offset| * 127 > 2^24; the module registers the exact integer.  At K = 4096 the two differ by at most the
    rounding of an fp32 sum of that magnitude, and the module's value equals the int64 sum."""
    torch.manual_seed(21)
    N, K = 64, 4096
    w = (torch.randn(N, K) * 0.05).to(torch.bfloat16)
    scale_w, _ = iq.weight_scale_offset(w, 'channel', True, 'int8')
    scale_d = torch.tensor([0.037])
    offset_d = torch.tensor([-77], dtype=torch.int32)
    buf = od.w8a8_buffers(w, None, scale_w, scale_d, offset_d, None)
    qm = quant_module(w.to(dev), None, scale_w=scale_w.to(dev), scale_d=scale_d.to(dev), offset_d=offset_d.to(dev))
    mod = HipQuantizationLinear(qm)
    exact = 77 * buf['quantized_weight'].to(torch.int64).sum(dim=0)       # -(offset * sum_k Wq[k, n])
    assert mod.bias.dtype == torch.int32 and torch.equal(mod.bias.cpu().to(torch.int64), exact)
    # the reference's fp32 evaluation: within one rounding per partial sum of the exact value
    ref_bias = buf['bias'].to(torch.int64)
    bound = exact.abs().max().item() * 2.0 ** -23 * 8 + 1
    assert (ref_bias - exact).abs().max().item() <= bound
    assert 'quantized_weight' in mod.state_dict() and '_dyn_scale_w' not in mod.state_dict()


def test_w8a8_module_dynamic(dev):
    torch.manual_seed(4)
    N, K, M = 64, 256, 40
    w = (torch.randn(N, K) * 0.05).to(torch.bfloat16)
    x = torch.randn(M, K).to(torch.bfloat16)
    scale_w, _ = iq.weight_scale_offset(w, 'channel', True, 'int8')
    qm = quant_module(w.to(dev), None, scale_w=scale_w.to(dev), scale_d=torch.ones(1, device=dev))
    mod = HipQuantizationLinear(qm, dynamic_act=True)
    got = mod(x.to(dev))
    xq, s_tok = iq.dynamic_token_quant(x)
    wq = iq.to_codes(w / scale_w, 'int8')
    want = od.quant_matmul(xq, wq.t(), scale_w.reshape(-1), s_tok, None, torch.bfloat16)
    assert_bits_equal(got, want, "dynamic forward")


@pytest.mark.parametrize("group,sym,with_awq", [(32, False, True), (128, False, False), (None, True, False), (64, True, True)])
def test_w4a16_module(dev, group, sym, with_awq):
    torch.manual_seed(5)
    N, K, M = 64, 256, 9
    w = (torch.randn(N, K) * 0.05).to(torch.bfloat16)
    b = torch.randn(N).to(torch.bfloat16)
    x = torch.randn(3, M, K).to(torch.bfloat16)
    awq_scale = (0.5 + torch.rand(1, K)).to(torch.bfloat16) if with_awq else None
    wa = iq.awq_weight(w, awq_scale) if with_awq else w
    strategy = 'group' if group else 'channel'
    scale_w, offset_w = iq.weight_scale_offset(wa, strategy, sym, 'int4', group)
    buf = od.w4a16_buffers(w, b, scale_w, offset_w, 'int4', group, awq_scale)
    qm = quant_module(w.to(dev), torch.nn.Parameter(b.to(dev), requires_grad=False), wts_type='int4',
                      scale_w=scale_w.to(dev), offset_w=None if offset_w is None else offset_w.to(dev),
                      scale=None if awq_scale is None else awq_scale.to(dev), group_size=group)
    mod = HipWeightQuantizedLinear(qm)
    # codes and factors agree with the reference's buffers after conversion to its layout
    words, sw, ow = mod.reference_layout()
    assert_bits_equal(words, buf['quantized_weight'], "int4 words [K,N/8]")
    assert words.dtype == torch.int32 and words.shape == (K, N // 8)
    assert_bits_equal(sw, buf['scale_w'], "scale_w [K/g,N]")
    if buf['offset_w'] is not None:
        assert_bits_equal(ow, buf['offset_w'], "offset_w [K/g,N]")
    assert mod.bias.dtype == torch.float32
    got = mod(x.to(dev))
    g = group or K
    assert got.shape == (3, M, N)
    module_forward_check(got, x, buf, N, K, g, awq_scale, 'int4')
    # operator-level drop-in with the reference's operand layouts gives the same result
    xs = x.to(dev) if awq_scale is None else torch.mul(x.to(dev), awq_scale.to(dev))
    out2 = torch_hip.npu_weight_quant_batchmatmul(xs.reshape(-1, K), words, sw, antiquant_offset=ow if not sym else None,
                                                  bias=mod.bias, antiquant_group_size=group or 0)
    assert_bits_equal(out2.reshape(3, M, N), got.cpu(), "operator vs module")


@pytest.mark.parametrize("kind", ['int8', 'int4'])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("strategy,group,sym,with_awq", [('group', 32, False, False), ('channel', None, True, False),
                                                         ('tensor', None, False, False), ('group', 64, True, True),
                                                         ('channel', None, False, True)])
@pytest.mark.parametrize("M", [9, 70])
def test_weight_only_module_matrix(dev, kind, dtype, strategy, group, sym, with_awq, M):
    """The weight-only half of the reference's deploy matrix (tests/amct_pytorch/test_minmax.py:56-381 followed by
    convert): int8 and int4 weights, bf16 and fp16 models, every granularity; buffers against the restatement of
    amct_pytorch/deploy_op/weight_npu_quant_module.py:29-100, the forward against the fp64 anchor."""
    torch.manual_seed(15)
    N, K = 72, 256
    w = (torch.randn(N, K) * 0.05).to(dtype)
    b = torch.randn(N).to(dtype)
    x = torch.randn(2, M, K).to(dtype)
    awq_scale = (0.5 + torch.rand(1, K)).to(dtype) if with_awq else None
    wa = iq.awq_weight(w, awq_scale) if with_awq else w
    scale_w, offset_w = iq.weight_scale_offset(wa, strategy, sym, kind, group)
    buf = od.w4a16_buffers(w, b, scale_w, offset_w, kind, group, awq_scale)
    qm = quant_module(w.to(dev), torch.nn.Parameter(b.to(dev), requires_grad=False), wts_type=kind,
                      scale_w=scale_w.to(dev), offset_w=None if offset_w is None else offset_w.to(dev),
                      scale=None if awq_scale is None else awq_scale.to(dev), group_size=group)
    mod = HipWeightQuantizedLinear(qm)
    qw, sw, ow = mod.reference_layout()
    assert_bits_equal(qw, buf['quantized_weight'], "quantized_weight in the reference's layout")
    assert qw.dtype == (torch.int8 if kind == 'int8' else torch.int32)
    assert_bits_equal(sw, buf['scale_w'], "scale_w [K/g,N]")
    if buf['offset_w'] is None:
        assert ow is None
    else:
        assert_bits_equal(ow, buf['offset_w'], "offset_w [K/g,N]")
    assert mod.group_size == buf['group_size']
    got = mod(x.to(dev))
    assert got.shape == (2, M, N) and got.dtype == dtype
    g = group or K
    module_forward_check(got, x, buf, N, K, g, awq_scale, kind)
    # operator-level drop-in with the reference's operand layouts: same bits as the module
    xs = x.to(dev) if awq_scale is None else torch.mul(x.to(dev), awq_scale.to(dev))
    for _ in range(2):                                               # the second call takes the cached layouts
        out2 = torch_hip.npu_weight_quant_batchmatmul(xs.reshape(-1, K), qw, sw, antiquant_offset=ow, bias=mod.bias,
                                                      antiquant_group_size=group or 0)
        assert_bits_equal(out2.reshape(2, M, N), got.cpu(), "operator vs module")
    keys = set(mod.state_dict().keys())
    assert {'quantized_weight', 'scale_w', 'bias'} <= keys and ('offset_w' in keys) == (not sym or kind == 'int4')


def test_weight_only_layout_cache_follows_in_place_updates(dev):
    """The operator-level path caches the converted weight per (tensor, version): an in-place write to the buffer
    must be seen by the next call."""
    torch.manual_seed(16)
    M, K, N = 8, 128, 32
    x = torch.randn(M, K).to(torch.bfloat16).to(dev)
    wq = torch.randint(-128, 128, (K, N), dtype=torch.int8).to(dev)
    sw = (torch.rand(1, N) * 0.01 + 0.001).to(torch.bfloat16).to(dev)
    a = torch_hip.npu_weight_quant_batchmatmul(x, wq, sw)
    wq.zero_()
    b = torch_hip.npu_weight_quant_batchmatmul(x, wq, sw)
    assert float(a.float().abs().max()) > 0 and float(b.float().abs().max()) == 0.0


def test_operator_level_w8a8(dev):
    torch.manual_seed(6)
    M, K, N = 20, 192, 72
    x = torch.randn(M, K).to(torch.bfloat16)
    sc = torch.tensor([31.0], dtype=torch.bfloat16)
    zp = torch.tensor([3.0], dtype=torch.bfloat16)
    xq = torch_hip.npu_quantize(x.to(dev), sc.to(dev), zp.to(dev), dtype=torch.int8, axis=-1, div_mode=False)
    assert_bits_equal(xq, iq.static_quantize(x, sc, zp), "npu_quantize")
    wq = torch.randint(-128, 128, (N, K), dtype=torch.int8)
    scale = torch.rand(N) * 0.01
    out = torch_hip.npu_quant_matmul(xq, wq.to(dev).t(), scale=scale.to(dev), pertoken_scale=None, bias=None,
                                     output_dtype=torch.bfloat16)
    assert_bits_equal(out, od.quant_matmul(xq.cpu(), wq.t(), scale, None, None, torch.bfloat16), "npu_quant_matmul")
    codes = torch.randint(-8, 8, (K, N), dtype=torch.int32)
    words = torch_hip.npu_convert_weight_to_int4pack(codes.to(dev))
    assert_bits_equal(words, od.pack_int4_words(codes), "int4pack")
    assert torch_hip.npu.is_available()


def test_dispatcher_operators(dev):
    """The same operators through torch.ops.amct_hip.*: identical results to the function-level entry points;
    a CPU tensor finds no kernel (there is no host implementation)."""
    torch.manual_seed(8)
    M, K, N, g = 12, 256, 64, 128
    x = torch.randn(M, K).to(torch.bfloat16)
    sc = torch.tensor([25.0], dtype=torch.bfloat16)
    xq = torch.ops.amct_hip.quantize(x.to(dev), sc.to(dev), None, -1, False)
    assert_bits_equal(xq, torch_hip.npu_quantize(x.to(dev), sc.to(dev)), "quantize")
    wq = torch.randint(-128, 128, (N, K), dtype=torch.int8)
    scale = (torch.rand(N) * 0.01).to(dev)
    tok = (torch.rand(M) * 0.1 + 0.01).to(dev)
    a = torch.ops.amct_hip.quant_matmul(xq, wq.to(dev).t(), scale, tok, None, torch.float16)
    b = torch_hip.npu_quant_matmul(xq, wq.to(dev).t(), scale=scale, pertoken_scale=tok, output_dtype=torch.float16)
    assert_bits_equal(a, b, "quant_matmul")
    codes = torch.randint(-8, 8, (K, N), dtype=torch.int32)
    words = torch.ops.amct_hip.convert_weight_to_int4pack(codes.to(dev))
    assert_bits_equal(words, od.pack_int4_words(codes), "int4pack")
    sw = (torch.rand(K // g, N) * 0.01 + 0.001).to(torch.bfloat16).to(dev)
    ow = torch.randint(-7, 8, (K // g, N)).to(torch.bfloat16).to(dev)
    c = torch.ops.amct_hip.weight_quant_batchmatmul(x.to(dev), words, sw, ow, None, g)
    d = torch_hip.npu_weight_quant_batchmatmul(x.to(dev), words, sw, antiquant_offset=ow, antiquant_group_size=g)
    assert_bits_equal(c, d, "weight_quant_batchmatmul")
    with pytest.raises(NotImplementedError):
        torch.ops.amct_hip.convert_weight_to_int4pack(codes)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_npu_quantize_div_mode(dev, dtype):
    """npu_quantize(div_mode=True), the operator's default mode (tests/amct_pytorch/mock_torch_npu.py:69-76: input / scales
    + zero_points): one scale per tensor or per token, with and without integer zero-points, leading batch dims; the
    codes are those of the weight quantiser's division (oracle.int_quant.quant_codes: fp32 x / s + z, round half even,
    saturate), bit for bit, and differ from the reciprocal-multiply mode only where that mode's rounded reciprocal moves
    a value across a rounding boundary."""
    g = torch.Generator().manual_seed(91)
    x = (torch.randn(2, 9, 192, generator=g) * 40).to(dtype)
    x[0, 0, :4] = torch.tensor([1e4, -1e4, 0.5 * 0.37, -0.0]).to(dtype)          # saturation both ways
    s1 = torch.tensor([0.37], dtype=dtype)
    st = (0.2 + torch.rand(9, generator=g)).to(dtype)
    zt = torch.randint(-20, 21, (9,), generator=g).to(dtype)
    for scales, zp, axis in ((s1, None, -1), (s1, torch.tensor([3.0]).to(dtype), -1), (st, None, -2), (st, zt, -2)):
        got = torch_hip.npu_quantize(x.to(dev), scales.to(dev), None if zp is None else zp.to(dev), torch.int8, axis, True)
        assert got.dtype == torch.int8 and got.shape == x.shape
        sc = scales.float().reshape(-1)
        z = None if zp is None else zp.float().round().to(torch.int32).reshape(-1)
        if sc.numel() == 1:
            want = iq.quant_codes(x.reshape(-1, 192), 'int8', sc.reshape(1, 1), None if z is None else z.reshape(1, 1))
        else:
            want = iq.quant_codes(x.reshape(-1, 192), 'int8', sc.repeat(2).reshape(-1, 1), None if z is None else z.repeat(2).reshape(-1, 1))
        assert torch.equal(got.cpu().reshape(-1, 192), want.to(torch.int8)), (axis, zp is not None)
    with pytest.raises(RuntimeError, match="integer zero_points"):
        torch_hip.npu_quantize(x.to(dev), s1.to(dev), torch.tensor([0.5]).to(dev), torch.int8, -1, True)
    with pytest.raises(RuntimeError, match="one scale per tensor or one per token"):
        torch_hip.npu_quantize(x.to(dev), torch.ones(5, dtype=dtype).to(dev), None, torch.int8, -2, True)


class _TwoLinears(torch.nn.Module):
    """Two linears on the same input, as the q/k/v projections of a block share theirs."""

    def __init__(self, k, n):
        super().__init__()
        self.a = torch.nn.Linear(k, n, bias=False)
        self.b = torch.nn.Linear(k, n, bias=False)

    def forward(self, x):
        return torch.cat([self.a(x), self.b(x)], dim=-1)


@pytest.mark.parametrize("strategy,group,sym", [('group', 32, False), ('channel', None, True)])
def test_awq_search_scale_on_device(dev, strategy, group, sym):
    """The scale search with the state resident on the device against the CPU restatement: same grid point
    chosen, the same scale up to the device's pow (not bit-identical to the host's), losses within 2 %, and
    the layers' weights are the untouched original tensors afterwards."""
    torch.manual_seed(11)
    T, K, N, grids = 64, 128, 48, 8
    c = cfg('int4', sym, strategy, group)
    c['algorithm'] = {'awq': {'grids_num': grids}}
    x = torch.randn(T, K) * (1.0 + 6.0 * (torch.arange(K) % 16 == 0))       # a few heavy input channels
    block = _TwoLinears(K, N)
    w_cpu = [block.a.weight.data.clone(), block.b.weight.data.clone()]
    want_scale, want_losses = iq.awq_search_scale(
        x, w_cpu, lambda inp, ws: torch.cat([inp @ ws[0].t(), inp @ ws[1].t()], dim=-1), grids, 'int4', strategy, sym,
        group)
    dblock = _TwoLinears(K, N).to(dev)
    dblock.a.weight.data.copy_(w_cpu[0])
    dblock.b.weight.data.copy_(w_cpu[1])
    before = [dblock.a.weight.data_ptr(), dblock.b.weight.data_ptr()]
    got = awq.search_scale(x.to(dev), [dblock.a, dblock.b], dblock, c)
    assert dblock.a.weight.data_ptr() == before[0] and dblock.b.weight.data_ptr() == before[1]
    assert_bits_equal(dblock.a.weight.data, w_cpu[0], "weight restored")
    best = min(range(grids), key=lambda i: want_losses[i])
    ranked = sorted(want_losses)
    if ranked[1] > 1.02 * ranked[0]:                                         # a clear winner on the host
        torch.testing.assert_close(got.cpu(), want_scale, rtol=2e-6, atol=0)
    assert got.shape == (1, K) and got.dtype == x.dtype
    # the search result used as the reference uses it
    xin = x.to(dev).clone()
    awq.apply_scale(got, dblock.a, xin)
    torch.testing.assert_close(xin.cpu(), x / got.cpu(), rtol=1e-6, atol=0)
    with pytest.raises(RuntimeError, match="Invalid value"):
        bad = x.clone()
        bad[0, 0] = float('nan')
        awq.search_scale(bad.to(dev), [dblock.a, dblock.b], dblock, c)
    assert best >= 0


@pytest.mark.parametrize("dt", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n", [1, 7, 8, 1000, 4099, 262144, 8 * 1024 * 1024 + 5])
def test_awq_loss_kernel(dev, dt, n):
    """mean((y - yhat)^4) in one pass against the fp64 restatement: 2e-6 relative (fp32 sum in a fixed order that
    is not torch's), identical bits on a second call, NaN for an empty tensor and for a NaN element."""
    g = torch.Generator().manual_seed(n % 1000 + 3)
    y = (3.0 * torch.randn(n, generator=g)).to(dt)
    yh = (y.float() + 0.2 * torch.randn(n, generator=g)).to(dt)
    got = ops.awq_loss(y.to(dev), yh.to(dev))
    want = iq.awq_loss(y, yh)
    assert got.dtype == torch.float32 and got.dim() == 0
    assert abs(float(got) - want) <= 2e-6 * want, (float(got), want)
    again = ops.awq_loss(y.to(dev), yh.to(dev))
    assert torch.equal(got.cpu().view(torch.int32), again.cpu().view(torch.int32))
    if n == 1000:
        bad = y.clone()
        bad[n // 2] = float('nan')
        assert torch.isnan(ops.awq_loss(bad.to(dev), yh.to(dev)))
        assert torch.isnan(ops.awq_loss(y[:0].to(dev), yh[:0].to(dev)))
        with pytest.raises(RuntimeError):
            ops.awq_loss(y.to(dev), yh[:-1].to(dev))


def test_calculate_scale_offset_without_the_synchronising_check(dev):
    mx = torch.tensor([[1.27], [float('inf')]], device=dev)
    mn = torch.tensor([[-1.0], [0.0]], device=dev)
    s, z = qutils.calculate_scale_offset(mx, mn, True, 'int8', check=False)       # no exception, no read-back
    assert z is None and s[0, 0].item() == torch.tensor(1.27).div(127).item() and torch.isinf(s[1, 0])
    with pytest.raises(RuntimeError, match="Param scale has invalid value"):
        qutils.check_scale_offset(s, None)
