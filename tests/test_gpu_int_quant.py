"""Parity of the integer quantisation kernels (through the C ABI) with the CPU oracle:
codes, scales, offsets and dequantised values bit for bit."""
import pytest
import torch

from amct_amd import ops
from oracle import int_quant as iq
from util import assert_bits_equal

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def rand_w(rows, cols, dtype, seed, std=0.02):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(rows, cols, generator=g) * std
    # a few exact zeros, an all-zero row and a tiny row exercise the guards
    w[0, : min(cols, 5)] = 0
    if rows > 2:
        w[1] = 0
        w[2] = w[2] * 1e-9
    return w.to(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape,group", [((16, 96), 0), ((16, 96), 32), ((7, 80), 32), ((5, 37), 0),
                                         ((64, 4096), 0), ((64, 4096), 128), ((3, 8200), 0), ((2, 20000), 0),
                                         ((9, 1024), 512), ((33, 2048), 0), ((3, 104), 8), ((5, 272), 16), ((7, 448), 64),
                                         ((3, 768), 256), ((1, 8), 8), ((37, 4096), 128), ((5, 24), 4)])
def test_minmax(dev, dtype, shape, group):
    w = rand_w(*shape, dtype, 11)
    mn, mx = ops.minmax(w.to(dev), group)
    if group:
        omn, omx = iq.weight_min_max(w, 'group', group)
        omn, omx = omn.squeeze(-1), omx.squeeze(-1)
    else:
        omn, omx = iq.weight_min_max(w, 'channel')
        omn, omx = omn.squeeze(-1), omx.squeeze(-1)
    # value equality: when a segment holds both -0.0 and +0.0 the sign of a zero extremum depends on
    # the reduction order (also inside torch) and has no effect on the factors derived from it
    assert torch.equal(mn.cpu(), omn.float()), "min"
    assert torch.equal(mx.cpu(), omx.float()), "max"


@pytest.mark.parametrize("dtype", DTYPES)
def test_minmax_groups_nan_and_inf(dev, dtype):
    """A NaN makes both extrema of its group NaN and leaves the neighbours alone (torch.amax / amin); infinities are
    ordinary values."""
    w = rand_w(6, 512, dtype, 5)
    w[1, 130] = float('nan')
    w[2, 3] = float('inf')
    w[4, 511] = float('-inf')
    mn, mx = ops.minmax(w.to(dev), 128)
    omn, omx = iq.weight_min_max(w, 'group', 128)
    omn, omx = omn.squeeze(-1).float(), omx.squeeze(-1).float()
    assert torch.isnan(mn[1, 1]) and torch.isnan(mx[1, 1]) and int(torch.isnan(mn).sum()) == 1
    assert torch.equal(torch.nan_to_num(mn.cpu(), nan=7.0), torch.nan_to_num(omn, nan=7.0))
    assert torch.equal(torch.nan_to_num(mx.cpu(), nan=7.0), torch.nan_to_num(omx, nan=7.0))


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("sym", [True, False])
def test_scale_offset(dev, bits, sym):
    g = torch.Generator().manual_seed(3)
    n = 300000
    a = torch.randn(n, generator=g) * torch.pow(10.0, torch.rand(n, generator=g) * 16 - 8)
    b = torch.randn(n, generator=g) * torch.pow(10.0, torch.rand(n, generator=g) * 16 - 8)
    special = torch.tensor([0.0, -0.0, 1e-8, 1e-7, 1.27, 127.25, 126.75, 1e-40, 3e38, 1.0, -1.0, 255.0, -255.0])
    a = torch.cat([a, special, special, torch.zeros(13)])
    b = torch.cat([b, special, -special, special])
    mx, mn = torch.maximum(a, b), torch.minimum(a, b)
    s, z = ops.scale_offset(mx.to(dev), mn.to(dev), bits, sym)
    os_, oz = iq.scale_offset(mx, mn, sym, 'int%d' % bits, check=False)
    assert_bits_equal(s, os_, "scale")
    if sym:
        assert z is None and oz is None
    else:
        assert_bits_equal(z, oz, "offset")


def test_scale_offset_bad_count(dev):
    mx = torch.tensor([1.0, float('inf'), float('nan'), 2.0])
    mn = torch.tensor([-1.0, 0.0, 0.0, -2.0])
    bad = torch.zeros(1, dtype=torch.int32, device=dev)
    ops.scale_offset(mx.to(dev), mn.to(dev), 8, True, bad=bad)
    # symmetric: where(|max| > |min|, |max|, |min|) drops a NaN maximum, exactly as the reference does
    assert bad.item() == 1
    bad.zero_()
    ops.scale_offset(mx.to(dev), mn.to(dev), 8, False, bad=bad)
    assert bad.item() == 2


FUSED_CASES = [((16, 96), 0), ((16, 96), 32), ((64, 64), 0), ((7, 80), 32), ((5, 37), 0), ((12, 128), 128),
               ((8, 4096), 0), ((8, 4096), 128), ((4, 8192), 0), ((3, 16384), 0), ((2, 20000), 0),
               ((6, 1024), 256), ((6, 4096), 2048), ((2, 16384), 8192), ((1, 8), 0), ((130, 256), 64),
               ((5, 11008), 0), ((4, 14336), 0), ((2, 28672), 0), ((2, 40000), 0)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("sym", [True, False])
@pytest.mark.parametrize("shape,group", FUSED_CASES)
def test_fakequant_fused(dev, dtype, bits, sym, shape, group):
    kind = 'int%d' % bits
    w = rand_w(*shape, dtype, 17 + bits)
    dq, codes, s, z = ops.fakequant_int(w.to(dev), bits, sym, group=group, codes_kind=ops.CODES_I8)
    strat = 'group' if group else 'channel'
    os_, oz = iq.weight_scale_offset(w, strat, sym, kind, group or None)
    odq = iq.fake_quant(w, kind, os_, oz, group or None)
    oc = iq.quant_codes(w, kind, os_, oz, group or None)
    if group:
        oc = oc.reshape(shape[0], -1)[:, :shape[1]]
    assert_bits_equal(s.reshape(-1), os_.reshape(-1), "scale")
    if not sym:
        assert_bits_equal(z.reshape(-1), oz.reshape(-1), "offset")
    assert_bits_equal(codes, oc.to(torch.int8), "codes")
    assert_bits_equal(dq, odq, "dq")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_fakequant_int32_codes_and_variant_b(dev, dtype):
    w = rand_w(40, 512, dtype, 23)
    w[1] = w[3]                                   # no all-zero row: variant B has no guard
    _, codes, s, _ = ops.fakequant_int(w.to(dev), 8, True, want_dq=False, codes_kind=ops.CODES_I32,
                                       scope_rule=ops.SCOPE_ABSMAX, qmin=-127, qmax=127, via_src=True)
    oq, os_ = iq.absmax_quant(w)
    assert codes.dtype == torch.int32
    assert_bits_equal(codes, oq.to(torch.int32), "variant B codes")
    assert_bits_equal(s, os_.reshape(-1), "variant B scale")
    assert oq.min() >= -127


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("bits,sym,group", [(4, False, 32), (4, False, 128), (8, True, 0), (4, True, 64), (8, False, 0)])
def test_awq_path(dev, dtype, bits, sym, group):
    """via_src rounding + column scale before/after = one AWQ grid point (awq.py:30-49)."""
    kind = 'int%d' % bits
    w = rand_w(48, 512, dtype, 29, std=0.05)
    g = torch.Generator().manual_seed(31)
    cs = (0.5 + torch.rand(1, 512, generator=g)).to(dtype)
    strat = 'group' if group else 'channel'
    want, os_, oz = iq.awq_grid_step(w, cs, kind, strat, sym, group or None)
    dq, _, s, z = ops.fakequant_int(w.to(dev), bits, sym, group=group, col_scale=cs.to(dev),
                                    col_mode=ops.COL_MUL_THEN_DIV, via_src=True)
    assert_bits_equal(s.reshape(-1), os_.reshape(-1), "scale")
    if not sym:
        assert_bits_equal(z.reshape(-1), oz.reshape(-1), "offset")
    assert_bits_equal(dq, want, "awq dq")


@pytest.mark.parametrize("dtype", DTYPES)
def test_col_scale_modes(dev, dtype):
    w = rand_w(24, 256, dtype, 37)
    g = torch.Generator().manual_seed(41)
    cs = (0.5 + torch.rand(1, 256, generator=g)).to(dtype)
    # smooth: W * s then per-channel int8 codes (npu_quantization_linear.py:49-53)
    ws = iq.smooth_weight(cs, w)
    os_, _ = iq.weight_scale_offset(ws, 'channel', True, 'int8')
    oc = iq.quant_codes(ws, 'int8', os_)
    _, codes, s, _ = ops.fakequant_int(w.to(dev), 8, True, want_dq=False, codes_kind=ops.CODES_I8,
                                       col_scale=cs.to(dev), col_mode=ops.COL_MUL)
    assert_bits_equal(s, os_.reshape(-1), "scale")
    assert_bits_equal(codes, oc, "codes")
    # awq deploy: W / s (weight_npu_quant_module.py:38-41)
    wd = iq.awq_weight(w, cs)
    os_, oz = iq.weight_scale_offset(wd, 'group', False, 'int4', 64)
    oc = iq.quant_codes(wd, 'int4', os_, oz, 64).reshape(24, -1)
    _, codes, s, z = ops.fakequant_int(w.to(dev), 4, False, group=64, want_dq=False, codes_kind=ops.CODES_I32,
                                       col_scale=cs.to(dev), col_mode=ops.COL_DIV)
    assert_bits_equal(codes, oc, "codes div")
    assert_bits_equal(z.reshape(-1), oz.reshape(-1), "offset div")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("group", [-1, 0, 32])
@pytest.mark.parametrize("shape", [(16, 96), (5, 37), (64, 1024)])
def test_quant_with_params(dev, dtype, group, shape):
    if group == 32 and shape[1] % 32 and shape[1] < 64:
        pass
    w = rand_w(*shape, dtype, 43)
    for kind, sym in (('int8', True), ('int4', False)):
        bits = int(kind[3:])
        strat = {-1: 'tensor', 0: 'channel', 32: 'group'}[group]
        os_, oz = iq.weight_scale_offset(w, strat, sym, kind, 32 if group == 32 else None)
        odq = iq.fake_quant(w, kind, os_, oz, 32 if group == 32 else None)
        oc = iq.quant_codes(w, kind, os_, oz, 32 if group == 32 else None)
        if group == 32:
            oc = oc.reshape(shape[0], -1)[:, :shape[1]]
        dq, codes = ops.quant_with_params(w.to(dev), os_.reshape(-1).to(dev), None if oz is None else oz.reshape(-1).to(dev),
                                          group, -(1 << (bits - 1)), (1 << (bits - 1)) - 1,
                                          codes_kind=ops.CODES_I32 if bits == 4 else ops.CODES_I8)
        assert_bits_equal(dq, odq, "dq")
        assert_bits_equal(codes, oc, "codes")


def test_awq_stages(dev):
    """do_quant and do_dequant as separate calls (awq.py:129-170)."""
    w = rand_w(32, 256, torch.bfloat16, 47, std=0.05)
    s, z = iq.weight_scale_offset(w, 'group', False, 'int4', 64)
    # stage SCALE
    t = iq.group_view(w, 64) / s
    t += z
    want = t.reshape(32, 256).to(torch.bfloat16)
    got, _ = ops.quant_with_params(w.to(dev), s.reshape(-1).to(dev), z.reshape(-1).to(dev), 64, -8, 7, stage=ops.STAGE_SCALE)
    assert_bits_equal(got, want, "do_quant")
    # stage DEQUANT on arbitrary bf16 input
    t = iq.group_view(w, 64) - z
    want = (t * s).reshape(32, 256).to(torch.bfloat16)
    got, _ = ops.quant_with_params(w.to(dev), s.reshape(-1).to(dev), z.reshape(-1).to(dev), 64, -8, 7, stage=ops.STAGE_DEQUANT)
    assert_bits_equal(got, want, "do_dequant")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_exhaustive_16bit_inputs(dev, dtype):
    """Every finite 16-bit pattern x 64 scales x {sym, asym} x {int4,int8} x {plain, via-src}."""
    bits16 = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    x = bits16.view(dtype)
    x = x[torch.isfinite(x.float())]
    n = x.numel()
    cols = 1024
    pad = (-n) % cols
    x = torch.cat([x, torch.zeros(pad, dtype=dtype)]).reshape(-1, cols)
    rows = x.shape[0]
    g = torch.Generator().manual_seed(53)
    scales = torch.cat([torch.pow(2.0, torch.arange(-12, 4).float()),
                        torch.pow(10.0, torch.rand(48, generator=g) * 8 - 6)])
    xd = x.to(dev)
    for si, sc in enumerate(scales.tolist()):
        s = torch.full((rows, 1), sc, dtype=torch.float32)
        for kind in ('int8', 'int4'):
            b = int(kind[3:])
            zs = [None, torch.full((rows, 1), -3 if b == 4 else -77, dtype=torch.int32)]
            for z in zs:
                for via in (False, True):
                    if via and si % 4:
                        continue
                    if via:
                        want = iq.awq_fake_quant(x, kind, s, z, 'channel')
                    else:
                        want = iq.fake_quant(x, kind, s, z)
                    dq, codes = ops.quant_with_params(xd, s.reshape(-1).to(dev), None if z is None else z.reshape(-1).to(dev),
                                                      0, -(1 << (b - 1)), (1 << (b - 1)) - 1, codes_kind=ops.CODES_I8,
                                                      via_src=via)
                    assert_bits_equal(dq, want, "dq scale=%g %s z=%s via=%s" % (sc, kind, z is not None, via))
                    if not via:
                        oc = iq.quant_codes(x, kind, s, z).to(torch.int8)
                        assert_bits_equal(codes, oc, "codes scale=%g %s" % (sc, kind))


def test_fp32_halfway_points(dev):
    """fp32 inputs that sit exactly on, just below and just above (q+0.5)*s."""
    g = torch.Generator().manual_seed(59)
    s = torch.pow(10.0, torch.rand(256, 1, generator=g) * 6 - 4)
    q = torch.arange(-130, 130).float().reshape(1, -1)
    mid = (q + 0.5) * s
    w = torch.cat([mid, torch.nextafter(mid, torch.full_like(mid, 1e30)), torch.nextafter(mid, torch.full_like(mid, -1e30))], 1)
    w = torch.nn.functional.pad(w, (0, (-w.shape[1]) % 4))
    dq, codes = ops.quant_with_params(w.to(dev), s.reshape(-1).to(dev), None, 0, -128, 127, codes_kind=ops.CODES_I8)
    assert_bits_equal(codes, iq.quant_codes(w, 'int8', s), "codes")
    assert_bits_equal(dq, iq.fake_quant(w, 'int8', s), "dq")


def test_config1_full_size(dev):
    """Benchmark configuration 1: W[4096,4096] fp32 N(0,0.02), int8 symmetric per channel."""
    from amct_amd import workloads
    w = workloads.c1_weight()
    dq, codes, s, _ = ops.fakequant_int(w.to(dev), 8, True, codes_kind=ops.CODES_I8)
    os_, _ = iq.weight_scale_offset(w, 'channel', True, 'int8')
    assert_bits_equal(s, os_.reshape(-1), "scale")
    assert_bits_equal(codes, iq.quant_codes(w, 'int8', os_), "codes")
    assert_bits_equal(dq, iq.fake_quant(w, 'int8', os_), "dq")
    assert (codes == -128).any().item()           # rows whose minimum dominates use scope 128
    # idempotence at full size
    dq2, _ = ops.quant_with_params(dq, s, None, 0, -128, 127)
    assert_bits_equal(dq2, dq.cpu(), "idempotent")


def test_fakequant_matches_exact_arithmetic_fixture(dev):
    """The committed known answers (exact fractions, one explicit rounding to binary32 per operation) through
    the C ABI: scale, offset, codes and dequantised values bit for bit, for int8 / int4, symmetric / asymmetric."""
    from util import load_int_quant_kat
    for bits, sym, w, scale, offset, codes, dq in load_int_quant_kat():
        got_dq, got_codes, got_s, got_z = ops.fakequant_int(w.to(dev), bits, sym, group=0, codes_kind=ops.CODES_I32)
        assert_bits_equal(got_s.cpu().reshape(()), scale, "scale int%d sym=%s" % (bits, sym))
        if not sym:
            assert int(got_z.cpu().reshape(())) == offset
        assert torch.equal(got_codes.cpu(), codes)
        assert_bits_equal(got_dq.cpu(), dq, "dq int%d sym=%s" % (bits, sym))
