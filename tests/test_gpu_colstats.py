"""Column statistics kernel (per input channel max / min over tokens, running update, |W| column maximum) and the
SmoothQuant calibration arithmetic built on it, against the oracle's restatement of
amct_pytorch/quantize_op/smooth_quant_module.py."""
import pytest
import torch

from amct_amd import ops
from amct_amd.quantize_op import smooth_quant_stats as sqs
from oracle import int_quant as iq
from util import assert_bits_equal

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,cols", [(1, 64), (7, 8), (300, 520), (2048, 4096), (65, 24), (33, 20), (20000, 40),
                                       (130, 1000)])
def test_col_minmax_bit_exact(dev, dtype, rows, cols):
    g = torch.Generator().manual_seed(rows * 131 + cols)
    x = (torch.randn(rows, cols, generator=g) * 3).to(dtype)
    mx, mn = ops.col_minmax(x.to(dev))
    assert_bits_equal(mx.cpu(), x.float().amax(dim=0), "col max")
    assert_bits_equal(mn.cpu(), x.float().amin(dim=0), "col min")
    am = ops.col_minmax(x.to(dev), absolute=True)
    assert_bits_equal(am.cpu(), x.float().abs().amax(dim=0), "col absmax")


def test_running_update_and_nan(dev):
    """Two batches through the running update, one of them with NaNs: a NaN batch extremum leaves the running
    value alone (torch.where(NaN > old) keeps old), a plain overwrite propagates it like torch.amax."""
    g = torch.Generator().manual_seed(5)
    w = torch.randn(16, 96, generator=g).to(torch.bfloat16)
    b1 = torch.randn(40, 96, generator=g).to(torch.bfloat16)
    b2 = torch.randn(3, 24, 96, generator=g).to(torch.bfloat16)        # rank 3: leading dims are tokens
    b1[5, 7] = float('nan')
    b2[1, 2, 50] = float('nan')
    dmax, dmin = sqs.new_channel_stats(w.to(dev))
    omax, omin = torch.full((1, 96), float('-inf'), dtype=torch.bfloat16), torch.full((1, 96), float('inf'),
                                                                                     dtype=torch.bfloat16)
    for b in (b1, b2):
        dmax, dmin = sqs.update_channel_min_max(b.to(dev), dmax, dmin)
        omax, omin = iq.channel_min_max_update(b, omax, omin)
        assert dmax.dtype == omax.dtype and dmax.shape == omax.shape
        assert_bits_equal(dmax.cpu(), omax, "running max")
        assert_bits_equal(dmin.cpu(), omin, "running min")
    mx, mn = ops.col_minmax(b1.to(dev))
    assert torch.isnan(mx[7]) and torch.isnan(mn[7]) and not torch.isnan(mx[8])
    # fp32 inputs against bf16 running values promote like torch.where
    d2max, _ = sqs.update_channel_min_max(b1.float().to(dev), *sqs.new_channel_stats(w.to(dev)))
    assert d2max.dtype == torch.float32


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_smooth_factor_and_per_tensor_params(dev, dtype):
    """The factor is two device pow results and a division; the device's pow is not bit-identical to the host's
    (each within an ulp), so 4 eps relative is allowed there.  Everything derived from the exact reductions is
    compared bit for bit on a factor of ones."""
    g = torch.Generator().manual_seed(9)
    w = (torch.randn(48, 256, generator=g) * 0.05).to(dtype)
    w[:, 11] = 0                                                          # a dead input channel: factor -> 1
    x = (torch.randn(200, 256, generator=g) * (1 + 5 * (torch.arange(256) % 32 == 0))).to(dtype)
    dmax, dmin = sqs.update_channel_min_max(x.to(dev), *sqs.new_channel_stats(w.to(dev)))
    omax, omin = iq.channel_min_max_update(x, torch.full((1, 256), float('-inf'), dtype=dtype),
                                           torch.full((1, 256), float('inf'), dtype=dtype))
    f = sqs.smooth_factor_from_stats(dmax, dmin, w.to(dev), 0.5)
    want = iq.smooth_factor(torch.max(omax.abs(), omin.abs()), w, 0.5)
    assert f.dtype == want.dtype and f.shape == want.shape
    ulp = torch.finfo(dtype).eps
    assert ((f.cpu().double() - want.double()).abs() <= 4 * ulp * want.double().abs()).all()
    assert f[0, 11] == 1
    ones = torch.ones(1, 256, dtype=dtype)
    for sym in (True, False):
        s, z = sqs.per_tensor_params(dmax, dmin, ones.to(dev), sym, 'int8')
        ws, wz = iq.scale_offset((omax / ones).max().reshape(-1), (omin / ones).min().reshape(-1), sym, 'int8')
        assert_bits_equal(s.cpu().reshape(ws.shape), ws, "scale_d")
        if not sym:
            assert torch.equal(z.cpu().reshape(wz.shape), wz)


def test_col_minmax_errors(dev):
    from amct_amd import _lib
    lib = _lib.load()
    x = torch.zeros(4, 8, device=dev)
    out = torch.zeros(8, device=dev)
    ws = torch.zeros(64, dtype=torch.uint8, device=dev)
    st = torch.cuda.current_stream(dev).cuda_stream
    need = lib.amct_col_minmax_workspace_bytes(4, 8)
    assert need == 64
    assert lib.amct_col_minmax(x.data_ptr(), out.data_ptr(), None, 4, 8, 0, 0, 0, ws.data_ptr(), 8, st) == -1
    assert lib.amct_col_minmax(x.data_ptr(), None, None, 4, 8, 0, 0, 0, ws.data_ptr(), need, st) == -1
    assert lib.amct_col_minmax(x.data_ptr(), out.data_ptr(), None, 4, 8, 0, 0, 9, ws.data_ptr(), need, st) == -1
    assert lib.amct_col_minmax(None, None, None, 0, 8, 0, 0, 0, None, 0, st) == 0
