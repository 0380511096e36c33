"""GPTQ inner-block kernel bit for bit against the oracle's restatement of
amct_pytorch/quantize_op/gptq_module.py:128-151, and the whole weight optimisation by tolerance (its
factorisations and GEMMs are library calls on both sides)."""
import pytest
import torch

from amct_amd.quantize_op import gptq
from oracle import gptq as og
from oracle import int_quant as iq
from util import assert_bits_equal

pytestmark = pytest.mark.gpu


def _hinv(count, seed):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(count, 3 * count, generator=g)
    h = a @ a.t() / (3 * count) + 0.05 * torch.eye(count)
    c = torch.linalg.cholesky(torch.cholesky_inverse(torch.linalg.cholesky(h)), upper=True)
    return c.contiguous()


@pytest.mark.parametrize("kind,sym", [('int4', False), ('int4', True), ('int8', False), ('int8', True)])
@pytest.mark.parametrize("n,count,strategy", [(64, 128, 'channel'), (37, 40, 'channel'), (5, 1, 'channel'),
                                              (130, 128, 'group'), (16, 70, 'tensor'), (4100, 128, 'channel')])
def test_gptq_block_bit_exact(dev, kind, sym, n, count, strategy):
    g = torch.Generator().manual_seed(n * 7 + count)
    columns = count + 24                                            # the block sits inside a wider matrix
    w = (torch.randn(n, columns, generator=g) * 0.05).float()
    hinv_full = _hinv(columns, count)
    i1, i2 = 8, 8 + count
    bits = int(kind[3:])
    if strategy == 'group':
        G = 4
        wg = (torch.randn(n, G * 32, generator=g) * 0.05).float()
        s, z = iq.weight_scale_offset(wg, 'group', sym, kind, 32)
        s, z = s.reshape(n, G), (None if z is None else z.reshape(n, G))
        gidx = torch.randint(0, G, (count,), generator=g, dtype=torch.int32)
        scale_cols = [s[:, int(j)].unsqueeze(-1) for j in gidx]
        offset_cols = None if z is None else [z[:, int(j)].unsqueeze(-1) for j in gidx]
    else:
        s, z = iq.weight_scale_offset(w, strategy, sym, kind)
        gidx = torch.zeros(count, dtype=torch.int32)
        scale_cols = [s.reshape(-1, 1)] * count
        offset_cols = None if z is None else [z.reshape(-1, 1)] * count
    want_w = w.clone()
    _, want_e = og.block_loop(want_w[:, i1:i2], hinv_full[i1:i2, i1:i2], kind, scale_cols, offset_cols)
    dw = w.clone().to(dev)
    got_e = gptq.gptq_block(dw, i1, i2, hinv_full.to(dev), s.reshape(-1).contiguous().to(dev),
                            None if z is None else z.reshape(-1).to(torch.int32).contiguous().to(dev), gidx.to(dev),
                            -(1 << (bits - 1)), (1 << (bits - 1)) - 1)
    assert_bits_equal(got_e.cpu(), want_e, "err block")
    assert_bits_equal(dw.cpu(), want_w, "weight block (columns outside the block untouched)")


@pytest.mark.parametrize("n,count", [(70, 128), (33, 40)])
def test_gptq_block_full_matrix_hinv(dev, n, count):
    """A step only touches the columns at and behind its own (gptq_module.py:141): with an inverse-Hessian block
    that is NOT triangular the entries in front of the diagonal must be ignored, in both kernels (full 128-column
    blocks and shorter ones)."""
    g = torch.Generator().manual_seed(count)
    w = (torch.randn(n, count, generator=g) * 0.05).float()
    hinv = _hinv(count, 3) + 0.01 * torch.randn(count, count, generator=g)       # dense, diagonal still dominant
    s, z = iq.weight_scale_offset(w, 'channel', False, 'int4')
    gidx = torch.zeros(count, dtype=torch.int32)
    want_w = w.clone()
    _, want_e = og.block_loop(want_w, hinv, 'int4', [s.reshape(-1, 1)] * count, [z.reshape(-1, 1)] * count)
    dw = w.clone().to(dev)
    got_e = gptq.gptq_block(dw, 0, count, hinv.to(dev), s.reshape(-1).contiguous().to(dev),
                            z.reshape(-1).to(torch.int32).contiguous().to(dev), gidx.to(dev), -8, 7)
    assert_bits_equal(got_e.cpu(), want_e, "err block")
    assert_bits_equal(dw.cpu(), want_w, "weight block")


@pytest.mark.parametrize("strategy,group,sym", [('channel', None, True), ('group', 32, False)])
def test_gptq_whole_routine(dev, strategy, group, sym):
    """End to end.  The two sides factorise and multiply with different libraries, so a weight that sits next
    to a rounding boundary may land on the neighbouring code: nearly all entries agree closely, none differs
    by more than one quantisation step, and the layer output error of the two results is the same."""
    torch.manual_seed(3)
    n, k, t = 48, 256, 512
    w = (torch.randn(n, k) * 0.05).to(torch.bfloat16)
    x = torch.randn(t, k) * (1 + 3 * (torch.arange(k) % 17 == 0))
    x[:, 5] = 0                                                     # a dead input channel
    hess, ns = og.update_hessian(None, 0, x[:256], k)
    hess, ns = og.update_hessian(hess, ns, x[256:].reshape(2, 128, k), k)
    dh, dn = gptq.update_hessian(None, 0, x[:256].to(dev), k)
    dh, dn = gptq.update_hessian(dh, dn, x[256:].reshape(2, 128, k).to(dev), k)
    assert dn == ns
    torch.testing.assert_close(dh.cpu(), hess, rtol=1e-4, atol=1e-4)
    cfg = {'weights_cfg': {'quant_type': 'int4', 'symmetric': sym, 'strategy': strategy}}
    if group:
        cfg['weights_cfg']['group_size'] = group
    want, ws, wz = og.optimize_weight(w, hess, 'int4', strategy, sym, group)
    got, gs, gz = gptq.get_opt_weight_and_quant_factor(w.to(dev), hess.to(dev), cfg)
    assert got.dtype == w.dtype
    assert_bits_equal(gs.cpu().reshape(ws.shape), ws, "scale_w")
    diff = (got.cpu().float() - want.float()).abs()
    step = ws.reshape(n, -1).float().amax(dim=1, keepdim=True)
    assert (diff <= 1.01 * step + 1e-6).all()
    assert (diff <= 1e-3 * step).float().mean() > 0.97
    ref_err = ((x @ w.float().t()) - (x @ want.float().t())).pow(2).mean()
    got_err = ((x @ w.float().t()) - (x @ got.cpu().float().t())).pow(2).mean()
    assert abs(float(got_err) - float(ref_err)) <= 0.05 * float(ref_err)
    # and it is an improvement over plain rounding, which is the point of the algorithm
    plain = iq.fake_quant(w, 'int4', ws, wz, group)
    plain_err = ((x @ w.float().t()) - (x @ plain.float().t())).pow(2).mean()
    assert float(got_err) < float(plain_err)
