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


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tokens,cols", [(256, 128), (1, 64), (63, 200), (65, 136), (1000, 520), (2048, 1024), (300, 4104), (77, 100), (130, 1099)])
def test_hessian_update_kernel(dev, dtype, tokens, cols):
    """H <- beta H + alpha X^T X (gptq_module.py:176-181) on the matrix pipe.  Small integers make every product
    and sum exact in fp32, so the first call (beta = 0, H full of NaN beforehand: it must not be read) and a second,
    accumulating call are compared bit for bit with an integer matmul; random activations are compared with the fp64
    product at the fp32 rounding of a sum of that many terms.  Ragged tokens and columns; H comes out exactly symmetric."""
    from amct_amd import ops
    g = torch.Generator().manual_seed(tokens * 31 + cols)
    xi = torch.randint(-4, 5, (tokens, cols), generator=g)
    h = torch.full((cols, cols), float('nan'), dtype=torch.float32, device=dev)
    ops.hessian_update(h, xi.to(dtype).to(dev), 0.0, 1.0)
    want = (xi.double().t() @ xi.double())
    assert_bits_equal(h, want.float() + 0.0, "first call, integers")     # (+ 0.0: a sum that starts at +0 never ends at -0)
    xj = torch.randint(-4, 5, (max(tokens // 2, 1), cols), generator=g)
    ops.hessian_update(h, xj.to(dtype).to(dev), 0.5, 2.0)            # powers of two: still exact
    want = 0.5 * want + 2.0 * (xj.double().t() @ xj.double())
    assert_bits_equal(h, want.float() + 0.0, "second call, integers")
    x = torch.randn(tokens, cols, generator=g).to(dtype)
    h0 = torch.randn(cols, cols, generator=g)
    h0 = (h0 + h0.t()).contiguous()
    hd = h0.clone().to(dev)
    beta, alpha = 0.75, 2.0 / (tokens + 7)
    ops.hessian_update(hd, x.to(dev), beta, alpha)
    ref = beta * h0.double() + alpha * (x.double().t() @ x.double())
    mag = beta * h0.double().abs() + alpha * (x.double().abs().t() @ x.double().abs())
    err = (hd.cpu().double() - ref).abs()
    assert (err <= 2.0 ** -20 * mag + 1e-30).all(), float((err / (mag + 1e-30)).max())
    assert torch.equal(hd, hd.t()), "symmetry"


def test_update_hessian_on_16_bit_activations(dev):
    """quantize_op.gptq.update_hessian with bf16 activations on the device takes the kernel; against the oracle's
    restatement of the reference (fp32 product of the scaled activations) within the rounding of the two orders of
    operations."""
    torch.manual_seed(5)
    k = 384
    x = (torch.randn(640, k) * (1 + 3 * (torch.arange(k) % 17 == 0))).to(torch.bfloat16)
    hess, ns = og.update_hessian(None, 0, x[:256], k)
    hess, ns = og.update_hessian(hess, ns, x[256:].reshape(3, 128, k), k)
    dh, dn = gptq.update_hessian(None, 0, x[:256].to(dev), k)
    dh, dn = gptq.update_hessian(dh, dn, x[256:].reshape(3, 128, k).to(dev), k)
    assert dn == ns and dh.dtype == torch.float32
    torch.testing.assert_close(dh.cpu(), hess, rtol=1e-4, atol=1e-4)
    # both are fp32 sums in different orders; against the same recurrence in fp64 the kernel is the closer one or as close
    xd = x.double()
    exact = (2 / 1) * (xd[:256].t() @ xd[:256]) * (1 / 1)            # first call: nsamples 0 -> 1
    exact = exact * (1 / 4) + (2 / 4) * (xd[256:].t() @ xd[256:])    # second call: batch of 3, nsamples 1 -> 4
    mine, theirs = (dh.cpu().double() - exact).abs().max(), (hess.double() - exact).abs().max()
    assert float(mine) <= 1.5 * float(theirs) + 1e-6, (float(mine), float(theirs))
