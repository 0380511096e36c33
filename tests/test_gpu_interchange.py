"""Interchange formats of the checkpoint converter on the device against the oracle's restatement of
amct_pytorch/experimental/quantization/DeepSeekV3.2/deploy.py."""
import pytest
import torch

from amct_amd import interchange as ic
from oracle import deploy as od
from oracle import int_quant as iq
from util import assert_bits_equal

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,cols,block", [(256, 512, 128), (130, 272, 128), (7, 48, 16), (5, 9, 4), (1024, 7168, 128)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_weight_dequant_bit_exact(dev, rows, cols, block, dtype):
    g = torch.Generator().manual_seed(rows + cols)
    codes = torch.randint(0, 256, (rows, cols), generator=g, dtype=torch.uint8)   # every code, NaNs included
    w = codes.view(torch.float8_e4m3fn)
    scale = torch.rand((rows + block - 1) // block, (cols + block - 1) // block, generator=g) * 0.01 + 1e-4
    old = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        got = ic.weight_dequant(w.to(dev), scale.to(dev), block)
    finally:
        torch.set_default_dtype(old)
    want = od.fp8_block_dequant(w, scale, block, dtype)
    assert got.dtype == dtype
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got.cpu()), nan)
    assert_bits_equal(torch.where(nan, torch.zeros_like(want), got.cpu()), torch.where(nan, torch.zeros_like(want), want),
                      "weight_dequant")


def test_all_fp8_codes_decode_like_torch(dev):
    codes = torch.arange(256, dtype=torch.uint8).reshape(16, 16)
    got = ic.weight_dequant(codes.view(torch.float8_e4m3fn).to(dev), torch.ones(1, 1, device=dev), 128)
    want = codes.view(torch.float8_e4m3fn).to(torch.float32)
    ok = ~torch.isnan(want)
    assert torch.equal(got.cpu().float()[ok], want[ok]) and torch.isnan(got.cpu()[~ok]).all()


@pytest.mark.parametrize("n,k", [(2, 16), (64, 256), (6, 7), (130, 4096)])
def test_pack_4bit_and_scale_widening(dev, n, k):
    g = torch.Generator().manual_seed(n * k)
    x = torch.randint(-8, 8, (n, k), generator=g, dtype=torch.int8)
    assert torch.equal(ic.pack_4bit(x.to(dev)).cpu(), od.pack_4bit(x))
    s = torch.randn(n, 1, generator=g)
    got = ic.scale_fp32_to_u64(s.to(dev))
    assert got.dtype == torch.uint64 and got.shape == (n, 1)
    assert torch.equal(got.cpu().view(torch.int64), od.scale_fp32_to_u64(s))


@pytest.mark.parametrize("bits", [8, 4])
def test_int_weight_quant(dev, bits):
    """Variant B of the weight quantisation (absmax / qmax, clamp to [-qmax, qmax]) with the converter's int4
    packaging; the assistance bias is a sum whose order belongs to the library, so it gets a tolerance."""
    g = torch.Generator().manual_seed(bits)
    w = (torch.randn(64, 512, generator=g) * 0.03).to(torch.bfloat16)
    q, s, b = ic.int_weight_quant(w.to(dev), bits)
    codes, scale = iq.absmax_quant(w, bits)
    if bits == 8:
        assert torch.equal(q.cpu(), codes.to(torch.int8)) and b is None
        assert_bits_equal(s.cpu(), scale.to(torch.float32), "scale")
    else:
        assert torch.equal(q.cpu(), od.pack_4bit(codes.to(torch.int8)))
        assert torch.equal(s.cpu().view(torch.int64), od.scale_fp32_to_u64(scale))
        # the reference forms the products in the weight's dtype (scale is still bf16 there), then sums
        prod = scale.to(w.dtype) * codes.to(torch.int8) * 8
        want_b = prod.sum(dim=1).float()
        bound = prod.float().abs().sum(dim=1) * 2.0 ** -8          # one bf16 rounding of a sum of that magnitude
        assert ((b.cpu() - want_b).abs() <= bound).all()
