"""Parity of the int4 group-pack kernel, the int4 layouts and the activation quantisers."""
import pytest
import torch

from amct_amd import ops, workloads
from oracle import deploy as od
from oracle import int_quant as iq
from util import assert_bits_equal

pytestmark = pytest.mark.gpu


def oracle_pack(w, group, sym, scale_dtype):
    s, z = iq.weight_scale_offset(w, 'group', sym, 'int4', group)
    codes = iq.quant_codes(w, 'int4', s, z, group).reshape(w.shape[0], -1)
    packed = od.pack_nibbles_k(codes)
    zeros = (z.squeeze(-1) + 8).to(torch.uint8) if z is not None else torch.full(s.shape[:2], 8, dtype=torch.uint8)
    return packed, s.squeeze(-1).to(scale_dtype), zeros, s.squeeze(-1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape,group", [((64, 256), 32), ((64, 256), 128), ((17, 1024), 256), ((8, 4096), 1024),
                                         ((3, 8192), 8192), ((130, 384), 128), ((4, 4096), 4096)])
@pytest.mark.parametrize("sym", [False, True])
def test_int4_group_pack(dev, dtype, shape, group, sym):
    g = torch.Generator().manual_seed(61)
    w = (torch.randn(*shape, generator=g) * 0.02)
    w[0, :group] = 0
    w = w.to(dtype)
    for sdt in (torch.float16, torch.bfloat16):
        packed, s16, zeros, s32 = ops.quant_int4_group_pack(w.to(dev), group, sym, sdt, want_scales32=True)
        op, os16, oz, os32 = oracle_pack(w, group, sym, sdt)
        assert_bits_equal(s32, os32, "scales32")
        assert_bits_equal(s16, os16, "scales16")
        assert_bits_equal(zeros, oz, "zeros")
        assert_bits_equal(packed, op, "packed")
        # u - zu == q - offset (round trip through the oracle's unpack)
        assert torch.equal(od.unpack_nibbles_k(packed.cpu()), od.unpack_nibbles_k(op))


def test_config2_slice(dev):
    """Benchmark configuration 2 (outliers, bf16, g=128) on the first 1024 rows vs the oracle."""
    w = workloads.c2_weight(1024, 4096)
    packed, s16, zeros, s32 = ops.quant_int4_group_pack(w.to(dev), 128, False, torch.float16, want_scales32=True)
    op, os16, oz, os32 = oracle_pack(w, 128, False, torch.float16)
    assert_bits_equal(s32, os32, "scales32")
    assert_bits_equal(s16, os16, "scales16")
    assert_bits_equal(zeros, oz, "zeros")
    assert_bits_equal(packed, op, "packed")


def test_config2_full_size_properties(dev):
    """Full [14336,4096]: size-independent properties -- fused pack == K1 codes packed by the
    oracle's packer on a row sample, zeros in range, dequantised error within half a step."""
    w = workloads.c2_weight()
    wd = w.to(dev)
    packed, s16, zeros, s32 = ops.quant_int4_group_pack(wd, 128, False, torch.float16, want_scales32=True)
    _, codes, s, z = ops.fakequant_int(wd, 4, False, group=128, want_dq=False, codes_kind=ops.CODES_I8)
    assert_bits_equal(s32, s.cpu(), "scale K2 vs K1")
    assert_bits_equal(zeros.cpu().to(torch.int32) - 8, z.cpu(), "zeros K2 vs K1")
    assert zeros.max().item() <= 15
    rows = torch.arange(0, 14336, 97)
    assert_bits_equal(packed.cpu()[rows], od.pack_nibbles_k(codes.cpu()[rows].to(torch.int32)), "packed sample")
    u = od.unpack_nibbles_k(packed.cpu()[rows]).float().reshape(len(rows), 32, 128)
    deq = (u - z.cpu()[rows].float().unsqueeze(-1)) * s32.cpu()[rows].unsqueeze(-1)
    err = (deq.reshape(len(rows), -1) - w[rows].float()).abs().reshape(len(rows), 32, 128)
    assert (err <= s32.cpu()[rows].unsqueeze(-1) * 0.5001).all()


@pytest.mark.parametrize("k,n", [(64, 48), (256, 384), (128, 128), (384, 1160), (192, 136), (2, 8)])
def test_int4_word_layouts(dev, k, n):
    """The layout converters on shapes that take the tiled / vector kernels (k % 128 == 0 and n % 128 == 0; k, n % 64
    == 0) and on shapes that take the element-wise ones; every conversion against the oracle and the round trip."""
    g = torch.Generator().manual_seed(67)
    codes = torch.randint(-8, 8, (k, n), generator=g, dtype=torch.int32)            # [k, n]
    words = ops.pack_int4_words(codes.to(dev))
    assert_bits_equal(words, od.pack_int4_words(codes), "words")
    assert torch.equal(od.unpack_int4_words(words.cpu()), codes)
    nib = ops.words_to_nibbles_nk(words, k, n)
    want_nib = od.pack_nibbles_k(codes.t().contiguous())
    assert_bits_equal(nib, want_nib, "nibbles [n,k/2]")
    assert_bits_equal(ops.pack_nibbles_nk(codes.t().contiguous().to(torch.int8).to(dev)), want_nib, "nibbles from int8 codes")
    assert_bits_equal(ops.unpack_nibbles_to_i32_kn(nib), codes, "codes [k,n] back from the nibbles")
    # nibble order agrees with the usual uint4 packing convention: low nibble = even index
    u = torch.tensor([[1, 2, 3, 4]], dtype=torch.int32) - 8
    assert od.pack_nibbles_k(u).tolist() == [[0x21, 0x43]]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(12, 128), (33, 4096), (5, 100), (2, 16384), (3, 20000), (1, 8), (3, 28672), (2, 40000)])
def test_dynamic_per_token(dev, dtype, shape):
    g = torch.Generator().manual_seed(71)
    x = torch.randn(*shape, generator=g).to(dtype)
    x[0] = 0
    q, s = ops.act_quant_per_token_int8(x.to(dev))
    oq, os_ = iq.dynamic_token_quant(x)
    assert_bits_equal(s, os_, "scale")
    assert_bits_equal(q, oq, "codes")
    # with the smoothing multiply fused in
    sm = (0.25 + torch.rand(shape[1], generator=g)).to(dtype)
    q, s = ops.act_quant_per_token_int8(x.to(dev), smooth=sm.to(dev))
    oq, os_ = iq.dynamic_token_quant(x, sm)
    assert_bits_equal(s, os_, "scale smooth")
    assert_bits_equal(q, oq, "codes smooth")
    # absmax/127 form, defined on fp32 values
    q, s = ops.act_quant_per_token_int8(x.float().to(dev), mode=1)
    oq, os_ = iq.dynamic_token_quant_absmax(x.float())
    assert_bits_equal(s, os_, "scale absmax")
    assert_bits_equal(q, oq.reshape(shape), "codes absmax")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(2, 24, 96), (1, 300, 4096), (3, 5, 100), (1, 7, 37)])
def test_static_quantize(dev, dtype, shape):
    """Vector kernel (K a multiple of 8, or of 4 for fp32) and scalar fallback, per tensor / per channel / per token,
    with and without zero-points."""
    g = torch.Generator().manual_seed(73)
    x = (torch.randn(*shape, generator=g) * 3).to(dtype)
    for per_token, n in ((False, 1), (False, shape[-1]), (True, shape[-2])):
        sc = (5 + 20 * torch.rand(n, generator=g)).to(dtype)
        zp = torch.randint(-20, 20, (n,), generator=g).to(dtype)
        for z in (zp, None):
            got = ops.quantize_static(x.to(dev), sc.to(dev), None if z is None else z.to(dev), per_token)
            want = iq.static_quantize(x, sc, z, axis=-2 if per_token else -1)
            assert_bits_equal(got, want, "static per_token=%s n=%d" % (per_token, n))
