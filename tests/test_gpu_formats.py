"""Parity of the MX (block-32 FP8/FP4 + E8M0) and HiFloat8 kernels with the CPU oracle.
The reference has neither format; the oracle is the specification."""
import numpy as np
import pytest
import torch

from amct_amd import ops, workloads
from oracle import hif8, mx
from util import assert_bits_equal

pytestmark = pytest.mark.gpu

SW = 0x100      # scale_mode bit selecting the bit-manipulation element cast


def all_bf16():
    return torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)


@pytest.mark.parametrize("fmt", [mx.E4M3, mx.E2M1])
@pytest.mark.parametrize("impl", [0, SW])
def test_mx_elements_exhaustive(dev, fmt, impl):
    """Every bf16 pattern as an element, against 40 block maxima spanning the exponent range.
    Blocks are laid out as [max, 31 elements]."""
    x = all_bf16()
    x = x[torch.isfinite(x.float())]
    n31 = (x.numel() // 31) * 31
    body = x[:n31].reshape(-1, 31)
    tail = x[n31:]
    if tail.numel():
        body = torch.cat([body, torch.cat([tail, torch.zeros(31 - tail.numel(), dtype=torch.bfloat16)]).reshape(1, 31)])
    for e in list(range(-126, 127, 7)) + [-133, 0, 127]:
        for man in (1.0, 1.984375):
            amax = torch.tensor(float(np.ldexp(man, e))).to(torch.bfloat16)
            blk = torch.cat([amax.expand(body.shape[0], 1), body], 1)          # [nblk, 32]
            # elements larger than the block maximum would change it: clip them to it
            blk = torch.where(blk.float().abs() > amax.float(), amax.expand_as(blk), blk)
            el, e8 = ops.mx_quant(blk.to(dev), fmt, mx.FLOOR | impl)
            oel, oe8 = mx.mx_quant(blk, fmt, mx.FLOOR)
            assert_bits_equal(e8, oe8, "e8m0 e=%d" % e)
            assert_bits_equal(el, oel, "elements e=%d man=%g" % (e, man))


@pytest.mark.parametrize("fmt", [mx.E4M3, mx.E2M1])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("mode", [mx.FLOOR, mx.RCEIL])
def test_mx_quant_random_and_special(dev, fmt, dtype, mode):
    g = torch.Generator().manual_seed(79)
    x = (torch.randn(96, 256, generator=g) * torch.pow(10.0, torch.rand(96, 1, generator=g) * 8 - 4)).to(dtype)
    x[0, :32] = 0
    x[1, 5] = float('nan')
    x[2, 40] = float('inf')
    x[3, :32] = 1e-7 if dtype != torch.float16 else 6e-8
    for impl in (0, SW):
        el, e8 = ops.mx_quant(x.to(dev), fmt, mode | impl)
        oel, oe8 = mx.mx_quant(x, fmt, mode)
        assert_bits_equal(e8, oe8, "e8m0")
        assert_bits_equal(el, oel, "elements impl=%d" % impl)


@pytest.mark.parametrize("fmt", [mx.E4M3, mx.E2M1])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_mx_dequant_all_codes(dev, fmt, dtype):
    if fmt == mx.E4M3:
        el = torch.arange(256, dtype=torch.int32).to(torch.uint8).repeat(1, 4).reshape(32, 32)     # every code
    else:
        el = torch.arange(256, dtype=torch.int32).to(torch.uint8).reshape(16, 16)                  # every nibble pair
    for byte in (0, 1, 100, 127, 130, 254, 255):
        if dtype == torch.float16 and byte in (254,):
            continue
        e8 = torch.full((el.shape[0], 1), byte, dtype=torch.uint8)
        got = ops.mx_dequant(el.to(dev), e8.to(dev), fmt, dtype)
        want = mx.mx_dequant(el, e8, fmt, dtype)
        g, w = got.cpu(), want
        nan = torch.isnan(w.float())
        assert torch.equal(torch.isnan(g.float()), nan)
        assert_bits_equal(torch.where(nan, torch.zeros_like(g), g), torch.where(nan, torch.zeros_like(w), w), "dequant byte=%d" % byte)


def test_mx_config3_roundtrip(dev):
    """Benchmark configuration 3 at full size: oracle parity on a row sample, idempotence on all of it."""
    x = workloads.c3_activations()
    xd = x.to(dev)
    rows = torch.arange(0, 8192, 61)
    for fmt in (mx.E4M3, mx.E2M1):
        el, e8 = ops.mx_quant(xd, fmt)
        oel, oe8 = mx.mx_quant(x[rows], fmt)
        assert_bits_equal(el.cpu()[rows], oel, "elements")
        assert_bits_equal(e8.cpu()[rows], oe8, "e8m0")
        dq = ops.mx_dequant(el, e8, fmt, torch.bfloat16)
        assert_bits_equal(dq.cpu()[rows], mx.mx_dequant(oel, oe8, fmt, torch.bfloat16), "dequant")
        el2, e82 = ops.mx_quant(dq, fmt)
        assert torch.equal(el2, el) and torch.equal(e82, e8)


def test_hif8_table_and_exhaustive_encode(dev):
    table = torch.from_numpy(hif8.decode_table())
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    got = ops.hif8_decode(codes.to(dev), torch.float32).cpu()
    nan = torch.isnan(table)
    assert torch.equal(torch.isnan(got), nan)
    assert_bits_equal(torch.where(nan, torch.zeros_like(got), got), torch.where(nan, torch.zeros_like(table), table), "decode table")
    # every bf16 and fp16 pattern through the encoder
    for dtype in (torch.bfloat16, torch.float16):
        x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
        for sat in (False, True):
            got = ops.hif8_encode(x.to(dev), sat).cpu().numpy()
            want = hif8.encode_bruteforce(x.float().numpy(), sat)
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, (dtype, sat, bad[:5], x[bad[:5].tolist()], got[bad[:5]], want[bad[:5]])
    # encode(decode(c)) == c for every non-NaN code
    rt = ops.hif8_encode(ops.hif8_decode(codes.to(dev), torch.float32)).cpu()
    keep = codes != 0x80
    assert torch.equal(rt[keep], codes[keep])


def test_hif8_fp32_random_and_ties(dev):
    rng = np.random.default_rng(83)
    x = (rng.standard_normal(1 << 20) * 10.0 ** rng.uniform(-9, 6, 1 << 20)).astype(np.float32)
    t = hif8.decode_table()
    fin = np.sort(t[np.isfinite(t) & (t > 0)])
    mids = ((fin[:-1].astype(np.float64) + fin[1:].astype(np.float64)) / 2).astype(np.float32)   # exact in fp32
    ties = np.concatenate([mids, -mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e30)),
                           np.array([2.0 ** -23, 2.0 ** -24, 1.25 * 2.0 ** 15, np.nextafter(np.float32(1.25 * 2.0 ** 15), np.float32(0))], dtype=np.float32)])
    x = np.concatenate([x, ties, np.zeros((-(x.size + ties.size)) % 4, dtype=np.float32)])
    got = ops.hif8_encode(torch.from_numpy(x).to(dev)).cpu().numpy()
    want = hif8.encode_bruteforce(x)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, (bad[:5], x[bad[:5]], got[bad[:5]], want[bad[:5]])


def test_hif8_config3(dev):
    x = workloads.c3_activations()
    c = ops.hif8_encode(x.to(dev))
    rows = torch.arange(0, 8192, 61)
    want = hif8.encode_bruteforce(x[rows].float().numpy())
    assert np.array_equal(c.cpu()[rows].numpy(), want)
    d = ops.hif8_decode(c, torch.bfloat16)
    assert_bits_equal(d.cpu()[rows], torch.from_numpy(hif8.decode(want)).to(torch.bfloat16), "decode")
    # decode -> encode is the identity on codes at full size
    assert torch.equal(ops.hif8_encode(d), c)
    # odd element counts take the scalar tail
    y = x.reshape(-1)[:1003].contiguous()
    assert np.array_equal(ops.hif8_encode(y.to(dev)).cpu().numpy(), hif8.encode_bruteforce(y.float().numpy()))


@pytest.mark.parametrize("sat", [False, True])
def test_hif8_bf16_specials_among_ordinary_values(dev, sat):
    """A bf16 tensor of many chunks (so that blocks loop) plus a ragged remainder, with infinities, NaNs of every kind
    (payload in the last three mantissa bits only included), signed zeros, values around the overflow threshold and
    below the smallest code scattered among ordinary values: waves with and without a special value take different
    routines and must agree with the brute-force encoder everywhere; decode then returns to the table values."""
    g = torch.Generator().manual_seed(29)
    n = 1024 * 8 * 300 + 8 * 77 + 5
    x = (torch.randn(n, generator=g) * torch.exp2(torch.randint(-26, 17, (n,), generator=g).float())).to(torch.bfloat16)
    bits = x.view(torch.int16).clone()
    special = torch.tensor([0x7F80, 0xFF80, 0x7FC0, 0xFFC0, 0x7F81, 0xFF87, 0x7FFF, 0x0000, 0x8000, 0x0001, 0x8001,
                            0x4700, 0x4720, 0x4740, 0xC720, 0x3400, 0x33C0, 0xB400, 0x3380], dtype=torch.int32).to(torch.int16)
    where = torch.randperm(n, generator=g)[: 4000]
    bits[where] = special[torch.arange(where.numel()) % special.numel()]
    # leave a long stretch without any special value, so that whole waves take the table routine
    bits[1024 * 8 * 100: 1024 * 8 * 200] = x.view(torch.int16)[1024 * 8 * 100: 1024 * 8 * 200]
    x = bits.view(torch.bfloat16)
    got = ops.hif8_encode(x.to(dev), sat)
    want = hif8.encode_bruteforce(x.float().numpy(), sat)
    bad = np.nonzero(got.cpu().numpy() != want)[0]
    assert bad.size == 0, (sat, bad[:5], x[bad[:5].tolist()], got.cpu().numpy()[bad[:5]], want[bad[:5]])
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        d = ops.hif8_decode(got, dtype).cpu()
        ref = torch.from_numpy(hif8.decode(want)).to(dtype)
        nan = torch.isnan(ref)
        assert torch.equal(torch.isnan(d), nan)
        assert_bits_equal(torch.where(nan, torch.zeros_like(d), d), torch.where(nan, torch.zeros_like(ref), ref), "decode")
