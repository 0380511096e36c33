"""Pins for oracle/mx.py (the reference has no MX code; the spec is ours)."""
import math

import numpy as np
import torch

from oracle import mx


def all_bf16():
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    return bits.view(torch.bfloat16)


def nearest_even_code(v, table):
    """Brute force: nearest table value, ties to the even code, saturating.
    table: 1-D float64 array of non-negative finite values indexed by code."""
    a = np.abs(v.astype(np.float64))
    d = np.abs(a[:, None] - table[None, :])
    best = d.min(axis=1)
    cand = d == best[:, None]
    # prefer even code among ties
    codes = np.arange(len(table))
    even = cand & (codes[None, :] % 2 == 0)
    pick = np.where(even.any(1), even.argmax(1), cand.argmax(1))
    pick = np.where(a > table.max(), len(table) - 1, pick)
    return pick


def test_e2m1_exhaustive_vs_bruteforce():
    x = all_bf16().float()
    fin = torch.isfinite(x)
    xv = x[fin]
    got = mx.encode_e2m1(xv).numpy()
    want = nearest_even_code(xv.numpy(), mx.E2M1_VALUES.astype(np.float64))
    sign = (xv.numpy().view(np.uint32) >> 31).astype(np.int64) << 3
    assert np.array_equal(got, (want | sign).astype(np.uint8))
    # midpoints go to the even code
    t = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 7.0, float('inf'), float('nan')])
    assert mx.encode_e2m1(t).tolist() == [0, 2, 2, 4, 4, 6, 6, 7, 7, 7]
    assert torch.equal(mx.decode_e2m1(torch.arange(8, dtype=torch.uint8)), torch.from_numpy(mx.E2M1_VALUES))


def test_e4m3_exhaustive_vs_bruteforce():
    table = mx.decode_e4m3(torch.arange(127, dtype=torch.uint8)).double().numpy()   # 0x7F is NaN
    assert table.max() == 448.0 and table[1] == 2.0 ** -9
    assert np.all(np.diff(table) > 0)
    x = all_bf16().float()
    xv = x[torch.isfinite(x)]
    got = mx.encode_e4m3(xv).numpy()
    want = nearest_even_code(xv.numpy(), table)
    sign = (xv.numpy().view(np.uint32) >> 31).astype(np.int64) << 7
    assert np.array_equal(got, (want | sign).astype(np.uint8))
    t = torch.tensor([float('nan'), float('inf'), -float('inf'), 464.0, 480.0, 1e9])
    assert mx.encode_e4m3(t).tolist()[1:] == [0x7E, 0xFE, 0x7E, 0x7E, 0x7E]
    assert mx.encode_e4m3(t)[0].item() & 0x7F == 0x7F


def test_shared_exponent_every_binade():
    for fmt, emax in ((mx.E4M3, 8), (mx.E2M1, 2)):
        for e in range(-126, 128):
            for man in (1.0, 1.5, 1.75, 1.9990234375):
                a = math.ldexp(man, e)
                if not math.isfinite(np.float32(a)):
                    continue
                blk = torch.zeros(1, 1, 32)
                blk[0, 0, 5] = -a
                byte = mx.shared_exponent(blk, fmt)[0, 0].item()
                fl = math.frexp(a)[1] - 1           # floor(log2 a)
                assert byte == min(max(fl - emax + 127, 0), 254)
    blk = torch.zeros(1, 1, 32)
    assert mx.shared_exponent(blk, mx.E4M3).item() == 0
    blk[0, 0, 0] = float('nan')
    assert mx.shared_exponent(blk, mx.E4M3).item() == 255
    # RCEIL: amax/2^X never exceeds the element max, and 2^X is the smallest such power of two
    g = torch.Generator().manual_seed(0)
    v = (torch.randn(4000, generator=g) * torch.logspace(-20, 20, 4000)).abs() + 1e-30
    for fmt, fmax in ((mx.E4M3, 448.0), (mx.E2M1, 6.0)):
        blk = torch.zeros(4000, 1, 32)
        blk[:, 0, 0] = v
        X = mx.shared_exponent(blk, fmt, mx.RCEIL)[:, 0].double() - 127
        scaled = v.double() / 2.0 ** X
        assert (scaled <= fmax).all() and (scaled * 2 > fmax).all()


def test_block_max_lands_in_top_binade_and_roundtrip():
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(64, 256, generator=g) * torch.logspace(-8, 8, 64).reshape(-1, 1)).to(torch.bfloat16)
    for fmt, emax, half_ulp_rel in ((mx.E4M3, 8, 2.0 ** -4), (mx.E2M1, 2, 2.0 ** -2)):
        el, byte = mx.mx_quant(x, fmt)
        assert byte.shape == (64, 8) and byte.dtype == torch.uint8
        assert el.shape == ((64, 256) if fmt == mx.E4M3 else (64, 128))
        dq = mx.mx_dequant(el, byte, fmt)
        amax = x.float().reshape(64, 8, 32).abs().amax(-1)
        top = dq.reshape(64, 8, 32).abs().amax(-1) / torch.ldexp(torch.ones(64, 8), byte.int() - 127)
        assert (top >= 2.0 ** emax).all()
        # error bound: half an ulp of the element at the block scale, except where saturated
        scale = torch.ldexp(torch.ones(64, 8), byte.int() - 127).unsqueeze(-1)
        xb = x.float().reshape(64, 8, 32)
        err = (xb - dq.reshape(64, 8, 32)).abs()
        fmax = 448.0 if fmt == mx.E4M3 else 6.0
        sat = xb.abs() > fmax * scale
        bound = torch.maximum(xb.abs() * half_ulp_rel, scale * (2.0 ** -10 if fmt == mx.E4M3 else 0.25))
        assert (err[~sat] <= bound[~sat]).all()
        assert (dq.reshape(64, 8, 32).abs()[sat] == (fmax * scale).expand(64, 8, 32)[sat]).all()
        # idempotence
        el2, byte2 = mx.mx_quant(dq.to(torch.bfloat16), fmt)
        assert torch.equal(byte2, byte) and torch.equal(el2, el)


def test_nan_block():
    x = torch.ones(1, 64, dtype=torch.bfloat16)
    x[0, 3] = float('nan')
    el, byte = mx.mx_quant(x, mx.E4M3)
    assert byte.tolist() == [[255, 127 - 8]]
    dq = mx.mx_dequant(el, byte, mx.E4M3)
    assert torch.isnan(dq[0, :32]).all() and (dq[0, 32:] == 1).all()
