"""Microscaling (MX) block-32 oracle (CPU) -- test infrastructure only.

The reference contains no MXFP8 / MXFP4 / E8M0 code at all, so parity with it
is UNPINNED by construction; this file freezes the specification the HIP
kernels implement and tests/test_oracle_mx.py pins that specification:

  * element casts are checked exhaustively (every bf16 bit pattern) against a
    brute-force nearest-value search over the decoded value tables with the
    tie rule applied explicitly, and the E4M3 cast additionally against an
    independent library routine, torch's own float8_e4m3fn conversion;
  * the shared exponent is checked against math.frexp on every fp32 binade;
  * invariants: the block maximum always lands in the top binade of the
    element format, re-quantising a dequantised tensor reproduces codes and
    exponents, |x - dq| <= half an element ulp at that scale.

Specification (OCP Microscaling v1.0 semantics, floor scale selection)
----------------------------------------------------------------------
block      32 consecutive elements along the last dimension
amax       largest |x| of the block, taken on the bit pattern (exact)
X (E8M0)   biased byte = clamp(biased_exp_fp32(amax) - emax_elem, 0, 254),
           emax_elem = 8 for E4M3 (max 448), 2 for E2M1 (max 6);
           a block holding a NaN stores 0xFF (the whole block decodes to NaN);
           scale_mode=RCEIL instead stores ceil(log2(amax / max_elem)) + 127
           (no element can saturate), clamped the same way
element    cast(x * 2^-(byte-127)) with round-half-even and SATURATION to
           +-max normal (448 / 6); E4M3 keeps NaN as 0x7F|sign, E2M1 has no
           NaN and maps it to +-6
fp4 pack   two codes per byte, even index in the low nibble
decode     elem_value * 2^(byte-127) in fp32, rounded once (half-even) to the
           output dtype; byte 0xFF gives NaN
"""
import numpy as np
import torch

E4M3 = 0
E2M1 = 1
FLOOR = 0
RCEIL = 1

BLOCK = 32
_EMAX = {E4M3: 8, E2M1: 2}
_FMAX = {E4M3: 448.0, E2M1: 6.0}

E2M1_VALUES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)


def _f32_bits(x):
    return x.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF


def shared_exponent(x_f32, fmt, scale_mode=FLOOR):
    """x_f32 [..., nblk, 32] fp32 -> uint8 [..., nblk] biased E8M0 byte."""
    mag = _f32_bits(x_f32) & 0x7FFFFFFF
    amax = mag.amax(dim=-1)
    has_nan = amax > 0x7F800000
    be = amax >> 23
    if scale_mode == FLOOR:
        byte = be - _EMAX[fmt]
    else:
        # ceil(log2(amax / fmax)): fmax = m * 2^emax with m = 1.75 (E4M3) or 1.5 (E2M1);
        # amax = f * 2^(be-127) with f in [1,2)  ->  exponent (be-127-emax) + (f > m)
        man = amax & 0x7FFFFF
        m_fmax = {E4M3: 0x600000, E2M1: 0x400000}[fmt]
        byte = be - _EMAX[fmt] + (man > m_fmax).to(torch.int64)
        # fp32 denormal amax: value = man * 2^-149, far below any representable scale
    byte = byte.clamp(0, 254)
    byte = torch.where(has_nan, torch.full_like(byte, 255), byte)
    return byte.to(torch.uint8)


def _pow2(e_unbiased):
    """2^e as fp32 for integer tensor e in [-127, 128) (denormal for -127)."""
    return torch.ldexp(torch.ones_like(e_unbiased, dtype=torch.float32), e_unbiased.to(torch.int32))


def encode_e4m3(v):
    """fp32 -> uint8 E4M3 (OCP, no infinities), half-even, saturating.  Uses
    torch's own float8 cast after clamping."""
    nan = torch.isnan(v)
    c = v.clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
    sign = ((_f32_bits(v) >> 31) << 7).to(torch.uint8)
    return torch.where(nan, sign | 0x7F, c)


def encode_e2m1(v):
    """fp32 -> uint8 code 0..15 (sign<<3 | index), half-even on the 1-bit
    mantissa, saturating, NaN -> +-6.  Written as threshold compares so it is
    independent of any bit trick the kernels use."""
    a = v.abs()
    # midpoints; a tie goes to the code with an even mantissa bit (even index)
    idx = torch.zeros(v.shape, dtype=torch.int64)
    idx += (a > 0.25)
    idx += (a >= 0.75)
    idx += (a > 1.25)
    idx += (a >= 1.75)
    idx += (a > 2.5)
    idx += (a >= 3.5)
    idx += (a > 5.0)
    idx = torch.where(torch.isnan(v), torch.full_like(idx, 7), idx)
    sign = (_f32_bits(v) >> 31) << 3
    return (sign | idx).to(torch.uint8)


def decode_e2m1(code):
    tbl = torch.from_numpy(E2M1_VALUES)
    c = code.to(torch.int64)
    val = tbl[c & 7]
    return torch.where((c & 8) != 0, -val, val)


def decode_e4m3(code):
    return code.view(torch.float8_e4m3fn).to(torch.float32)


def mx_quant(x, fmt, scale_mode=FLOOR):
    """x [..., K] (K % 32 == 0), any float dtype -> (elements, e8m0).
    elements: uint8 [..., K] for E4M3, uint8 [..., K/2] for E2M1.
    e8m0: uint8 [..., K/32]."""
    k = x.shape[-1]
    assert k % BLOCK == 0
    xb = x.to(torch.float32).reshape(*x.shape[:-1], k // BLOCK, BLOCK)
    byte = shared_exponent(xb, fmt, scale_mode)
    eff = torch.where(byte == 255, torch.full_like(byte, 254), byte).to(torch.int64) - 127
    # multiply by 2^-e in two exact power-of-two steps so neither factor overflows
    h = eff // 2
    v = xb * _pow2(-h).unsqueeze(-1) * _pow2(-(eff - h)).unsqueeze(-1)
    if fmt == E4M3:
        el = encode_e4m3(v).reshape(*x.shape[:-1], k)
    else:
        c = encode_e2m1(v).reshape(*x.shape[:-1], k // 2, 2)
        el = (c[..., 0] | (c[..., 1] << 4)).to(torch.uint8)
    return el, byte


def mx_dequant(el, byte, fmt, dtype=torch.float32):
    if fmt == E4M3:
        v = decode_e4m3(el)
    else:
        lo = decode_e2m1(el & 0xF)
        hi = decode_e2m1(el >> 4)
        v = torch.stack((lo, hi), dim=-1).reshape(*el.shape[:-1], el.shape[-1] * 2)
    k = v.shape[-1]
    vb = v.reshape(*v.shape[:-1], k // BLOCK, BLOCK)
    e = byte.to(torch.int64) - 127
    h = e // 2
    y = vb * _pow2(h).unsqueeze(-1) * _pow2(e - h).unsqueeze(-1)
    y = torch.where((byte == 255).unsqueeze(-1), torch.full_like(y, float('nan')), y)
    return y.reshape(*v.shape[:-1], k).to(dtype)
