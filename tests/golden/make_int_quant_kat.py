#!/usr/bin/env python3
"""Writes tests/golden/int_quant_kat.json: known answers for the integer weight quantisation chain
(min/max -> scale/offset -> codes -> dequantised value), computed with exact rational arithmetic.

Every fp32 operation of the chain is modelled as "exact result as a fraction, then one rounding to
the nearest binary32 value, ties to even", written out here from the IEEE-754 definition with
Python integers and `fractions.Fraction`.  No floating-point library takes part, so a mistake in
the torch-based oracle (a fused or reordered operation, a division replaced by a reciprocal, a
different rounding of ties, a dtype promotion) shows up as a mismatch against this file.

The chain (the formulas of the quantisation scheme, one rounding per operation):
  symmetric:   bound = max(|max|, |min|); scope = 2^(b-1) - 1, plus 1 when |max| < |min|;
               s = fl(bound / scope)
  asymmetric:  max' = max(max, 0); min' = min(min, 0); scope = 2^b - 1;
               s = fl(fl(max' - min') / scope);
               z = rne(fl(-2^(b-1) - fl(min' / s)))   (z = -2^(b-1) when max' == min')
  guard:       s < 1.192092896e-7 -> s = 1 (and z = -2^(b-1))
  element:     t = fl(w / s); asymmetric: t = fl(t + z); q = clamp(rne(t), -2^(b-1), 2^(b-1) - 1)
               dq = fl(fl(q - z) * s), with the IEEE sign rules for zero results

Values are stored as binary32 bit patterns (hex) so that nothing is lost in the text form.
A second file, int_quant_kat16.json, holds the same chain for bf16 / fp16 / fp32 sources with per-group factors
(ragged last groups included) and the variant that narrows the scaled value to the source format before the
round-to-integer (the AWQ search's fake-quant); see main16 below.
Run from the repository root:  python tests/golden/make_int_quant_kat.py
"""
import json
import os
import random
import struct
from fractions import Fraction

EPS = Fraction(struct.unpack('<f', struct.pack('<f', 1.192092896e-7))[0])


def f32_to_frac(bits):
    """binary32 bit pattern -> exact Fraction (finite values only)."""
    sign = -1 if bits >> 31 else 1
    e = (bits >> 23) & 0xFF
    m = bits & 0x7FFFFF
    if e == 0:
        return sign * Fraction(m, 1 << 149)
    return sign * Fraction((1 << 23) | m, 1) * Fraction(2) ** (e - 150)


def fl(x):
    """Fraction -> bit pattern of the nearest binary32, ties to even (no overflow handling needed)."""
    if x == 0:
        return 0
    sign = 0x80000000 if x < 0 else 0
    a = -x if x < 0 else x
    # exponent e with 2^e <= a < 2^(e+1)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    if Fraction(2) ** (e + 1) <= a:
        e += 1
    e_eff = max(e, -126)                       # subnormals share the exponent of the smallest normal
    scaled = a / Fraction(2) ** (e_eff - 23)   # significand in units of one ulp
    n = scaled.numerator // scaled.denominator
    rem = scaled - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (n & 1)):
        n += 1
    if n == 0:
        return sign
    if n >= (1 << 24):                         # rounded up into the next binade
        n >>= 1
        e_eff += 1
    if n < (1 << 23):                          # subnormal
        return sign | n
    return sign | ((e_eff + 127) << 23) | (n & 0x7FFFFF)


def rne_int(x):
    """Fraction -> nearest integer, ties to even."""
    n = x.numerator // x.denominator
    rem = x - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (n & 1)):
        n += 1
    return n


def F(bits):
    return f32_to_frac(bits)


def chain(w_bits, bits, symmetric):
    w = [F(b) for b in w_bits]
    vmax, vmin = max(w), min(w)
    half = 1 << (bits - 1)
    if symmetric:
        neg = abs(vmax) < abs(vmin)
        scope = half - 1 + (1 if neg else 0)
        bound = abs(vmax) if abs(vmax) > abs(vmin) else abs(vmin)
        s = F(fl(bound / scope))
        z = None
        if s < EPS:
            s = Fraction(1)
    else:
        vmax = max(vmax, Fraction(0))
        vmin = min(vmin, Fraction(0))
        scope = (1 << bits) - 1
        s = F(fl(F(fl(vmax - vmin)) / scope))
        if s < EPS:
            s = Fraction(1)
            zf = Fraction(-half)
        elif vmax != vmin:
            zf = F(fl(Fraction(-half) - F(fl(vmin / s))))
        else:
            zf = Fraction(-half)
        z = rne_int(zf)
    codes, dq = [], []
    for x, xb in zip(w, w_bits):
        t = F(fl(x / s))
        if z is not None:
            t = F(fl(t + z))
        q = min(max(rne_int(t), -half), half - 1)
        codes.append(q)
        d = F(fl(Fraction(q - (z or 0))))
        bits_out = fl(d * s)
        if d == 0:
            # sign of a zero result (IEEE-754): rounding a negative value to zero gives -0, -0 * s = -0,
            # (-0) + (+0) = +0, (-0) - (+0) = -0, x - x = +0
            if z is None:
                neg = x < 0 or (x == 0 and xb >> 31)
            else:
                neg = (z == 0) and t < 0
            bits_out = 0x80000000 if neg else 0
        dq.append(bits_out)
    return fl(s), z, codes, dq


def rand_bits(rng, kind):
    """A binary32 pattern: 'small' ~ weights of magnitude 1e-2, 'wide' any exponent in a safe range,
    'grid' multiples of 1/64 (many exact ties once divided by a power-of-two scale)."""
    if kind == 'grid':
        v = Fraction(rng.randint(-640, 640), 64)
        return fl(v)
    sign = rng.getrandbits(1) << 31
    if kind == 'small':
        e = rng.randint(115, 122)
    else:
        e = rng.randint(90, 160)
    return sign | (e << 23) | rng.getrandbits(23)


def main():
    rng = random.Random(20240611)
    cases = []
    for bits in (8, 4):
        for symmetric in (True, False):
            for kind in ('small', 'wide', 'grid'):
                for n in (1, 5, 32, 128):
                    w_bits = [rand_bits(rng, kind) for _ in range(n)]
                    if kind == 'grid' and n >= 5:
                        # force a power-of-two scale: extremum +-(scope)/2^k makes s = 2^-k exactly
                        scope = (1 << (bits - 1)) - 1 if symmetric else (1 << bits) - 1
                        w_bits[0] = fl(Fraction(scope, 4)) if symmetric else fl(Fraction(scope, 8))
                        if not symmetric:
                            w_bits[1] = fl(Fraction(-scope, 8))
                            w_bits = [b for b in w_bits if abs(F(b)) <= Fraction(scope, 8)] + [w_bits[0], w_bits[1]]
                        else:
                            w_bits = [b for b in w_bits if abs(F(b)) < Fraction(scope, 4)] + [w_bits[0]]
                    s, z, codes, dq = chain(w_bits, bits, symmetric)
                    cases.append({"bits": bits, "symmetric": symmetric, "kind": kind,
                                  "w": ["%08x" % b for b in w_bits], "scale": "%08x" % s, "offset": z,
                                  "codes": codes, "dq": ["%08x" % b for b in dq]})
    # hand-picked rows: negative extremum dominates (scope 2^(b-1)), all zero (guard), one-sided
    # ranges (the zero clamp of the asymmetric form), exact half-way quotients
    special = [
        [fl(Fraction(-1)), fl(Fraction(1, 2)), fl(Fraction(127, 128)), fl(Fraction(-127, 256))],
        [0, 0, 0x80000000, 0],
        [fl(Fraction(3, 8)), fl(Fraction(5, 8)), fl(Fraction(1, 8))],
        [fl(Fraction(-3, 8)), fl(Fraction(-5, 8)), fl(Fraction(-1, 8))],
        [fl(Fraction(127, 2)), fl(Fraction(1, 4)), fl(Fraction(3, 4)), fl(Fraction(5, 4)), fl(Fraction(-7, 4)),
         fl(Fraction(-9, 4))],
        [fl(Fraction(1, 1 << 30)), fl(Fraction(-1, 1 << 31))],
    ]
    for bits in (8, 4):
        for symmetric in (True, False):
            for w_bits in special:
                s, z, codes, dq = chain(w_bits, bits, symmetric)
                cases.append({"bits": bits, "symmetric": symmetric, "kind": "special",
                              "w": ["%08x" % b for b in w_bits], "scale": "%08x" % s, "offset": z,
                              "codes": codes, "dq": ["%08x" % b for b in dq]})
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "int_quant_kat.json")
    with open(out, "w") as f:
        json.dump({"format": "binary32 bit patterns as hex; one case = one row quantised per-channel",
                   "cases": cases}, f, indent=0, separators=(",", ":"))
    print("wrote", out, len(cases), "cases")


# ---- second file: 16-bit sources, per-group factors, AWQ's cast-before-round path -----------------------------
# A 16-bit source only adds roundings to its own format: the dequantised value is rounded to the source format at
# the end (after the fp32 product), and on AWQ's path the scaled value t is rounded to the source format BEFORE the
# round-to-integer.  Formats: (significand bits incl. the hidden one, minimum normal exponent).
FORMATS = {"f32": (24, -126), "bf16": (8, -126), "f16": (11, -14)}


def fl_fmt(x, fmt):
    """Fraction -> nearest value of the format as a Fraction, ties to even (finite range assumed)."""
    if x == 0:
        return Fraction(0)
    p, emin = FORMATS[fmt]
    a = -x if x < 0 else x
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    if Fraction(2) ** (e + 1) <= a:
        e += 1
    ulp = Fraction(2) ** (max(e, emin) - (p - 1))
    scaled = a / ulp
    n = scaled.numerator // scaled.denominator
    rem = scaled - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (n & 1)):
        n += 1
    r = n * ulp
    return -r if x < 0 else r


def bits_of(x, fmt, negative_zero=False):
    """Fraction (exactly representable) -> bit pattern of the format."""
    if fmt == "f32":
        b = fl(x)
        return 0x80000000 if (x == 0 and negative_zero) else b
    b32 = fl(x)
    if x == 0:
        return 0x8000 if negative_zero else 0
    if fmt == "bf16":
        assert b32 & 0xFFFF == 0
        return b32 >> 16
    sign = (b32 >> 31) << 15
    a = -x if x < 0 else x
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    if e < -14:
        m = a / Fraction(2) ** -24
        assert m.denominator == 1
        return sign | int(m)
    m = a / Fraction(2) ** (e - 10)
    assert m.denominator == 1 and (1 << 10) <= m < (1 << 11)
    return sign | ((e + 15) << 10) | (int(m) & 0x3FF)


def frac_of(bits, fmt):
    if fmt == "f32":
        return f32_to_frac(bits)
    if fmt == "bf16":
        return f32_to_frac(bits << 16)
    sign = -1 if bits >> 15 else 1
    e = (bits >> 10) & 0x1F
    m = bits & 0x3FF
    if e == 0:
        return sign * Fraction(m, 1 << 24)
    return sign * Fraction((1 << 10) | m) * Fraction(2) ** (e - 25)


def is_neg_zero(bits, fmt):
    return bits == (0x80000000 if fmt == "f32" else 0x8000)


def factors(seg, bits, symmetric):
    """(s as Fraction, z int|None) of one segment (list of Fractions, padding zeros included)."""
    vmax, vmin = max(seg), min(seg)
    half = 1 << (bits - 1)
    if symmetric:
        neg = abs(vmax) < abs(vmin)
        scope = half - 1 + (1 if neg else 0)
        bound = abs(vmax) if abs(vmax) > abs(vmin) else abs(vmin)
        s = F(fl(bound / scope))
        if s < EPS:
            s = Fraction(1)
        return s, None
    vmax = max(vmax, Fraction(0))
    vmin = min(vmin, Fraction(0))
    scope = (1 << bits) - 1
    s = F(fl(F(fl(vmax - vmin)) / scope))
    if s < EPS:
        return Fraction(1), -half
    if vmax != vmin:
        return s, rne_int(F(fl(Fraction(-half) - F(fl(vmin / s)))))
    return s, -half


def chain16(w_bits, fmt, bits, symmetric, group):
    """Per element: code, plain dequantised value and AWQ-path dequantised value (bit patterns of `fmt`)."""
    w = [frac_of(b, fmt) for b in w_bits]
    n = len(w)
    g = group if group else n
    half = 1 << (bits - 1)
    scales, offsets, codes, dq, adq = [], [], [], [], []
    for g0 in range(0, n, g):
        seg = w[g0:g0 + g]
        real = len(seg)
        seg = seg + [Fraction(0)] * (g - real)              # the zero padding takes part in min / max
        s, z = factors(seg, bits, symmetric)
        scales.append(fl(s))
        offsets.append(z)
        for i in range(real):
            x, xb = seg[i], w_bits[g0 + i]
            t = F(fl(x / s))
            if z is not None:
                t = F(fl(t + z))
            for path, out in (("plain", dq), ("awq", adq)):
                tt = fl_fmt(t, fmt) if path == "awq" else t
                q = min(max(rne_int(tt), -half), half - 1)
                if path == "plain":
                    codes.append(q)
                d = Fraction(q - (z or 0))
                v = fl_fmt(F(fl(d * s)), fmt)
                negz = False
                if v == 0:
                    if d != 0:
                        negz = d < 0                          # a product that underflows keeps its sign
                    elif z is None:
                        negz = x < 0 or (x == 0 and is_neg_zero(xb, fmt))
                    else:
                        negz = (z == 0) and t < 0
                out.append(bits_of(v, fmt, negz))
    return scales, (None if symmetric else offsets), codes, dq, adq


def rand_bits16(rng, fmt, kind):
    if kind == 'grid':
        return bits_of(fl_fmt(Fraction(rng.randint(-160, 160), 16), fmt), fmt)
    if fmt == "f32":
        return rand_bits(rng, kind)
    sign = rng.getrandbits(1) << 15
    if fmt == "bf16":
        e = rng.randint(115, 122) if kind == 'small' else rng.randint(100, 150)
        return sign | (e << 7) | rng.getrandbits(7)
    e = rng.randint(6, 12) if kind == 'small' else rng.randint(1, 26)
    return sign | (e << 10) | rng.getrandbits(10)


def main16():
    rng = random.Random(20250215)
    cases = []
    hexw = {"f32": "%08x", "bf16": "%04x", "f16": "%04x"}
    for fmt in ("bf16", "f16", "f32"):
        for bits in (8, 4):
            for symmetric in (True, False):
                for kind in ('small', 'wide', 'grid'):
                    for n, group in ((48, 0), (64, 32), (80, 32), (37, 0)):
                        if fmt == "f32" and group == 0 and n == 48:
                            continue                         # the first file covers whole-row fp32
                        w_bits = [rand_bits16(rng, fmt, kind) for _ in range(n)]
                        if kind == 'grid':
                            # an extremum that makes the scale a power of two, so quotients hit exact ties
                            scope = (1 << (bits - 1)) - 1 if symmetric else (1 << bits) - 1
                            w_bits[0] = bits_of(fl_fmt(Fraction(scope, 8), fmt), fmt)
                        sc, off, codes, dq, adq = chain16(w_bits, fmt, bits, symmetric, group)
                        cases.append({"src": fmt, "bits": bits, "symmetric": symmetric, "group": group, "kind": kind,
                                      "w": [hexw[fmt] % b for b in w_bits], "scale": ["%08x" % b for b in sc],
                                      "offset": off, "codes": codes, "dq": [hexw[fmt] % b for b in dq],
                                      "awq_dq": [hexw[fmt] % b for b in adq]})
    ndiff = sum(1 for c in cases if c["dq"] != c["awq_dq"])
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "int_quant_kat16.json")
    with open(out, "w") as f:
        json.dump({"format": "bit patterns as hex (binary32 for scales, the source format for w / dq / awq_dq); "
                             "one case = one row, factors per group of `group` columns (0: the whole row), a ragged "
                             "last group is zero-padded; awq_dq = the value is narrowed to the source format before "
                             "the round-to-integer",
                   "cases": cases}, f, indent=0, separators=(",", ":"))
    print("wrote", out, len(cases), "cases;", ndiff, "of them have awq_dq != dq")


if __name__ == "__main__":
    main()
    main16()
