"""HiFloat8 oracle (CPU, numpy) -- test infrastructure only.

The reference contains no HiFloat8 code, so parity with it is UNPINNED by
construction.  The format follows the public description of HiFloat8
(tapered precision: a prefix-coded "dot" field selects how many bits go to
the exponent); the exact bit layout below is this repository's and is what
the HIP kernels implement.  tests/test_oracle_hif8.py pins the table through
its structural invariants (value counts per binade, sign symmetry, range
2^-22 .. 2^15, unique values, encode(decode(c)) == c).

Layout, MSB first:  S | dot | exponent (D bits) | mantissa
  dot 11   -> D=4, 1 mantissa bit      |E| in 8..15
  dot 10   -> D=3, 2 mantissa bits     |E| in 4..7
  dot 01   -> D=2, 3 mantissa bits     |E| in 2..3
  dot 001  -> D=1, 3 mantissa bits     |E| = 1
  dot 0001 -> D=0, 3 mantissa bits     E = 0
  dot 0000 -> denormal, 3-bit field M: value 2^(M-23), M = 1..7
The exponent field is sign-magnitude: first bit = sign of E, the remaining
D-1 bits are the magnitude below a hidden leading one.
Normal value (-1)^S * 2^E * (1 + mantissa / 2^mbits).
0x00 = zero, 0x80 = NaN, E=+15 with mantissa 1 (0x6F / 0xEF) = +-Inf, so the
largest finite magnitude is 2^15 and the smallest is 2^-22.

Encoding rounds to the nearest representable value, ties AWAY from zero;
|x| >= 1.25 * 2^15 becomes Inf (or +-2^15 with saturate=True), |x| < 2^-23
becomes zero (0x00 for either sign), NaN becomes 0x80.
"""
import numpy as np

NAN_CODE = 0x80
POS_INF = 0x6F
NEG_INF = 0xEF
MAX_FINITE_CODE = 0x6E          # +2^15


def _decode_one(c):
    s = -1.0 if c & 0x80 else 1.0
    b = c & 0x7F
    if b >> 5 == 0b11:
        d, mb = 4, 1
    elif b >> 5 == 0b10:
        d, mb = 3, 2
    elif b >> 5 == 0b01:
        d, mb = 2, 3
    elif b >> 4 == 0b001:
        d, mb = 1, 3
    elif b >> 3 == 0b0001:
        d, mb = 0, 3
    else:
        m = b & 7
        if m == 0:
            return float('nan') if c & 0x80 else 0.0
        return s * 2.0 ** (m - 23)
    man = b & ((1 << mb) - 1)
    ef = (b >> mb) & ((1 << d) - 1) if d else 0
    if d == 0:
        e = 0
    else:
        esign = (ef >> (d - 1)) & 1
        mag = (1 << (d - 1)) | (ef & ((1 << (d - 1)) - 1))
        e = -mag if esign else mag
    if e == 15 and man == 1:
        return s * float('inf')
    return s * 2.0 ** e * (1.0 + man / (1 << mb))


def decode_table():
    """256 fp32 values indexed by code."""
    return np.array([_decode_one(c) for c in range(256)], dtype=np.float32)


_TABLE = decode_table()


def decode(codes):
    return _TABLE[np.asarray(codes, dtype=np.uint8)]


def encode_bruteforce(x, saturate=False):
    """Nearest-value search over the table; x: fp32 array."""
    x = np.asarray(x, dtype=np.float32)
    pos_codes = np.array([c for c in range(128) if np.isfinite(_TABLE[c]) and _TABLE[c] > 0], dtype=np.int64)
    vals = _TABLE[pos_codes].astype(np.float64)
    order = np.argsort(vals)
    vals, pos_codes = vals[order], pos_codes[order]
    a = np.abs(x.astype(np.float64)).ravel()
    neg = np.signbit(x).ravel()
    out = np.zeros(a.shape, dtype=np.uint8)
    # candidates: 0 and every positive finite value; ties go to the larger magnitude
    grid = np.concatenate(([0.0], vals))
    gcodes = np.concatenate(([0], pos_codes))
    hi = np.searchsorted(grid, a, side='right')          # first grid value > a
    hi = np.clip(hi, 1, len(grid) - 1)
    lo = hi - 1
    pick_hi = (grid[hi] - a) <= (a - grid[lo])
    idx = np.where(pick_hi, hi, lo)
    mag_code = gcodes[idx]
    res = np.where(mag_code == 0, 0, mag_code | (neg.astype(np.int64) << 7))
    over = a >= 1.25 * 2.0 ** 15
    top = MAX_FINITE_CODE if saturate else POS_INF
    res = np.where(over, top | (neg.astype(np.int64) << 7), res)
    res = np.where(np.isnan(a), NAN_CODE, res)
    out[:] = res.astype(np.uint8)
    return out.reshape(x.shape)
