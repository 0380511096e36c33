"""Pins for oracle/hif8.py: structural invariants of the value table and the
encoder's consistency with it (the reference has no HiFloat8 code)."""
import math

import numpy as np

from oracle import hif8


def test_table_structure():
    t = hif8.decode_table()
    assert t[0] == 0 and np.isnan(t[0x80])
    assert np.isposinf(t[hif8.POS_INF]) and np.isneginf(t[hif8.NEG_INF])
    pos = [c for c in range(1, 128) if np.isfinite(t[c])]
    assert len(pos) == 126                       # 128 - zero - inf
    vals = t[pos].astype(np.float64)
    assert len(np.unique(vals)) == 126           # no value encoded twice
    assert vals.min() == 2.0 ** -22 and vals.max() == 2.0 ** 15
    assert t[hif8.MAX_FINITE_CODE] == 2.0 ** 15
    # sign symmetry
    for c in pos:
        assert t[c | 0x80] == -t[c]
    # mantissa bits per binade: 3 for |E|<=3, 2 for 4..7, 1 for 8..15, 0 in the denormal range
    per = {}
    for v in vals:
        per.setdefault(math.frexp(v)[1] - 1, []).append(v)
    for e, vs in per.items():
        want = 8 if abs(e) <= 3 else 4 if abs(e) <= 7 else 2 if abs(e) <= 15 else 1
        if e == 15:
            want = 1                             # the other slot is Inf
        assert len(vs) == want, (e, vs)
        fr = sorted(v / 2.0 ** e for v in vs)
        assert fr == [1 + i / want for i in range(want)] or e == 15
    assert sorted(per) == list(range(-22, 16))   # 38 binades


def test_encode_roundtrip_and_ties():
    t = hif8.decode_table()
    for c in range(256):
        if c == 0x80:
            continue
        got = hif8.encode_bruteforce(np.array([t[c]], dtype=np.float32))[0]
        assert got == c, (hex(c), t[c], hex(got))
    x = np.array([np.nan, 0.0, -0.0, 2.0 ** -24, 2.0 ** -23, -2.0 ** -23, 1.5 * 2.0 ** -22,
                  1.0625, 1.1875, -1.0625, 2.0 ** 15 * 1.2, 2.0 ** 15 * 1.25, -1e9, np.inf], dtype=np.float32)
    c = hif8.encode_bruteforce(x)
    d = hif8.decode(c)
    assert c[0] == 0x80 and c[1] == 0 and c[2] == 0 and c[3] == 0
    assert d[4] == 2.0 ** -22 and d[5] == -2.0 ** -22          # tie between 0 and min goes away from zero
    assert d[6] == 2.0 ** -21                                   # tie goes up
    assert d[7] == 1.125 and d[8] == 1.25 and d[9] == -1.125    # ties away from zero (ulp 1/8 at E=0)
    assert d[10] == 2.0 ** 15 and np.isposinf(d[11]) and np.isneginf(d[12]) and np.isposinf(d[13])
    cs = hif8.encode_bruteforce(x, saturate=True)
    assert hif8.decode(cs)[11] == 2.0 ** 15 and hif8.decode(cs)[12] == -2.0 ** 15


def test_encode_is_nearest_on_random():
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(20000) * 10.0 ** rng.uniform(-8, 5, 20000)).astype(np.float32)
    c = hif8.encode_bruteforce(x)
    t = hif8.decode_table().astype(np.float64)
    fin = np.array([v for v in t if np.isfinite(v)])
    d = hif8.decode(c).astype(np.float64)
    ok = np.isfinite(d)
    best = np.abs(x[ok, None].astype(np.float64) - fin[None, :]).min(1)
    assert np.allclose(np.abs(x[ok] - d[ok]), best, rtol=0, atol=0)
