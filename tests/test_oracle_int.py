"""Pins for oracle/int_quant.py: hand-computed known answers (exact in fp32),
numpy float32 recomputation of the IEEE chain, the zero-pad rule, invariants."""
import numpy as np
import pytest
import torch

from oracle import int_quant as iq
from util import assert_bits_equal


def T(*v, dtype=torch.float32):
    return torch.tensor(v, dtype=dtype).reshape(-1, 1)


# ---- scale / offset known answers -----------------------------------------
def test_sym_scope_127_vs_128():
    s, z = iq.scale_offset(T(1.27), T(-1.0), True, 'int8')
    assert z is None and s.dtype == torch.float32
    assert s.item() == np.float32(1.27) / np.float32(127)
    s, _ = iq.scale_offset(T(1.0), T(-1.28), True, 'int8')
    assert s.item() == np.float32(1.28) / np.float32(128)
    # exact cases: power-of-two bounds
    s, _ = iq.scale_offset(T(127.0), T(-1.0), True, 'int8')
    assert s.item() == 1.0
    s, _ = iq.scale_offset(T(1.0), T(-128.0), True, 'int8')
    assert s.item() == 1.0
    s, _ = iq.scale_offset(T(7.0), T(-8.0), True, 'int4')
    assert s.item() == 1.0
    s, _ = iq.scale_offset(T(8.0), T(-8.0), True, 'int4')      # equal magnitudes -> 7
    assert s.item() == np.float32(8) / np.float32(7)


def test_zero_range_guard():
    s, z = iq.scale_offset(T(0.0), T(0.0), True, 'int8')
    assert s.item() == 1.0 and z is None
    s, z = iq.scale_offset(T(0.0), T(0.0), False, 'int8')
    assert s.item() == 1.0 and z.item() == -128 and z.dtype == torch.int32
    s, z = iq.scale_offset(T(0.0), T(0.0), False, 'int4')
    assert s.item() == 1.0 and z.item() == -8
    # below eps but not zero: guard still fires
    s, z = iq.scale_offset(T(1e-6), T(0.0), False, 'int8')     # 1e-6/255 < eps
    assert s.item() == 1.0 and z.item() == -128
    s, z = iq.scale_offset(T(1e-6), T(-1e-6), True, 'int8')
    assert s.item() == 1.0


def test_asym_known_answers():
    s, z = iq.scale_offset(T(1.5), T(0.0), False, 'int4')
    assert s.item() == np.float32(1.5) / np.float32(15) and z.item() == -8
    # min > 0 is clamped to 0, max < 0 is clamped to 0
    s, z = iq.scale_offset(T(255.0), T(3.0), False, 'int8')
    assert s.item() == 1.0 and z.item() == -128
    s, z = iq.scale_offset(T(-3.0), T(-255.0), False, 'int8')
    assert s.item() == 1.0 and z.item() == 127
    # tie in the offset rounding goes to even: s = 0.5, z = -128 + 0.5 = -127.5 -> -128
    s, z = iq.scale_offset(T(127.25), T(-0.25), False, 'int8')
    assert s.item() == 0.5 and z.item() == -128
    # -128 + 1.5 = -126.5 -> -126
    s, z = iq.scale_offset(T(126.75), T(-0.75), False, 'int8')
    assert s.item() == 0.5 and z.item() == -126


def test_scale_offset_matches_numpy_f32_chain():
    rng = np.random.default_rng(0)
    n = 200000
    mx = (rng.standard_normal(n) * 10 ** rng.uniform(-6, 6, n)).astype(np.float32)
    mn = (rng.standard_normal(n) * 10 ** rng.uniform(-6, 6, n)).astype(np.float32)
    mx, mn = np.maximum(mx, mn), np.minimum(mx, mn)
    for kind, b in (('int8', 8), ('int4', 4)):
        # symmetric
        s, _ = iq.scale_offset(torch.from_numpy(mx), torch.from_numpy(mn), True, kind)
        amx, amn = np.abs(mx), np.abs(mn)
        scope = np.where(amx < amn, 2 ** (b - 1), 2 ** (b - 1) - 1).astype(np.float32)
        ref = (np.where(amx > amn, amx, amn) / scope).astype(np.float32)
        ref = np.where(ref < np.float32(1.192092896e-7), np.float32(1), ref)
        assert np.array_equal(s.numpy(), ref)
        # asymmetric
        s, z = iq.scale_offset(torch.from_numpy(mx), torch.from_numpy(mn), False, kind)
        cmx, cmn = np.maximum(mx, 0), np.minimum(mn, 0)
        sc = ((cmx - cmn).astype(np.float32) / np.float32(2 ** b - 1)).astype(np.float32)
        with np.errstate(all='ignore'):
            off = (np.float32(-(2 ** (b - 1))) - (cmn / sc).astype(np.float32)).astype(np.float32)
        off = np.where(cmx != cmn, off, np.float32(-(2 ** (b - 1))))
        tiny = sc < np.float32(1.192092896e-7)
        off = np.where(tiny, np.float32(-(2 ** (b - 1))), off)
        sc = np.where(tiny, np.float32(1), sc)
        assert np.array_equal(s.numpy(), sc)
        assert np.array_equal(z.numpy(), np.rint(off).astype(np.int32))
        assert z.min() >= -(2 ** (b - 1)) and z.max() <= 2 ** (b - 1) - 1


def test_invalid_scale_raises():
    with pytest.raises(RuntimeError, match="Param scale has invalid value"):
        iq.scale_offset(T(float('inf')), T(0.0), True, 'int8')
    with pytest.raises(RuntimeError, match="Param scale has invalid value"):
        iq.scale_offset(T(float('nan')), T(0.0), False, 'int8')


# ---- min/max ---------------------------------------------------------------
def test_group_zero_pad_participates():
    w = torch.full((2, 40), 3.0)                 # K=40, g=32 -> second group has 8 values + 24 zeros
    mn, mx = iq.weight_min_max(w, 'group', 32)
    assert mn.shape == (2, 2, 1) and mx.shape == (2, 2, 1)
    assert mn[0, 0, 0] == 3.0 and mn[0, 1, 0] == 0.0 and mx[0, 1, 0] == 3.0
    w = -w
    mn, mx = iq.weight_min_max(w, 'group', 32)
    assert mx[0, 1, 0] == 0.0 and mn[0, 1, 0] == -3.0


def test_min_max_shapes():
    w = torch.randn(8, 64)
    mn, mx = iq.weight_min_max(w, 'channel')
    assert mn.shape == (8, 1) and torch.equal(mx[:, 0], w.amax(1))
    mn, mx = iq.weight_min_max(w, 'tensor')
    assert mn.shape == (1, 1) and mx.item() == w.max().item()


# ---- elementwise -----------------------------------------------------------
def test_to_codes_ties_even_and_saturation():
    t = torch.tensor([0.5, 1.5, 2.5, -0.5, -1.5, 126.5, 127.5, 300.0, -128.5, -129.5, -400.0])
    assert iq.to_codes(t, 'int8').tolist() == [0, 2, 2, 0, -2, 126, 127, 127, -128, -128, -128]
    c4 = iq.to_codes(torch.tensor([6.5, 7.5, 9.0, -7.5, -8.5, -20.0]), 'int4')
    assert c4.dtype == torch.int32 and c4.tolist() == [6, 7, 7, -8, -8, -8]
    with pytest.raises(ValueError, match="Not supported quant_dtype int2"):
        iq.to_codes(t, 'int2')


def test_variant_b_known_answer():
    q, s = iq.absmax_quant(torch.tensor([[-127.0, 63.5, 62.5]]))
    assert s.item() == 1.0 and q.tolist() == [[-127, 64, 62]]
    q, s = iq.absmax_quant(torch.tensor([[-128.0, 127.0, 1.0]]))    # clamp at -qmax
    assert q.min().item() >= -127


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kind", ['int8', 'int4'])
@pytest.mark.parametrize("sym", [True, False])
def test_fake_quant_matches_numpy_chain(dtype, kind, sym):
    g = torch.Generator().manual_seed(5)
    w = (torch.randn(16, 96, generator=g) * 0.02).to(dtype)
    s, z = iq.weight_scale_offset(w, 'channel', sym, kind)
    dq = iq.fake_quant(w, kind, s, z)
    assert dq.dtype == dtype
    b = int(kind[3:])
    wf = w.float().numpy()
    t = (wf / s.numpy()).astype(np.float32)
    if z is not None:
        t = (t + z.numpy().astype(np.float32)).astype(np.float32)
    q = np.clip(np.rint(t), -(2 ** (b - 1)), 2 ** (b - 1) - 1)
    codes = iq.quant_codes(w, kind, s, z)
    assert np.array_equal(codes.numpy().astype(np.float32), q)
    if z is not None:
        q = (q - z.numpy().astype(np.float32)).astype(np.float32)
    ref = torch.from_numpy((q * s.numpy()).astype(np.float32)).to(dtype)
    assert torch.equal(dq, ref)
    # invariants
    assert codes.min() >= -(2 ** (b - 1)) and codes.max() <= 2 ** (b - 1) - 1
    if dtype == torch.float32:
        # scope 128 rows can clip their largest positive value by one step
        assert ((w - dq).abs() <= s * (1.0001 if sym else 0.50001)).all()
        # idempotent given the same factors
        assert torch.equal(iq.fake_quant(dq, kind, s, z), dq)


def test_fake_quant_group_ragged():
    g = torch.Generator().manual_seed(6)
    w = torch.randn(4, 80, generator=g)
    s, z = iq.weight_scale_offset(w, 'group', False, 'int4', 32)
    assert s.shape == (4, 3, 1) and z.shape == (4, 3, 1)
    dq = iq.fake_quant(w, 'int4', s, z, 32)
    assert dq.shape == w.shape
    # group 2 has 16 real columns: recompute by hand with zeros appended
    blk = torch.cat([w[:, 64:], torch.zeros(4, 16)], 1)
    s2, z2 = iq.scale_offset(blk.amax(1, keepdim=True), blk.amin(1, keepdim=True), False, 'int4')
    assert torch.equal(s2, s[:, 2]) and torch.equal(z2, z[:, 2])


def test_awq_path_differs_only_by_the_cast():
    g = torch.Generator().manual_seed(7)
    w = (torch.randn(8, 64, generator=g) * 0.05).to(torch.bfloat16)
    s, z = iq.weight_scale_offset(w, 'group', False, 'int4', 32)
    a = iq.awq_fake_quant(w, 'int4', s, z, 'group', 32)
    b = iq.fake_quant(w, 'int4', s, z, 32)
    assert a.dtype == b.dtype == torch.bfloat16 and a.shape == b.shape
    # on fp32 weights the cast is the identity, so both paths agree exactly
    wf = w.float()
    s, z = iq.weight_scale_offset(wf, 'channel', True, 'int8')
    assert torch.equal(iq.awq_fake_quant(wf, 'int8', s, z, 'channel'), iq.fake_quant(wf, 'int8', s, z))
    # a value that the cast moves across a rounding boundary: bf16 w = 3.5, fp32 s = 1.0003 -> w/s = 3.49895,
    # which rounds to 3 in fp32 but is 3.5 once narrowed to bf16 and then rounds (half to even) to 4
    wv = torch.tensor([[3.5, 100.0]], dtype=torch.bfloat16)
    s1 = torch.tensor([[1.0003]])
    assert torch.round(wv.float() / s1)[0, 0].item() == 3.0
    assert iq.quant_codes(wv, 'int8', s1)[0, 0].item() == 3
    assert iq.fake_quant(wv, 'int8', s1)[0, 0].item() == torch.tensor(3 * 1.0003).to(torch.bfloat16).item()
    assert iq.awq_fake_quant(wv, 'int8', s1, None, 'channel')[0, 0].item() == \
        torch.tensor(4 * 1.0003).to(torch.bfloat16).item()


def test_dynamic_token_quant():
    g = torch.Generator().manual_seed(8)
    x = torch.randn(12, 128, generator=g).to(torch.bfloat16)
    x[3] = 0
    q, s = iq.dynamic_token_quant(x)
    assert q.dtype == torch.int8 and s.shape == (12,) and s[3].item() == 1.0 and q[3].abs().max() == 0
    xf = x.float()
    for m in range(12):
        amx, amn = xf[m].max().abs().item(), xf[m].min().abs().item()
        scope = 128 if amx < amn else 127
        sm = np.float32(max(amx, amn)) / np.float32(scope) if max(amx, amn) > 0 else np.float32(1)
        assert s[m].item() == sm
    q2, s2 = iq.dynamic_token_quant_absmax(x)
    assert s2[3].item() == 1.0 and q2.dtype == torch.int8


def test_static_quantize_axes():
    x = torch.tensor([[1.0, 2.5, -3.5], [100.0, -100.0, 0.25]], dtype=torch.bfloat16)
    q = iq.static_quantize(x, torch.tensor([1.0], dtype=torch.bfloat16), torch.tensor([0.0], dtype=torch.bfloat16), -1)
    assert q.tolist() == [[1, 2, -4], [100, -100, 0]]
    q = iq.static_quantize(x, torch.tensor([2.0, 4.0], dtype=torch.bfloat16),
                           torch.tensor([1.0, 0.0], dtype=torch.bfloat16), -2)
    assert q.tolist() == [[3, 6, -6], [127, -128, 1]]


def test_oracle_matches_exact_arithmetic_fixture():
    """tests/golden/int_quant_kat.json holds the whole chain computed with exact fractions and an explicit
    round-to-nearest-even to binary32 after every operation (no floating-point library involved): scale,
    offset, codes and dequantised values must agree bit for bit."""
    from util import load_int_quant_kat
    cases = load_int_quant_kat()
    assert len(cases) >= 70
    for bits, sym, w, scale, offset, codes, dq in cases:
        kind = 'int%d' % bits
        s, z = iq.weight_scale_offset(w, 'channel', sym, kind)
        assert_bits_equal(s.reshape(()), scale, "scale")
        if sym:
            assert z is None
        else:
            assert int(z.reshape(())) == offset
        got_codes = iq.quant_codes(w, kind, s, z)
        assert torch.equal(got_codes.to(torch.int32), codes)
        assert_bits_equal(iq.fake_quant(w, kind, s, z), dq, "dq")


def test_oracle_matches_exact_arithmetic_fixture_16bit_group_awq():
    """tests/golden/int_quant_kat16.json: the same exact-fraction model for bf16 / fp16 / fp32 sources, factors per
    group (ragged last group zero-padded) and the cast-before-round variant of the AWQ search."""
    from util import load_int_quant_kat16
    cases = load_int_quant_kat16()
    assert len(cases) >= 130
    differs = 0
    for c in cases:
        kind = 'int%d' % c["bits"]
        w, g, sym = c["w"], c["group"], c["symmetric"]
        strat = 'group' if g else 'channel'
        s, z = iq.weight_scale_offset(w, strat, sym, kind, g or None)
        assert_bits_equal(s.reshape(-1), c["scale"], "scale")
        if sym:
            assert z is None
        else:
            assert torch.equal(z.reshape(-1), c["offset"])
        codes = iq.quant_codes(w, kind, s, z, g or None).reshape(1, -1)[:, :w.shape[1]]
        assert torch.equal(codes.to(torch.int32), c["codes"])
        assert_bits_equal(iq.fake_quant(w, kind, s, z, g or None), c["dq"], "dq")
        assert_bits_equal(iq.awq_fake_quant(w, kind, s, z, strat, g or None), c["awq_dq"], "awq dq")
        differs += int(not torch.equal(c["dq"], c["awq_dq"]))
    assert differs >= 20                                  # the file does separate the two paths


def test_dynamic_token_quant_absmax_known_answers():
    """The experimental tree's per-token form (node.py:39-43,181-204): s = absmax / 127 with s = 1 for a dead row,
    q = clamp(rne(x / s), -128, 127).  Rows whose absmax is 127 * 2^k have a power-of-two scale, so every quotient
    and tie is exact in fp32."""
    x = torch.tensor([[127.0, -63.5, 62.5, 0.5, -0.5, 1.5, -127.0, 0.0],
                      [-254.0, 3.0, 1.0, -1.0, 5.0, 7.0, 253.0, 2.0],
                      [0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0],
                      [-31.75, 0.125, 0.375, 0.625, -0.125, -0.375, 31.5, 0.25]], dtype=torch.float32)
    q, s = iq.dynamic_token_quant_absmax(x)
    assert s.tolist() == [1.0, 2.0, 1.0, 0.25]
    assert q.dtype == torch.int8
    assert q.tolist() == [[127, -64, 62, 0, 0, 2, -127, 0],
                          [-127, 2, 0, 0, 2, 4, 126, 1],
                          [0, 0, 0, 0, 0, 0, 0, 0],
                          [-127, 0, 2, 2, 0, -2, 126, 1]]
    # the positive extremum never produces -128, the negative one never exceeds -127 (absmax rule, no 128 scope)
    xb = torch.tensor([[-1.0, 0.999]], dtype=torch.bfloat16)
    qb, sb = iq.dynamic_token_quant_absmax(xb)
    assert sb.dtype == torch.bfloat16 and qb[0, 0].item() == -127 and qb[0, 1].item() == 127
    # the AMCT rule on the same row uses scope 128 where the negative extremum dominates
    qa, sa = iq.dynamic_token_quant(x[1:2])
    assert sa.item() == 254.0 / 128 and qa[0, 0].item() == -128


def test_awq_search_special_cases():
    """Closed-form cases of the scale search: one grid point means ratio 0, whose scale is all ones, and the
    grid step then is the plain AWQ fake-quant; equal-magnitude inputs give an all-ones scale at every ratio, so
    every grid point has the same loss and the first one wins; non-finite data raises like the reference."""
    torch.manual_seed(3)
    x = torch.randn(16, 64)
    w = [torch.randn(24, 64) * 0.05]
    fwd = lambda inp, ws: inp @ ws[0].t()
    s, losses = iq.awq_search_scale(x, w, fwd, 1, 'int4', 'group', False, 32)
    assert torch.equal(s, torch.ones(1, 64))
    sc, off = iq.weight_scale_offset(w[0], 'group', False, 'int4', 32)
    dq = iq.awq_fake_quant(w[0], 'int4', sc, off, 'group', 32)
    assert abs(losses[0] - float((fwd(x, w) - fwd(x, [dq])).float().pow(4).mean())) == 0.0
    xs = torch.sign(torch.randn(16, 64)) * 0.5                        # mean|x| identical in every channel
    s, losses = iq.awq_search_scale(xs, w, fwd, 5, 'int4', 'group', False, 32)
    assert torch.equal(s, torch.ones(1, 64)) and len(set(losses)) == 1
    bad = x.clone()
    bad[1, 2] = float('inf')
    with pytest.raises(RuntimeError, match="Invalid value"):
        iq.awq_search_scale(bad, w, fwd, 2, 'int4', 'group', False, 32)


def test_channel_stats_known_answers():
    """Column statistics: hand-checkable values, the running update over two batches, a NaN batch value
    that the update ignores (NaN > x is false), and the smoothing factor's closed forms (strength 1 gives
    act_max, strength 0 gives 1 / wts_max, non-positive or non-finite factors become 1)."""
    x1 = torch.tensor([[1.0, -2.0, 0.5], [3.0, -1.0, float('nan')]])
    dmax = torch.full((1, 3), float('-inf'))
    dmin = torch.full((1, 3), float('inf'))
    dmax, dmin = iq.channel_min_max_update(x1, dmax, dmin)
    assert dmax.tolist() == [[3.0, -1.0, float('-inf')]] and dmin.tolist() == [[1.0, -2.0, float('inf')]]
    x2 = torch.tensor([[[2.0, -5.0, 0.25]], [[-4.0, 0.0, 0.75]]])          # rank 3: all leading dims are tokens
    dmax, dmin = iq.channel_min_max_update(x2, dmax, dmin)
    assert dmax.tolist() == [[3.0, 0.0, 0.75]] and dmin.tolist() == [[-4.0, -5.0, 0.25]]
    w = torch.tensor([[0.5, -4.0, 0.0], [-2.0, 1.0, 0.0]])
    act = torch.tensor([[4.0, 9.0, 1.0]])
    assert torch.equal(iq.smooth_factor(act, w, 1.0), act)
    assert torch.equal(iq.smooth_factor(act, w, 0.0)[:, :2], torch.tensor([[0.5, 0.25]]))
    assert torch.equal(iq.smooth_factor(act, w, 0.5), torch.tensor([[2.0 / 2.0 ** 0.5, 1.5, 1.0]]))   # x / 0 -> inf -> 1


def test_interchange_known_answers():
    """fp8 block dequant, pair packing and scale widening on values whose results are known exactly."""
    from oracle import deploy as od
    codes = torch.tensor([[0x38, 0xB8, 0x40, 0x01], [0x7E, 0x00, 0x80, 0x30]], dtype=torch.uint8)   # 1, -1, 2, 2^-9; 448, 0, -0, 0.5
    w = codes.view(torch.float8_e4m3fn)
    scale = torch.tensor([[0.5, 4.0]])
    out = od.fp8_block_dequant(w, scale, block_size=2, out_dtype=torch.float32)
    assert out.tolist() == [[0.5, -0.5, 8.0, 2.0 ** -7], [224.0, 0.0, -0.0, 2.0]]
    x = torch.tensor([[5, -7], [-8, 7], [0, 1], [-1, -2]], dtype=torch.int8)
    y = od.pack_4bit(x)
    # rows (0,1) -> (x1 << 4) | (x0 & 15): 5,-8 -> 0x85 ; -7,7 -> 0x79 ; rows (2,3): 0,-1 -> 0xF0 ; 1,-2 -> 0xE1
    assert y.view(torch.uint8).tolist() == [[0x85, 0x79], [0xF0, 0xE1]]
    s = torch.tensor([[1.0, -2.0]])
    assert od.scale_fp32_to_u64(s).tolist() == [[0x3F800000, 0xC0000000]]


def test_gptq_block_loop_against_scalar_model():
    """The block loop restated with numpy float32 scalars, one rounding per operation written out, and the
    invariant that a finished column holds w - err * d."""
    from oracle import gptq as og
    rng = np.random.default_rng(4)
    n, count = 5, 7
    w0 = (rng.standard_normal((n, count)) * 0.1).astype(np.float32)
    a = rng.standard_normal((count, count)).astype(np.float32)
    hinv = np.triu(a * 0.1 + np.eye(count, dtype=np.float32))
    for sym in (True, False):
        wt = torch.from_numpy(w0.copy())
        s, z = iq.weight_scale_offset(wt, 'channel', sym, 'int4')
        got_w, got_e = og.block_loop(wt.clone(), torch.from_numpy(hinv), 'int4', [s.reshape(-1, 1)] * count,
                                     None if z is None else [z.reshape(-1, 1)] * count)
        w = w0.copy()
        e = np.zeros_like(w)
        sn = s.numpy().reshape(-1)
        zn = None if z is None else z.numpy().reshape(-1).astype(np.float32)
        for i in range(count):
            for r in range(n):
                t = np.float32(w[r, i] / sn[r])
                if zn is not None:
                    t = np.float32(t + zn[r])
                q = np.float32(min(max(np.rint(t), -8), 7))
                wq = np.float32(np.float32(q - (zn[r] if zn is not None else np.float32(0))) * sn[r])
                err = np.float32(np.float32(w[r, i] - wq) / hinv[i, i])
                e[r, i] = err
                for j in range(i, count):
                    w[r, j] = np.float32(w[r, j] - np.float32(err * hinv[i, j]))
        assert np.array_equal(got_w.numpy().view(np.uint32), w.view(np.uint32))
        assert np.array_equal(got_e.numpy().view(np.uint32), e.view(np.uint32))


def test_awq_loss_closed_forms():
    """oracle.int_quant.awq_loss against what the expression fixes: constant difference, one non-zero
    difference, sign symmetry, the rounding of the difference to the dtype, and torch's own evaluation of the
    reference's expression (awq.py:96)."""
    n = 1000
    a = torch.full((n,), 3.0)
    assert iq.awq_loss(a, a - 0.5) == 0.5 ** 4
    assert iq.awq_loss(a - 0.5, a) == 0.5 ** 4
    b = a.clone()
    b[17] += 2.0
    assert iq.awq_loss(a, b) == 16.0 / n
    # bf16: 512 - 1 = 511 is not a bf16 value (8 significant bits): the difference is rounded to 512 first
    y, yh = torch.tensor([512.0], dtype=torch.bfloat16), torch.tensor([1.0], dtype=torch.bfloat16)
    assert iq.awq_loss(y, yh) == 512.0 ** 4
    g = torch.Generator().manual_seed(5)
    for dt in (torch.float32, torch.float16, torch.bfloat16):
        y = torch.randn(64, 96, generator=g).to(dt)
        yh = (y.float() + 0.1 * torch.randn(64, 96, generator=g)).to(dt)
        ref = float((y - yh).float().pow(4).mean())
        assert abs(iq.awq_loss(y, yh) - ref) <= 1e-5 * ref
    assert iq.awq_loss(torch.zeros(0), torch.zeros(0)) != iq.awq_loss(torch.zeros(0), torch.zeros(0))   # NaN
