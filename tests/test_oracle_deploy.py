"""CPU pins of the deploy-path oracle (oracle/deploy.py): the functions the GPU parity tests of the two quantized Linears
lean on are checked here, without a GPU, against scalar loops written out operation by operation (Python integers,
Fractions and numpy float32), against known answers and through round trips -- so that a mistake in the oracle (a
transposed operand, a dropped bias, the wrong nibble, a rounding in the wrong place) fails on the CPU."""
from fractions import Fraction

import numpy as np
import torch

from oracle import deploy as od


def bf16_round(v):
    """Round-to-nearest-even of a Python float to bfloat16, written out on the binary32 bits."""
    b = int(np.float32(v).view(np.uint32))
    b = (b + 0x7FFF + ((b >> 16) & 1)) & 0xFFFF0000
    return float(np.uint32(b).view(np.float32))


def f16_round(v):
    return float(np.float16(np.float32(v)))


def case_w8a8(M, N, K, seed, per_token, bias_kind):
    g = torch.Generator().manual_seed(seed)
    xq = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int16).to(torch.int8)
    wq = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int16).to(torch.int8)
    s_ch = 1e-3 + 9e-3 * torch.rand(N, generator=g)
    s_tok = (0.01 + torch.rand(M, generator=g)) if per_token else None
    bias = None
    if bias_kind == 'int':
        bias = torch.randint(-5000, 5000, (N,), generator=g, dtype=torch.int32)
    elif bias_kind == 'float':
        bias = torch.randn(N, generator=g)
    return xq, wq, s_ch, s_tok, bias


def test_int8_matmul_exact_against_integer_loops():
    """Python integers cannot round: the fp64 matmul of the oracle must give the same sums, extremes included."""
    for M, N, K, seed in ((3, 5, 7, 1), (2, 4, 64, 2), (1, 1, 4096, 3)):
        xq, wq, _, _, _ = case_w8a8(M, N, K, seed, False, None)
        if K == 4096:                                # the largest magnitude an accumulator can reach
            xq[:] = -128
            wq[:] = -128
        got = od.int8_matmul_exact(xq, wq.t())
        for m in range(M):
            for n in range(N):
                want = sum(int(xq[m, k]) * int(wq[n, k]) for k in range(K))
                assert int(got[m, n]) == want
    assert int(od.int8_matmul_exact(torch.full((1, 4096), -128, dtype=torch.int8), torch.full((4096, 1), -128, dtype=torch.int8))) == 4096 * 16384


def test_quant_matmul_epilogue_against_a_float32_loop():
    """acc (+ int32 bias) -> fp32 -> * s_ch[n] -> * s_tok[m] -> + float bias -> one rounding to the output dtype, each
    step a separate numpy float32 operation on Python-integer accumulators."""
    for per_token, bias_kind, odt in ((True, 'float', torch.bfloat16), (False, 'int', torch.float16), (True, None, torch.float32),
                                      (False, 'float', torch.bfloat16), (True, 'int', torch.bfloat16)):
        M, N, K = 4, 6, 40
        xq, wq, s_ch, s_tok, bias = case_w8a8(M, N, K, 10 + M, per_token, bias_kind)
        got = od.quant_matmul(xq, wq.t(), s_ch, s_tok, bias, odt)
        assert got.dtype == odt and got.shape == (M, N)
        for m in range(M):
            for n in range(N):
                acc = sum(int(xq[m, k]) * int(wq[n, k]) for k in range(K))
                if bias_kind == 'int':
                    acc += int(bias[n])
                f = np.float32(acc)
                f = np.float32(f * np.float32(s_ch[n].item()))
                if per_token:
                    f = np.float32(f * np.float32(s_tok[m].item()))
                if bias_kind == 'float':
                    f = np.float32(f + np.float32(bias[n].item()))
                want = torch.tensor(float(f), dtype=torch.float32).to(odt)
                assert got[m, n].item() == want.item(), (per_token, bias_kind, odt, m, n)
        # the fp64 anchor is the same expression without the intermediate roundings
        f64 = od.quant_matmul_f64(xq, wq.t(), s_ch, s_tok, bias)
        ulp = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -23}[odt]
        assert ((got.double() - f64).abs() <= f64.abs() * (ulp + 3 * 2.0 ** -24) + 1e-30).all()


def test_quant_matmul_leading_dims_share_the_token_scales():
    xq, wq, s_ch, s_tok, _ = case_w8a8(6, 5, 16, 21, True, None)
    flat = od.quant_matmul(xq, wq.t(), s_ch, s_tok.repeat(1)[:3].repeat(2), None, torch.bfloat16)
    batched = od.quant_matmul(xq.reshape(2, 3, 16), wq.t(), s_ch, s_tok[:3], None, torch.bfloat16)
    assert batched.shape == (2, 3, 5) and torch.equal(batched.reshape(6, 5), flat)


def w4_case(N, K, group, seed, sdt):
    g = torch.Generator().manual_seed(seed)
    codes = torch.randint(-8, 8, (N, K), generator=g, dtype=torch.int32)
    scales = (1e-3 + 9e-3 * torch.rand(N, K // group, generator=g)).to(sdt)
    anti = torch.randint(-7, 9, (N, K // group), generator=g).float()           # antiquant_offset = -offset_w
    return codes, scales, anti


def test_dequant_weight_both_readings_against_fractions():
    """(q + antiquant_offset) * antiquant_scale per group: exact as a Fraction; the rounded reading is ONE rounding of
    that exact value to the 16-bit type."""
    for sdt, dt, rnd in ((torch.float16, torch.bfloat16, bf16_round), (torch.bfloat16, torch.bfloat16, bf16_round),
                         (torch.float16, torch.float16, f16_round)):
        N, K, group = 3, 64, 32
        codes, scales, anti = w4_case(N, K, group, 31, sdt)
        exact = od.dequant_weight(codes, scales, anti, group, None)
        rounded = od.dequant_weight(codes, scales, anti, group, dt)
        assert exact.dtype == torch.float64 and rounded.dtype == dt
        for n in range(N):
            for k in range(K):
                gi = k // group
                want = (Fraction(int(codes[n, k])) + Fraction(anti[n, gi].item())) * Fraction(scales[n, gi].item())
                assert Fraction(exact[n, k].item()) == want
                assert rounded[n, k].item() == rnd(float(want)), (sdt, dt, n, k)
    # symmetric weights (no offset) and per-channel factors (group 0 = the whole row)
    codes, scales, _ = w4_case(2, 32, 32, 32, torch.float16)
    e = od.dequant_weight(codes, scales, None, 0, None)
    assert torch.equal(e, codes.double() * scales.double())


def test_w4a16_forward_against_a_scalar_loop():
    """x' = dt(x * scale_factor); y = sum_k x'_k * w_k + bias with exact products: Fractions, both readings."""
    M, N, K, group = 3, 4, 64, 32
    g = torch.Generator().manual_seed(41)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    sf = (0.5 + torch.rand(1, K, generator=g)).to(torch.bfloat16)
    bias = torch.randn(N, generator=g)
    codes, scales, anti = w4_case(N, K, group, 42, torch.float16)
    for round_weight in (False, True):
        got = od.w4a16_forward_f64(x, codes, scales, anti, group, bias, sf, round_weight=round_weight)
        for m in range(M):
            for n in range(N):
                tot = Fraction(bias[n].item())
                for k in range(K):
                    xs = bf16_round(float(np.float32(x[m, k].item()) * np.float32(sf[0, k].item())))
                    w = (Fraction(int(codes[n, k])) + Fraction(anti[n, k // group].item())) * Fraction(scales[n, k // group].item())
                    if round_weight:
                        w = Fraction(bf16_round(float(w)))
                    tot += Fraction(xs) * w
                assert abs(got[m, n].item() - float(tot)) <= 1e-12 * max(1.0, abs(float(tot)))
    # leading dims are flattened and restored
    y3 = od.w4a16_forward_f64(x.reshape(1, M, K), codes, scales, anti, group)
    assert y3.shape == (1, M, N)


def test_error_bounds_of_the_rounded_reading():
    """hard = u * sum |x' w| bounds the move of the output for ANY rounding of the weights (checked with the actual
    bf16 / fp16 rounding and with the adversarial choice, which attains it); likely = 7 u sqrt(sum (x' w)^2)."""
    M, N, K, group = 5, 7, 256, 64
    g = torch.Generator().manual_seed(51)
    codes, scales, anti = w4_case(N, K, group, 52, torch.float16)
    w = od.dequant_weight(codes, scales, anti, group, None)
    for dt, u in ((torch.bfloat16, 2.0 ** -8), (torch.float16, 2.0 ** -11)):
        x = torch.randn(M, K, generator=g).to(dt)
        hard, likely = od.weight_only_error_bounds(x, w)
        exact = x.double() @ w.t()
        actual = x.double() @ w.to(dt).double().t()
        assert ((actual - exact).abs() <= hard).all()
        assert ((actual - exact).abs() <= likely).all()
        # the relative rounding error of every weight is within u
        nz = w != 0
        assert ((w.to(dt).double() - w).abs()[nz] <= u * w.abs()[nz]).all()
        # adversarial: every weight moved by u in the direction that helps -> the hard bound, exactly
        for m in range(2):
            for n in range(2):
                worst = sum(abs(x[m, k].item() * w[n, k].item()) * u for k in range(K))
                assert abs(hard[m, n].item() - worst) <= 1e-12 * worst
                rss = 7 * u * sum((x[m, k].item() * w[n, k].item()) ** 2 for k in range(K)) ** 0.5
                assert abs(likely[m, n].item() - rss) <= 1e-12 * rss


def test_int4_word_packing_known_answers_and_round_trip():
    """Little-endian nibbles: column 8 i + j of a row in bits 4 j .. 4 j + 3 of word i, two's complement nibbles."""
    row = torch.tensor([[0, 1, 2, 3, 4, 5, 6, 7, -8, -7, -6, -5, -4, -3, -2, -1]], dtype=torch.int32)
    words = od.pack_int4_words(row)
    assert words.dtype == torch.int32 and words.shape == (1, 2)
    assert int(words[0, 0]) == 0x76543210
    assert int(words[0, 1]) & 0xFFFFFFFF == 0xFEDCBA98 and int(words[0, 1]) < 0          # the top nibble sets the sign bit
    assert torch.equal(od.unpack_int4_words(words), row)
    g = torch.Generator().manual_seed(61)
    codes = torch.randint(-8, 8, (9, 64), generator=g, dtype=torch.int32)
    assert torch.equal(od.unpack_int4_words(od.pack_int4_words(codes)), codes)
    # one nibble at a time: a single non-zero code lands in exactly its nibble
    for j in range(8):
        one = torch.zeros(1, 8, dtype=torch.int32)
        one[0, j] = 5
        assert int(od.pack_int4_words(one)[0, 0]) == 5 << (4 * j)


def test_k_major_nibble_layout_known_answers_and_round_trip():
    """The deploy layout of this repo: unsigned code + 8, even k in the low nibble of byte k / 2."""
    row = torch.tensor([[-8, 7, 0, -1]], dtype=torch.int32)
    packed = od.pack_nibbles_k(row)
    assert packed.dtype == torch.uint8 and packed.tolist() == [[0x0 | (15 << 4), 8 | (7 << 4)]]
    assert torch.equal(od.unpack_nibbles_k(packed), row)
    g = torch.Generator().manual_seed(62)
    codes = torch.randint(-8, 8, (5, 128), generator=g, dtype=torch.int32)
    assert torch.equal(od.unpack_nibbles_k(od.pack_nibbles_k(codes)), codes)
    # the two layouts hold the same codes: [N,K] nibbles <-> [K,N/8] words of the transposed matrix
    n8 = torch.randint(-8, 8, (16, 32), generator=g, dtype=torch.int32)
    assert torch.equal(od.unpack_int4_words(od.pack_int4_words(n8.t().contiguous())).t(), od.unpack_nibbles_k(od.pack_nibbles_k(n8)))
