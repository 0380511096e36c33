"""Tensors beyond 2^31 elements and 4 GiB: every index of the kernels must be 64 bits wide where it has to be, and the
GEMM dispatch must keep operands of that size away from the kernels that address with 32-bit lane offsets.

A reference result for 2 * 10^9 elements is out of reach of a CPU oracle, so these tests use a property that does
not depend on the size: every kernel here works row by row (or column by column, for the Linears), so the rows of the
big call must equal, bit for bit, what the same entry point returns for a small tensor that holds only those rows --
and the small shapes are what the other test files pin against the oracle.  The sampled rows straddle the places where
a 32-bit element index (2^31) and a 32-bit byte offset (2^32) wrap.

Every buffer a kernel reads or writes lies in the MIDDLE of a much larger allocation: an index that wrapped, or went
negative, then lands inside memory this test owns and shows up as a wrong value, not as a memory fault.  The calls go
through the C ABI directly, because the Python wrappers allocate their outputs themselves."""
import math

import pytest
import torch

from amct_amd import _lib, ops
from util import check_weight_only

pytestmark = pytest.mark.gpu

GUARD = 9 << 30                                      # bytes on either side of a buffer: +-2^31 elements of 4 bytes, and more
NEED_FREE = 200 << 30


@pytest.fixture()
def big(dev):
    free, _ = torch.cuda.mem_get_info(dev)
    if free < NEED_FREE:
        pytest.skip("needs {} GiB of free device memory, {} GiB are free".format(NEED_FREE >> 30, free >> 30))
    ops.release_workspaces()
    yield dev
    torch.cuda.synchronize(dev)
    torch.cuda.empty_cache()


def banded(shape, dtype, dev):
    """An uninitialised tensor of this shape in the middle of an allocation with GUARD bytes before and behind it."""
    n = math.prod(shape) * torch.empty((), dtype=dtype).element_size()
    raw = torch.empty(2 * GUARD + n + 512, dtype=torch.uint8, device=dev)
    off = GUARD + (-(raw.data_ptr() + GUARD)) % 256
    return raw[off:off + n].view(dtype).reshape(shape)


def stream(dev):
    return torch.cuda.current_stream(dev).cuda_stream


def call(fn, *args):
    _lib.check(fn(*[a.data_ptr() if isinstance(a, torch.Tensor) else a for a in args]))


R, C = 65536 + 16, 32768                             # 2^31 + 2^19 elements; row 65536 starts at element 2^31 (byte 2^32 for 16 bits)
ROWS = [0, 1, 32767, 32768, 65535, 65536, 65537, R - 1]


def same(a, b, what):
    assert a.dtype == b.dtype and a.shape == b.shape, what
    if a.dtype in (torch.float32, torch.float16, torch.bfloat16):
        it = {4: torch.int32, 2: torch.int16}[a.element_size()]
        a, b = a.contiguous().view(it), b.contiguous().view(it)
    assert torch.equal(a, b), what


def test_int8_fakequant_beyond_2g_elements(big):
    """K1 on bf16 [65552, 32768], int8 symmetric per channel, with codes: the sampled rows of the dequantised tensor, of
    the codes and of the scales equal the call on those rows alone."""
    dev, lib = big, _lib.load()
    x = banded((R, C), torch.bfloat16, dev).normal_()
    dq = banded((R, C), torch.bfloat16, dev)
    codes = banded((R, C), torch.int8, dev)
    scale = banded((R,), torch.float32, dev)
    call(lib.amct_fakequant_int, x, dq, codes, _lib.CODES_I8, scale, None, None, None, _lib.COL_NONE, R, C, 0, 8, 1,
         _lib.SCOPE_AMCT, -128, 127, 0, _lib.BF16, stream(dev))
    sdq, scodes, sscale, _ = ops.fakequant_int(x[ROWS].contiguous(), 8, True, codes_kind=_lib.CODES_I8)
    same(dq[ROWS], sdq, "dequantised rows")
    same(codes[ROWS], scodes, "codes")
    same(scale[ROWS], sscale, "scales")


def test_int4_group_pack_beyond_2g_elements(big):
    """K2 on the same shape, asymmetric groups of 128 (16.8 million groups): packed nibbles, fp16 scales, zero-points."""
    dev, lib = big, _lib.load()
    x = banded((R, C), torch.bfloat16, dev).normal_()
    packed = banded((R, C // 2), torch.uint8, dev)
    s16 = banded((R, C // 128), torch.float16, dev)
    zeros = banded((R, C // 128), torch.uint8, dev)
    call(lib.amct_quant_int4_group_pack, x, packed, s16, _lib.F16, None, zeros, None, None, _lib.COL_NONE, R, C, 128, 0,
         _lib.BF16, stream(dev))
    sp, ss, sz, _ = ops.quant_int4_group_pack(x[ROWS].contiguous(), 128, scale_dtype=torch.float16)
    same(packed[ROWS], sp, "packed nibbles")
    same(s16[ROWS], ss, "scales")
    same(zeros[ROWS], sz, "zero-points")


@pytest.mark.parametrize("fmt", [_lib.MX_E4M3, _lib.MX_E2M1])
def test_mx_quant_and_dequant_beyond_2g_elements(big, fmt):
    dev, lib = big, _lib.load()
    x = banded((R, C), torch.bfloat16, dev).normal_()
    ecols = C if fmt == _lib.MX_E4M3 else C // 2
    el = banded((R, ecols), torch.uint8, dev)
    e8 = banded((R, C // 32), torch.uint8, dev)
    y = banded((R, C), torch.bfloat16, dev)
    call(lib.amct_mx_quant, x, el, e8, R, C, fmt, _lib.MX_FLOOR, _lib.BF16, stream(dev))
    call(lib.amct_mx_dequant, el, e8, y, R, C, fmt, _lib.BF16, stream(dev))
    sel, se8 = ops.mx_quant(x[ROWS].contiguous(), fmt)
    same(el[ROWS], sel, "element codes")
    same(e8[ROWS], se8, "shared exponents")
    same(y[ROWS], ops.mx_dequant(sel, se8, fmt, torch.bfloat16), "dequantised rows")


def test_hif8_beyond_2g_elements(big):
    dev, lib = big, _lib.load()
    n = R * C
    x = banded((n,), torch.bfloat16, dev).normal_()
    c = banded((n,), torch.uint8, dev)
    y = banded((n,), torch.bfloat16, dev)
    call(lib.amct_hif8_encode, x, c, n, _lib.BF16, 0, stream(dev))
    call(lib.amct_hif8_decode, c, y, n, _lib.BF16, stream(dev))
    for lo in (0, (1 << 31) - 4096, (1 << 31), n - 8192):
        sc = ops.hif8_encode(x[lo:lo + 8192].clone())
        same(c[lo:lo + 8192], sc, "codes at {}".format(lo))
        same(y[lo:lo + 8192], ops.hif8_decode(sc, torch.bfloat16), "decoded values at {}".format(lo))


def test_per_token_quantise_beyond_2g_elements(big):
    """K3 on [65552, 32768] bf16 with a smoothing vector: codes and scales of the sampled tokens."""
    dev, lib = big, _lib.load()
    x = banded((R, C), torch.bfloat16, dev).normal_()
    smooth = (0.5 + torch.rand(C, device=dev)).to(torch.bfloat16)
    q = banded((R, C), torch.int8, dev)
    scale = banded((R,), torch.float32, dev)
    call(lib.amct_act_quant_per_token_int8, x, smooth, q, scale, R, C, 0, _lib.BF16, stream(dev))
    sq, ss = ops.act_quant_per_token_int8(x[ROWS].contiguous(), smooth)
    same(q[ROWS], sq, "codes")
    same(scale[ROWS], ss.reshape(-1), "scales")


def test_column_statistics_beyond_2g_elements(big):
    """N2 on [1048592, 2048] bf16: per-column maximum and minimum over all rows against torch's own reduction."""
    dev, lib = big, _lib.load()
    rows, cols = (1 << 20) + 16, 2048
    x = banded((rows, cols), torch.bfloat16, dev).normal_()
    x[rows - 1, 5] = 77.0                              # extremes that only the rows beyond 2^31 elements hold
    x[rows - 3, 9] = -88.0
    cmax = banded((cols,), torch.float32, dev)
    cmin = banded((cols,), torch.float32, dev)
    wsb = lib.amct_col_minmax_workspace_bytes(rows, cols)
    ws = banded((wsb,), torch.uint8, dev)
    call(lib.amct_col_minmax, x, cmax, cmin, rows, cols, 0, 0, _lib.BF16, ws, wsb, stream(dev))
    assert float(cmax[5]) == 77.0 and float(cmin[9]) == -88.0
    want_max = torch.stack([x[i:i + 65536].amax(dim=0) for i in range(0, rows, 65536)]).amax(dim=0).float()
    want_min = torch.stack([x[i:i + 65536].amin(dim=0) for i in range(0, rows, 65536)]).amin(dim=0).float()
    same(cmax, want_max, "column maxima")
    same(cmin, want_min, "column minima")


def col_sample(N, step):
    """Column indices at the start, around the row whose weights start at byte 2^32 (index `step`), and at the end."""
    idx = list(range(0, 32)) + list(range(step - 32, step + 32)) + list(range(N - 32, N))
    return torch.tensor(idx)


@pytest.mark.parametrize("M", [16, 48, 320])
def test_w8a8_weight_beyond_4gib(big, M):
    """K6 with W [1048640, 4096] int8 (2^32 + 2^18 bytes): the output columns around the first weight row beyond 4 GiB,
    and the first and last ones, equal the call on those weight rows alone (integer accumulation: bit for bit whatever
    kernel either call takes)."""
    dev, lib = big, _lib.load()
    N, K = (1 << 20) + 64, 4096
    g = torch.Generator(device=dev).manual_seed(7)
    wq = banded((N, K), torch.int8, dev)
    for i in range(0, N, 65536):
        wq[i:i + 65536] = torch.randint(-128, 128, wq[i:i + 65536].shape, generator=g, device=dev, dtype=torch.int8)
    xq = banded((M, K), torch.int8, dev)
    xq.copy_(torch.randint(-128, 128, (M, K), generator=g, device=dev, dtype=torch.int8))
    s_ch = banded((N,), torch.float32, dev).uniform_(1e-3, 1e-2)
    s_tok = banded((M,), torch.float32, dev).uniform_(0.01, 1.0)
    out = banded((M, N), torch.bfloat16, dev)
    call(lib.amct_gemm_w8a8, xq, wq, s_tok, s_ch, None, 0, out, None, M, N, K, _lib.BF16, stream(dev))
    cols = col_sample(N, 1 << 20).to(dev)
    want = ops.gemm_w8a8(xq.clone(), wq[cols].contiguous(), s_ch[cols].contiguous(), s_tok.clone(), None)
    same(out[:, cols], want, "output columns")


@pytest.mark.parametrize("M", [16, 48])
def test_w4a16_weight_beyond_4gib(big, M):
    """K7 with packed W [2097280, 4096] int4 (2^32 + 2^18 bytes), groups of 128: the sampled output columns against the
    exact anchor, within the bound of the reading the library reports for the call."""
    dev, lib = big, _lib.load()
    N, K, G = (1 << 21) + 128, 4096, 32
    g = torch.Generator(device=dev).manual_seed(11)
    packed = banded((N, K // 2), torch.uint8, dev)
    for i in range(0, N, 131072):
        packed[i:i + 131072] = torch.randint(0, 256, packed[i:i + 131072].shape, generator=g, device=dev, dtype=torch.uint8)
    scales = banded((N, G), torch.float16, dev)
    scales.copy_((1e-3 + 9e-3 * torch.rand(N, G, generator=g, device=dev)).to(torch.float16))
    zeros = banded((N, G), torch.uint8, dev)
    zeros.copy_(torch.randint(0, 16, (N, G), generator=g, device=dev, dtype=torch.uint8))
    x = banded((M, K), torch.bfloat16, dev).normal_()
    out = banded((M, N), torch.bfloat16, dev)
    wsb = lib.amct_gemm_w4a16_workspace_bytes(M, N, K, 128, 0)
    ws = banded((max(wsb, 16),), torch.uint8, dev)
    call(lib.amct_gemm_w4a16, x, None, packed, scales, _lib.F16, zeros, None, out, M, N, K, 128, _lib.BF16, ws, wsb, stream(dev))
    rounded = lib.amct_gemm_w4a16_weight_rounded(M, N, K, 128, _lib.BF16, wsb)
    assert rounded in (0, 1)
    cols = col_sample(N, 1 << 21)
    pk = packed[cols.to(dev)].cpu()
    codes = torch.stack([pk & 15, pk >> 4], dim=-1).reshape(len(cols), K).to(torch.int32) - 8
    check_weight_only(out[:, cols.to(dev)].cpu(), x.cpu(), codes, scales[cols.to(dev)].cpu(),
                      -(zeros[cols.to(dev)].cpu().float() - 8), 128, None, None, bool(rounded), what=M)


@pytest.mark.parametrize("M", [16, 48])
def test_w8a16_weight_beyond_4gib(big, M):
    """The int8 weight-only Linear with W [1048640, 4096] int8, one fp16 scale per output channel."""
    dev, lib = big, _lib.load()
    N, K = (1 << 20) + 64, 4096
    g = torch.Generator(device=dev).manual_seed(13)
    wq = banded((N, K), torch.int8, dev)
    for i in range(0, N, 65536):
        wq[i:i + 65536] = torch.randint(-128, 128, wq[i:i + 65536].shape, generator=g, device=dev, dtype=torch.int8)
    scales = banded((N, 1), torch.float16, dev)
    scales.copy_((1e-4 + 9e-4 * torch.rand(N, 1, generator=g, device=dev)).to(torch.float16))
    x = banded((M, K), torch.bfloat16, dev).normal_()
    out = banded((M, N), torch.bfloat16, dev)
    wsb = lib.amct_gemm_w8a16_workspace_bytes(M, N, K, K, 0)
    ws = banded((max(wsb, 16),), torch.uint8, dev)
    call(lib.amct_gemm_w8a16_ws, x, None, wq, scales, _lib.F16, None, None, out, M, N, K, K, _lib.BF16, ws, wsb, stream(dev))
    rounded = lib.amct_gemm_w8a16_weight_rounded(M, N, K, K, _lib.BF16, wsb)
    assert rounded in (0, 1)
    cols = col_sample(N, 1 << 20).to(dev)
    check_weight_only(out[:, cols].cpu(), x.cpu(), wq[cols].cpu().to(torch.int32), scales[cols].cpu(), None, K, None, None,
                      bool(rounded), what=M, exact_rel=2e-5)


R4, C4 = 32768 + 8, 65536                            # fp32: row 32768 starts at element 2^31 (byte 2^33)
ROWS4 = [0, 1, 16383, 32767, 32768, 32769, R4 - 1]


def test_quantise_with_given_factors_and_minmax_beyond_2g_elements(big):
    """amct_quant_with_params and amct_minmax on fp32 [32776, 65536], groups of 128 (int4 range, asymmetric), codes as
    int32 (8.6 GB of them): the sampled rows against the call on those rows alone."""
    dev, lib = big, _lib.load()
    G = C4 // 128
    w = banded((R4, C4), torch.float32, dev).normal_()
    scale = banded((R4, G), torch.float32, dev).uniform_(0.05, 0.5)
    offset = banded((R4, G), torch.int32, dev)
    offset.copy_(torch.randint(-8, 8, (R4, G), device=dev, dtype=torch.int32))
    dq = banded((R4, C4), torch.float32, dev)
    codes = banded((R4, C4), torch.int32, dev)
    call(lib.amct_quant_with_params, w, scale, offset, dq, codes, _lib.CODES_I32, None, _lib.COL_NONE, R4, C4, 128, -8, 7, 0,
         _lib.STAGE_FULL, _lib.F32, stream(dev))
    sdq, scodes = ops.quant_with_params(w[ROWS4].contiguous(), scale[ROWS4].contiguous(), offset[ROWS4].contiguous(), 128, -8, 7,
                                        codes_kind=_lib.CODES_I32)
    same(dq[ROWS4], sdq, "dequantised rows")
    same(codes[ROWS4], scodes, "codes")
    del dq, codes
    mn = banded((R4, G), torch.float32, dev)
    mx = banded((R4, G), torch.float32, dev)
    call(lib.amct_minmax, w, mn, mx, R4, C4, 128, _lib.F32, stream(dev))
    smn, smx = ops.minmax(w[ROWS4].contiguous(), 128)
    same(mn[ROWS4], smn, "group minima")
    same(mx[ROWS4], smx, "group maxima")


def test_static_quantise_beyond_2g_elements(big):
    """amct_quantize on bf16 [65552, 32768] with one scale and zero-point per column."""
    dev, lib = big, _lib.load()
    x = banded((R, C), torch.bfloat16, dev).normal_()
    sc = (20.0 + 20.0 * torch.rand(C, device=dev)).to(torch.bfloat16)
    zp = torch.randint(-20, 20, (C,), device=dev).to(torch.bfloat16)
    q = banded((R, C), torch.int8, dev)
    call(lib.amct_quantize, x, None, sc, zp, q, R, C, C, 0, _lib.BF16, stream(dev))
    same(q[ROWS], ops.quantize_static(x[ROWS].contiguous(), sc, zp, False), "codes")


def test_fp8_block_dequant_beyond_2g_elements(big):
    """The checkpoint converter's fp8 weight with one fp32 scale per 128 x 128 block: whole block rows of the big call
    (the first, and the ones around element 2^31) against the call on those rows alone."""
    dev, lib = big, _lib.load()
    rows = R - R % 128 + 128                          # 65664: whole blocks
    w = banded((rows, C), torch.uint8, dev)
    for i in range(0, rows, 8192):
        w[i:i + 8192] = torch.randint(0, 256, w[i:i + 8192].shape, device=dev, dtype=torch.uint8)
    scale = banded((rows // 128, C // 128), torch.float32, dev).uniform_(0.5, 2.0)
    out = banded((rows, C), torch.bfloat16, dev)
    call(lib.amct_fp8_block_dequant, w, scale, out, rows, C, 128, _lib.BF16, stream(dev))
    small = banded((256, C), torch.bfloat16, dev)
    for r0 in (0, 65536 - 128, rows - 256):
        call(lib.amct_fp8_block_dequant, w[r0:r0 + 256].clone(), scale[r0 // 128:r0 // 128 + 2].clone(), small, 256, C, 128,
             _lib.BF16, stream(dev))
        same(out[r0:r0 + 256], small, "rows from {}".format(r0))


def test_int4_pair_packing_beyond_2g_elements(big):
    """pack_4bit of the converter: int8 [65552, 32768] int4 values -> two output channels per byte."""
    dev, lib = big, _lib.load()
    x = banded((R, C), torch.int8, dev)
    for i in range(0, R, 8192):
        x[i:i + 8192] = torch.randint(-8, 8, x[i:i + 8192].shape, device=dev, dtype=torch.int8)
    y = banded((R // 2, C), torch.int8, dev)
    call(lib.amct_pack_int4_pairs_n, x, y, R, C, stream(dev))
    small = torch.empty(1, C, dtype=torch.int8, device=dev)
    for r in (0, 32767, 32768, R // 2 - 1):
        call(lib.amct_pack_int4_pairs_n, x[2 * r:2 * r + 2].clone(), small, 2, C, stream(dev))
        same(y[r:r + 1], small, "output row {}".format(r))


def test_int4_layout_conversions_beyond_4gib(big):
    """The reference's operand int32 [k, n] (one int4 each, 34 GB here) -> words [k, n/8] -> the GEMM layout uint8
    [n, k/2] (2^32 + 2^17 bytes) -> back to int32 [k, n]: column blocks at the start, around the packed row that starts
    at byte 2^32, and at the end, against the conversions of those columns alone; and the round trip as a whole."""
    dev, lib = big, _lib.load()
    k, n = 4096, (1 << 21) + 64
    codes = banded((k, n), torch.int32, dev)
    for i in range(0, k, 64):
        codes[i:i + 64] = torch.randint(-8, 8, (64, n), device=dev, dtype=torch.int32)
    words = banded((k, n // 8), torch.int32, dev)
    call(lib.amct_pack_int4_words, codes, words, k, n, stream(dev))
    packed = banded((n, k // 2), torch.uint8, dev)
    call(lib.amct_words_to_nibbles_nk, words, packed, k, n, stream(dev))
    for c0 in (0, (1 << 21) - 64, 1 << 21, n - 64):
        sub = codes[:, c0:c0 + 64].contiguous()
        sw = ops.pack_int4_words(sub)
        same(words[:, c0 // 8:c0 // 8 + 8].contiguous(), sw, "words of columns from {}".format(c0))
        same(packed[c0:c0 + 64], ops.words_to_nibbles_nk(sw, k, 64), "nibbles of columns from {}".format(c0))
    back = banded((k, n), torch.int32, dev)
    call(lib.amct_nibbles_nk_to_codes_kn, packed, back, k, n, stream(dev))
    for i in range(0, k, 256):
        assert torch.equal(back[i:i + 256], codes[i:i + 256]), "round trip, rows from {}".format(i)


def test_awq_loss_beyond_2g_elements(big):
    """mean((y - yhat)^4) over 2^31 + 2^19 bf16 elements against torch in fp64, block by block."""
    dev, lib = big, _lib.load()
    n = R * C
    y = banded((n,), torch.bfloat16, dev).normal_()
    yhat = banded((n,), torch.bfloat16, dev).normal_()
    yhat[n - 1] = 300.0                               # a term that only an index beyond 2^31 reaches: (300 - y)^4 / n is ~4
    loss = banded((1,), torch.float32, dev)
    wsb = lib.amct_awq_loss_workspace_bytes()
    ws = banded((wsb,), torch.uint8, dev)
    call(lib.amct_awq_loss, y, yhat, n, _lib.BF16, loss, ws, wsb, stream(dev))
    tot = 0.0
    for i in range(0, n, 1 << 26):
        d = (y[i:i + (1 << 26)] - yhat[i:i + (1 << 26)]).double()
        tot += float((d * d * d * d).sum())
    want = tot / n
    assert want > 10.0 and abs(float(loss[0]) - want) <= 1e-5 * want, (float(loss[0]), want)
