"""Parity of the two quantized Linear kernels with the CPU oracle."""
import pytest
import torch

from amct_amd import ops, workloads
from oracle import deploy as od
from util import assert_bits_equal, check_weight_only

pytestmark = pytest.mark.gpu


def w8a8_case(M, N, K, seed, per_token=True, bias=None):
    g = torch.Generator().manual_seed(seed)
    xq = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8)
    wq = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
    s_ch = 1e-3 + 9e-3 * torch.rand(N, generator=g)
    s_tok = (0.01 + torch.rand(M, generator=g)) if per_token else None
    b = None
    if bias == 'int':
        b = torch.randint(-100000, 100000, (N,), generator=g, dtype=torch.int32)
    elif bias == 'float':
        b = torch.randn(N, generator=g)
    return xq, wq, s_ch, s_tok, b


def brute_int_matmul(xq, wq):
    M, K = xq.shape
    N = wq.shape[0]
    out = torch.zeros(M, N, dtype=torch.int64)
    for m in range(M):
        for n in range(N):
            acc = 0
            for k in range(K):
                acc += int(xq[m, k]) * int(wq[n, k])
            out[m, n] = acc
    return out


@pytest.mark.parametrize("M,N,K", [(5, 7, 9), (16, 16, 64), (33, 17, 100), (64, 64, 64)])
def test_w8a8_tiny_bruteforce(dev, M, N, K):
    xq, wq, s_ch, s_tok, b = w8a8_case(M, N, K, 89, True, 'int')
    out, acc = ops.gemm_w8a8(xq.to(dev), wq.to(dev), s_ch.to(dev), s_tok.to(dev), b.to(dev), want_acc=True)
    want_acc = brute_int_matmul(xq, wq) + b.to(torch.int64)
    assert torch.equal(acc.cpu().to(torch.int64), want_acc)
    assert torch.equal(od.int8_matmul_exact(xq, wq.t()) + b.to(torch.int64), want_acc)      # pins the fp64 oracle too
    assert_bits_equal(out, od.quant_matmul(xq, wq.t(), s_ch, s_tok, b, torch.bfloat16), "out")


@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (256, 384, 512), (130, 200, 192), (16, 512, 4096), (1, 256, 1024),
                                   (300, 129, 320), (2048, 256, 4096), (2, 72, 4096), (8, 40, 2048), (7, 33, 768), (12, 100, 1280),
                                   (3, 48, 256)])
@pytest.mark.parametrize("per_token,bias", [(True, None), (True, 'float'), (False, 'int'), (False, None)])
def test_w8a8_vs_oracle(dev, M, N, K, per_token, bias):
    xq, wq, s_ch, s_tok, b = w8a8_case(M, N, K, 97, per_token, bias)
    for odt in (torch.bfloat16, torch.float16, torch.float32):
        out, acc = ops.gemm_w8a8(xq.to(dev), wq.to(dev), s_ch.to(dev), None if s_tok is None else s_tok.to(dev),
                                 None if b is None else b.to(dev), out_dtype=odt, want_acc=True)
        want_acc = od.int8_matmul_exact(xq, wq.t())
        if bias == 'int':
            want_acc = want_acc + b.to(torch.int64)
        assert torch.equal(acc.cpu().to(torch.int64), want_acc), "accumulators"
        want = od.quant_matmul(xq, wq.t(), s_ch, s_tok, b, odt)
        assert_bits_equal(out, want, "out %s" % odt)
        # tolerance anchor: fp64 epilogue, 1e-3 of the largest magnitude
        f64 = od.quant_matmul_f64(xq, wq.t(), s_ch, s_tok, b)
        tol = 1e-3 if odt != torch.bfloat16 else 2.0 ** -8
        assert ((out.cpu().double() - f64).abs() <= tol * f64.abs().clamp_min(f64.abs().max() * 1e-3)).all()


@pytest.mark.parametrize("M,N,K", [(300, 1000, 320), (256, 448, 128), (512, 832, 256), (2048, 14336, 192), (1100, 9000, 64),
                                   (2000, 14328, 128), (100, 1000, 256), (200, 520, 384), (384, 14336, 128), (17, 72, 128),
                                   (640, 14336, 128), (33, 40000, 128), (5, 64, 128), (3, 14336, 384), (64, 200, 384),
                                   (33, 14336, 256), (100, 14336, 128), (128, 8200, 256), (16, 40000, 128), (1, 16392, 128),
                                   (16, 520, 14336), (40, 1000, 8192), (130, 2056, 8192), (300, 1000, 4224), (5, 64, 6144),
                                   (1000, 1032, 4096), (520, 4096, 2304)])
def test_w8a8_large_shapes_mixed_blocks(dev, M, N, K):
    """Block shapes of the tile kernels: 64x64 and 128x64 blocks for small M, 128x128 and 128x256 for medium M, 256x256 for large M, where a launch
    may mix in 256x192 blocks so that the blocks fill the CUs evenly; ragged edges in M and N, accumulators bit for bit.
    The last shapes (few column blocks, long rows) split K over several blocks per tile (ops.gemm_w8a8 lends the
    workspace for the int32 partial sums): the same bits."""
    xq, wq, s_ch, s_tok, b = w8a8_case(M, N, K, 131, True, 'float')
    want_acc = od.int8_matmul_exact(xq, wq.t())
    for odt in (torch.bfloat16, torch.float32):
        out, acc = ops.gemm_w8a8(xq.to(dev), wq.to(dev), s_ch.to(dev), s_tok.to(dev), b.to(dev), out_dtype=odt, want_acc=True)
        assert torch.equal(acc.cpu().to(torch.int64), want_acc), "accumulators"
        assert_bits_equal(out, od.quant_matmul(xq, wq.t(), s_ch, s_tok, b, odt), "out %s" % odt)
    # the other epilogue variants on the same operands: no per-token factor with an int32 bias (fp16 out), no bias at all
    _, _, _, _, ib = w8a8_case(M, N, K, 133, False, 'int')
    out, acc = ops.gemm_w8a8(xq.to(dev), wq.to(dev), s_ch.to(dev), None, ib.to(dev), out_dtype=torch.float16, want_acc=True)
    assert torch.equal(acc.cpu().to(torch.int64), want_acc + ib.to(torch.int64)), "accumulators with int bias"
    assert_bits_equal(out, od.quant_matmul(xq, wq.t(), s_ch, None, ib, torch.float16), "out fp16, int bias")
    out = ops.gemm_w8a8(xq.to(dev), wq.to(dev), s_ch.to(dev), s_tok.to(dev), None)
    assert_bits_equal(out, od.quant_matmul(xq, wq.t(), s_ch, s_tok, None, torch.bfloat16), "out bf16, no bias")


@pytest.mark.parametrize("M,N,K", [(1, 64, 1024), (16, 200, 2048), (9, 72, 1024), (5, 33, 2048), (16, 1000, 1024),
                                   (13, 14336, 4096), (1, 14336, 2048), (3, 16, 4096), (16, 15, 1024), (2, 4104, 4096)])
def test_w8a8_weight_streaming_kernel(dev, M, N, K):
    """The kernel for a few rows (M <= 16, K of 1024/2048/4096): both block widths, ragged N, every epilogue variant
    and output dtype; accumulators and outputs bit for bit."""
    for per_token, bias_kind in ((True, 'float'), (False, 'int'), (True, None)):
        xq, wq, s_ch, s_tok, b = w8a8_case(M, N, K, 150 + M, per_token, bias_kind)
        want_acc = od.int8_matmul_exact(xq, wq.t())
        if bias_kind == 'int':
            want_acc = want_acc + b.to(torch.int64)
        for odt in (torch.bfloat16, torch.float16, torch.float32):
            out, acc = ops.gemm_w8a8(xq.to(dev), wq.to(dev), s_ch.to(dev), None if s_tok is None else s_tok.to(dev),
                                     None if b is None else b.to(dev), out_dtype=odt, want_acc=True)
            assert torch.equal(acc.cpu().to(torch.int64), want_acc), "accumulators"
            assert_bits_equal(out, od.quant_matmul(xq, wq.t(), s_ch, s_tok, b, odt), "out %s" % odt)


@pytest.mark.parametrize("M,N,K", [(1, 64, 1024), (16, 200, 2048), (9, 72, 4096), (16, 14336, 4096), (5, 33, 2048), (3, 4104, 4096),
                                   (16, 1000, 1024), (40, 200, 1024), (7, 136, 8192), (300, 520, 4096)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_linear_w8a8_one_call(dev, M, N, K, dtype):
    """Static activation quantisation + W8A8 Linear in one library call (the deploy module's forward): up to 16 rows and K
    of 1024/2048/4096 the activations are quantised inside the weight-streaming kernel, otherwise the two kernels run through
    the workspace (the last shapes).  Per-tensor and per-token scales, with and without offsets and smoothing, both bias
    kinds, every output dtype: the bits of npu_quantize followed by npu_quant_matmul (the oracle), and of the two separate
    library calls."""
    from oracle import int_quant as iq
    g = torch.Generator().manual_seed(300 + M)
    x = (torch.randn(M, K, generator=g) * 3).to(dtype)
    smooth = (0.5 + torch.rand(K, generator=g)).to(dtype)
    for per_token, zp, sm, bias_kind, odt in ((False, False, False, 'int', torch.bfloat16), (True, True, True, 'float', torch.float16),
                                              (True, False, False, None, torch.float32), (False, True, True, 'float', torch.bfloat16)):
        _, wq, s_ch, s_tok, b = w8a8_case(M, N, K, 310 + M, per_token, bias_kind)
        ns = M if per_token else 1
        act_scale = (20 + 20 * torch.rand(ns, generator=g)).to(dtype)
        act_off = torch.randint(-20, 21, (ns,), generator=g).to(dtype) if zp else None
        dv = lambda t: None if t is None else t.to(dev)
        out = ops.linear_w8a8(x.to(dev), act_scale.to(dev), dv(act_off), per_token, wq.to(dev), s_ch.to(dev), dv(s_tok), dv(b), odt,
                              smooth.to(dev) if sm else None)
        xq = ops.quantize_static(x.to(dev), act_scale.to(dev), dv(act_off), per_token, smooth.to(dev) if sm else None)
        two = ops.gemm_w8a8(xq, wq.to(dev), s_ch.to(dev), dv(s_tok), dv(b), odt)
        assert_bits_equal(out, two.cpu(), "one call against two")
        xs = (x * smooth).to(dtype) if sm else x
        xq_o = iq.static_quantize(xs, act_scale, act_off if zp else torch.zeros(ns, dtype=dtype), axis=-2 if per_token else -1)
        assert torch.equal(xq.cpu(), xq_o), "codes"
        assert_bits_equal(out, od.quant_matmul(xq_o, wq.t(), s_ch, s_tok, b, odt), "against the oracle")


def w4a16_case(M, N, K, group, seed, sdt=torch.float16):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    codes = torch.randint(0, 16, (N, K), generator=g, dtype=torch.uint8)
    scales = (1e-3 + 9e-3 * torch.rand(N, K // group, generator=g)).to(sdt)
    zeros = torch.randint(0, 16, (N, K // group), generator=g, dtype=torch.uint8)
    smooth = (0.5 + torch.rand(K, generator=g)).to(torch.bfloat16)
    bias = torch.randn(N, generator=g)
    return x, codes, scales, zeros, smooth, bias


def w4a16_check(out, x, codes, scales, zeros, group, smooth, bias, rows=None, what=""):
    """Against the exact fp64 anchor, with the bound of the reading the LIBRARY says this call took (tests.util).
    rows: the number of rows of the call when x / out are a sample of them."""
    m = x.shape[0] if rows is None else rows
    rounded = ops.gemm_w4a16_weight_rounded(m, codes.shape[0], x.shape[1], group, x.dtype)
    return check_weight_only(out, x, codes.to(torch.int32) - 8, scales, -(zeros.to(torch.float32) - 8), group, bias, smooth,
                             rounded, what)


@pytest.mark.parametrize("M,N,K,group", [(300, 1000, 256, 64), (256, 448, 128, 128), (2048, 14336, 256, 128), (2000, 14328, 128, 64),
                                         (65, 72, 128, 64), (100, 1000, 384, 128), (200, 520, 640, 64), (384, 14336, 128, 128),
                                         (130, 40000, 128, 64), (640, 14336, 256, 128), (100, 1000, 512, 128), (256, 136, 1024, 64),
                                         (65, 14336, 256, 256), (25, 200, 128, 64), (40, 14336, 256, 128), (48, 40000, 128, 64),
                                         (100, 14336, 128, 128), (128, 8200, 256, 64), (64, 14336, 128, 128), (300, 14336, 128, 128),
                                         (512, 14328, 256, 64), (257, 1000, 384, 128), (33, 200, 512, 64), (100, 520, 768, 128), (64, 14336, 256, 128),
                                         (40, 520, 8192, 128), (8, 1000, 14336, 128), (100, 4096, 4096, 128), (200, 264, 11008, 64),
                                         (17, 14336, 4096, 128), (64, 1000, 2048, 64), (33, 4104, 4096, 256), (50, 8200, 3072, 128)])
def test_w4a16_large_shapes_ragged(dev, M, N, K, group):
    """The wide tile kernels (M > 24, group % 64 == 0) in their block shapes (64x64, 128x64, 128x128 with and without specialised
    waves, 128x256, 256x256; two or three LDS stages) on ragged edges in M and N, both scale dtypes; the last shapes (few
    column blocks, long rows) with K split over several blocks per tile and the partial sums added by a second kernel.
    Every output against the exact anchor within the bound of the reading the library reports for the call."""
    for sdt in (torch.float16, torch.bfloat16):
        x, codes, scales, zeros, smooth, bias = w4a16_case(M, N, K, group, 137, sdt)
        packed = workloads.pack_nibbles(codes)
        out = ops.gemm_w4a16(x.to(dev), packed.to(dev), scales.to(dev), zeros.to(dev), group, None, bias.to(dev))
        w4a16_check(out, x, codes, scales, zeros, group, None, bias, what=str(sdt))
    # with smoothing: the pre-pass into the workspace, then the same kernels
    out = ops.gemm_w4a16(x.to(dev), packed.to(dev), scales.to(dev), zeros.to(dev), group, smooth.to(dev), None)
    w4a16_check(out, x, codes, scales, zeros, group, smooth, None, what="smoothed")


@pytest.mark.parametrize("M,N,K,group", [(1, 64, 256, 128), (16, 128, 512, 128), (7, 33, 128, 32), (64, 64, 256, 64),
                                         (130, 200, 384, 128), (256, 256, 1024, 128), (2048, 128, 4096, 128),
                                         (16, 136, 4096, 128), (3, 72, 1024, 256), (20, 64, 768, 128),
                                         (40, 96, 1024, 128), (64, 200, 2048, 128), (33, 64, 384, 128),
                                         (8, 96, 4096, 128), (5, 80, 2048, 64), (12, 64, 4096, 128), (2, 48, 8192, 128)])
@pytest.mark.parametrize("sdt", [torch.float16, torch.bfloat16])
def test_w4a16_vs_oracle(dev, M, N, K, group, sdt):
    x, codes, scales, zeros, smooth, bias = w4a16_case(M, N, K, group, 101, sdt)
    packed = workloads.pack_nibbles(codes)
    for sm, b in ((None, None), (smooth, bias)):
        out = ops.gemm_w4a16(x.to(dev), packed.to(dev), scales.to(dev), zeros.to(dev), group,
                             None if sm is None else sm.to(dev), None if b is None else b.to(dev))
        w4a16_check(out, x, codes, scales, zeros, group, sm, b)


@pytest.mark.parametrize("M,N,K", [(1, 64, 1024), (16, 200, 2048), (9, 72, 1024), (5, 33, 2048), (16, 1000, 1024),
                                   (13, 14336, 4096), (1, 14336, 2048), (3, 16, 4096), (16, 15, 1024),
                                   (16, 40000, 1024), (16, 20008, 4096), (1, 70000, 1024), (4, 33000, 2048), (2, 16392, 4096),
                                   (16, 1000, 8192), (8, 520, 14336), (6, 264, 5120), (16, 20008, 8192), (12, 200, 28672),
                                   (1, 72, 12288), (16, 520, 11008), (8, 264, 13824), (5, 200, 2816), (1, 72, 13824), (2, 136, 11008), (16, 4104, 11008)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_w4a16_weight_streaming_kernel(dev, M, N, K, dtype):
    """The kernel for a few rows (M <= 16, K of 1024/2048/4096, groups of 128): every block width, ragged N, both factor
    dtypes, with and without smoothing, against the fp64 anchor whose dequantised weight is not rounded (the last
    shapes: more column tiles than the device runs blocks at once, so that a block walks several tiles -- one, two, three
    or more, with a ragged last one -- on one staged copy of the activations; rows of 2 ... 14 slices of 1024, 2048 or 4096
    elements, whose partial sums a second kernel adds in slice order, the last slice shorter for K = 11008, 13824, 2816); then the
    integer special case (scale 1, small integer activations), where both readings of the dequantisation give the same
    bits as an integer matmul."""
    assert not ops.gemm_w4a16_weight_rounded(M, N, K, 128, dtype), "the library reports a rounding kernel for this shape"
    for sdt in (torch.float16, torch.bfloat16):
        x, codes, scales, zeros, smooth, bias = w4a16_case(M, N, K, 128, 140 + M, sdt)
        x, smooth = x.to(dtype), smooth.to(dtype)
        packed = workloads.pack_nibbles(codes).to(dev)
        for sm, b in ((None, None), (smooth, bias)):
            out = ops.gemm_w4a16(x.to(dev), packed, scales.to(dev), zeros.to(dev), 128,
                                 None if sm is None else sm.to(dev), None if b is None else b.to(dev))
            # exact weights, fp32 accumulation: an ulp of the value plus 1e-5 of the row's largest output
            w4a16_check(out, x, codes, scales, zeros, 128, sm, b)
            assert out.dtype == dtype
    g = torch.Generator().manual_seed(141)
    xi = torch.randint(-4, 5, (M, K), generator=g).to(dtype)
    ones = torch.ones(N, K // 128, dtype=torch.float16)
    out = ops.gemm_w4a16(xi.to(dev), packed, ones.to(dev), zeros.to(dev), 128)
    wi = codes.float() - zeros.float().repeat_interleave(128, dim=1)
    want = torch.matmul(xi.double(), wi.double().t())                # integers below 2^24: exact in the kernel's fp32 too
    assert_bits_equal(out, want.to(dtype), "integer special case")


def w8a16_check(out, x, codes, scales, offsets, group, smooth, bias, rows=None, what="", workspace_bytes=None):
    """As w4a16_check for the int8 weight-only Linear (exact reading: 2e-5 of the row's largest output, the correction
    term of its q + 128 form is larger than the int4 kernel's)."""
    m = x.shape[0] if rows is None else rows
    rounded = ops.gemm_w8a16_weight_rounded(m, codes.shape[0], x.shape[1], group, x.dtype, workspace_bytes)
    return check_weight_only(out, x, codes.to(torch.int32), scales, None if offsets is None else -offsets.float(), group, bias,
                             smooth, rounded, what, exact_rel=2e-5)


def w8a16_case(M, N, K, group, seed, dtype, sdt, sym):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).to(dtype)
    codes = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int16).to(torch.int8)
    scales = (1e-3 + 9e-3 * torch.rand(N, K // group, generator=g)).to(sdt)
    offsets = None if sym else torch.randint(-128, 128, (N, K // group), generator=g, dtype=torch.int16).to(torch.int8)
    smooth = (0.5 + torch.rand(K, generator=g)).to(dtype)
    bias = torch.randn(N, generator=g)
    return x, codes, scales, offsets, smooth, bias


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K,group", [(1, 64, 1024, 128), (16, 200, 2048, 256), (9, 72, 1024, 1024), (5, 33, 2048, 128),
                                         (16, 1000, 4096, 4096), (13, 14336, 4096, 128), (1, 14336, 4096, 4096),
                                         (3, 16, 4096, 512), (16, 15, 1024, 512), (2, 300, 4096, 2048), (16, 520, 4096, 1024),
                                         (16, 1000, 8192, 128), (8, 520, 14336, 14336), (6, 264, 5120, 256), (12, 200, 28672, 4096),
                                         (1, 72, 12288, 12288), (16, 136, 8192, 8192), (16, 520, 11008, 11008), (3, 264, 13824, 128),
                                         (9, 200, 2816, 256)])
def test_w8a16_weight_streaming_kernel(dev, dtype, M, N, K, group):
    """The int8 weight-only kernel for a few rows (M <= 16, K of 1024/2048/4096 or 2 ... 14 slices of those, whose partial
    sums a second kernel adds in slice order; groups of 128, 256, ... up to K, i.e.
    per-channel factors too): every block width, ragged N, both activation and factor dtypes, symmetric and with
    offsets, with and without smoothing and bias, against the fp64 anchor whose dequantised weight is not rounded; then
    the integer special case (scale 1, small integer activations), where the result is an integer matmul bit for bit."""
    assert not ops.gemm_w8a16_weight_rounded(M, N, K, group, dtype), "the library reports a rounding kernel for this shape"
    for sdt, sym in ((torch.float16, False), (torch.bfloat16, True)):
        x, codes, scales, offsets, smooth, bias = w8a16_case(M, N, K, group, 150 + M, dtype, sdt, sym)
        for sm, b in ((None, None), (smooth, bias)):
            out = ops.gemm_w8a16(x.to(dev), codes.to(dev), scales.to(dev), None if offsets is None else offsets.to(dev), group,
                                 None if sm is None else sm.to(dev), None if b is None else b.to(dev))
            assert out.dtype == dtype
            # exact weights, fp32 accumulation of x' * (q + 128) and of the correction term: 2e-5 of the row's largest
            # output plus an ulp of the value
            w8a16_check(out, x, codes, scales, offsets, group, sm, b, what=(sdt, sym, sm is not None))
    g = torch.Generator().manual_seed(151)
    xi = torch.randint(-4, 5, (M, K), generator=g).to(dtype)
    wi = torch.randint(-7, 8, (N, K), generator=g, dtype=torch.int16).to(torch.int8)
    zi = torch.randint(-3, 4, (N, K // group), generator=g, dtype=torch.int16).to(torch.int8)
    ones = torch.ones(N, K // group, dtype=torch.float16)
    out = ops.gemm_w8a16(xi.to(dev), wi.to(dev), ones.to(dev), zi.to(dev), group)
    want = torch.matmul(xi.double(), (wi.double() - zi.double().repeat_interleave(group, dim=1)).t())
    # every partial sum is an integer below 2^24, so the kernel's fp32 result is exact and its one rounding is torch's
    assert_bits_equal(out, want.to(dtype), "integer special case")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K,group", [(2048, 14336, 4096, 128), (256, 264, 64, 64), (300, 1000, 320, 32), (513, 2056, 1024, 1024),
                                         (1000, 4104, 192, 64), (300, 16, 65536, 256), (700, 1032, 4096, 128)])
def test_w8a16_many_rows_through_the_workspace(dev, dtype, M, N, K, group):
    """Int8 weight-only Linear from 256 rows on: with the workspace the library asks for, the weight is dequantised once
    and the product is the plain 16-bit GEMM on the large tiles (uniform and mixed tile launches, ragged M and N, K of
    one and of many steps); without it the shared 128x128 kernel runs.  Both compute dt((q - offset) * scale) and
    accumulate the exact products in fp32: sampled rows against the exact anchor within the bound of the rounded
    reading and within 2e-5 of the row's largest output (plus an ulp) of the anchor with the same rounding; small integers give an integer matmul bit for bit."""
    from amct_amd import _lib
    lib = _lib.load()
    rows = [r for r in FULL_ROWS if r < M]
    assert lib.amct_gemm_w8a16_workspace_bytes(M, N, K, group, 1) >= N * K * 2 + M * K * 2
    for sdt, sym in ((torch.float16, False), (torch.bfloat16, True)):
        x, codes, scales, offsets, smooth, bias = w8a16_case(M, N, K, group, 170 + M % 97, dtype, sdt, sym)
        for sm, b in ((None, None), (smooth, bias)):
            out = ops.gemm_w8a16(x.to(dev), codes.to(dev), scales.to(dev), None if offsets is None else offsets.to(dev), group,
                                 None if sm is None else sm.to(dev), None if b is None else b.to(dev)).cpu()[rows]
            w8a16_check(out, x[rows], codes, scales, offsets, group, sm, b, rows=M, what=(sdt, sym, sm is not None))
    g = torch.Generator().manual_seed(171)
    xi = torch.randint(-4, 5, (M, K), generator=g).to(dtype)
    wi = torch.randint(-7, 8, (N, K), generator=g, dtype=torch.int16).to(torch.int8)
    zi = torch.randint(-3, 4, (N, K // group), generator=g, dtype=torch.int16).to(torch.int8)
    ones = torch.ones(N, K // group, dtype=torch.float16)
    out = ops.gemm_w8a16(xi.to(dev), wi.to(dev), ones.to(dev), zi.to(dev), group)
    want = torch.matmul(xi[rows].double(), (wi.double() - zi.double().repeat_interleave(group, dim=1)).t())
    assert_bits_equal(out.cpu()[rows], want.to(dtype), "integer special case")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K,group", [(17, 14336, 4096, 128), (40, 520, 1024, 128), (64, 14336, 4096, 4096), (65, 200, 512, 64),
                                         (128, 8200, 256, 64), (200, 1000, 768, 256), (256, 14336, 4096, 128), (100, 264, 320, 64),
                                         (33, 20000, 256, 128), (512, 14336, 1024, 128), (8, 520, 8192, 128), (100, 2048, 8192, 256),
                                         (1, 1000, 14336, 128), (300, 40000, 256, 128), (500, 70000, 256, 256)])
def test_w8a16_medium_rows_specialised_waves(dev, dtype, M, N, K, group):
    """Int8 weight-only Linear from 17 rows on, up to 384 rows (512 unless a last round of blocks would run half empty):
    the tile kernels with specialised waves (K a multiple of 256; 64x64, 128x64 and 128x128 blocks, the latter in as
    many rounds as it takes: the two widest shapes), ragged M and N, per-channel and grouped
    factors, symmetric and with offsets, with smoothing (through the workspace ops.gemm_w8a16 lends) and bias; one shape
    the shared kernel keeps (K = 320); the last shapes (few column blocks, long rows, any number of rows) with K split
    over several blocks per tile.  Against the exact anchor within the bound of the reading the library reports; small integers give an integer matmul bit for bit."""
    from amct_amd import _lib
    assert _lib.load().amct_gemm_w8a16_workspace_bytes(M, N, K, group, 1) >= M * K * 2
    for sdt, sym in ((torch.float16, False), (torch.bfloat16, True)):
        x, codes, scales, offsets, smooth, bias = w8a16_case(M, N, K, group, 190 + M % 97, dtype, sdt, sym)
        for sm, b in ((None, None), (smooth, bias)):
            out = ops.gemm_w8a16(x.to(dev), codes.to(dev), scales.to(dev), None if offsets is None else offsets.to(dev), group,
                                 None if sm is None else sm.to(dev), None if b is None else b.to(dev)).cpu()
            assert out.dtype == dtype
            w8a16_check(out, x, codes, scales, offsets, group, sm, b, what=(sdt, sym, sm is not None))
    g = torch.Generator().manual_seed(191)
    xi = torch.randint(-4, 5, (M, K), generator=g).to(dtype)
    wi = torch.randint(-7, 8, (N, K), generator=g, dtype=torch.int16).to(torch.int8)
    zi = torch.randint(-3, 4, (N, K // group), generator=g, dtype=torch.int16).to(torch.int8)
    ones = torch.ones(N, K // group, dtype=torch.float16)
    out = ops.gemm_w8a16(xi.to(dev), wi.to(dev), ones.to(dev), zi.to(dev), group)
    want = torch.matmul(xi.double(), (wi.double() - zi.double().repeat_interleave(group, dim=1)).t())
    assert_bits_equal(out, want.to(dtype), "integer special case")


@pytest.mark.parametrize("M", [40, 300])
def test_w8a16_smoothing_with_and_without_workspace(dev, M):
    """With a smoothing vector the fast int8 weight-only tile kernels need the lent workspace (M * K * 2 bytes); without
    it, or with one that is too small, the call is still served (shared kernel, smoothing inside the tile) and both
    answers are within the tolerance of the fp64 anchor.  Through the C ABI."""
    from amct_amd import _lib
    lib = _lib.load()
    N, K, group = 520, 1024, 128
    x, codes, scales, offsets, smooth, bias = w8a16_case(M, N, K, group, 777, torch.bfloat16, torch.float16, False)
    xd, cd, sd, zd, smd, bd = (t.to(dev) for t in (x, codes, scales, offsets, smooth, bias))
    st = torch.cuda.current_stream(dev).cuda_stream
    need = lib.amct_gemm_w8a16_workspace_bytes(M, N, K, group, 1)
    assert need >= M * K * 2
    for nbytes in (need, 0, M * K * 2 - 16):
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)
        out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
        _lib.check(lib.amct_gemm_w8a16_ws(xd.data_ptr(), smd.data_ptr(), cd.data_ptr(), sd.data_ptr(), _lib.F16, zd.data_ptr(),
                                          bd.data_ptr(), out.data_ptr(), M, N, K, group, _lib.BF16,
                                          ws.data_ptr() if nbytes else None, nbytes, st))
        w8a16_check(out, x, codes, scales, offsets, group, smooth, bias, what=nbytes, workspace_bytes=nbytes)


def test_w4a16_reduces_to_plain_matmul(dev):
    """zero = 8 (code 0 in signed terms), scale = 1: the kernel is a bf16 GEMM against integer
    weights, checked against torch.matmul."""
    g = torch.Generator().manual_seed(103)
    M, N, K = 64, 96, 256
    x = torch.randint(-4, 5, (M, K), generator=g).to(torch.bfloat16)
    codes = torch.randint(0, 16, (N, K), generator=g, dtype=torch.uint8)
    scales = torch.ones(N, K // 128, dtype=torch.float16)
    zeros = torch.full((N, K // 128), 8, dtype=torch.uint8)
    out = ops.gemm_w4a16(x.to(dev), workloads.pack_nibbles(codes).to(dev), scales.to(dev), zeros.to(dev), 128)
    want = torch.matmul(x.float(), (codes.float() - 8).t())          # small integers: exact in fp32
    assert_bits_equal(out, want.to(torch.bfloat16), "plain matmul")


BOUNDARY_M = [1, 2, 3, 15, 16, 17, 24, 25, 32, 33, 40, 41, 63, 64, 65, 127, 128, 129, 255, 256, 257, 300, 513]


@pytest.mark.parametrize("N,K", [(136, 256), (4104, 128)])
def test_gemm_dispatch_boundaries_in_m(dev, N, K):
    """Every row count at which the libraries switch kernels (decode, 64x64, 128x64, 128x128, 128x256, 256x256 tiles;
    with smoothing the W4A16 switch points move), on one weight: W8A8 bit for bit, W4A16 within its tolerance."""
    xq, wq, s_ch, s_tok, b = w8a8_case(max(BOUNDARY_M), N, K, 211, True, 'float')
    x, codes, scales, zeros, smooth, bias = w4a16_case(max(BOUNDARY_M), N, K, 64, 212)
    packed = workloads.pack_nibbles(codes).to(dev)
    want8 = od.quant_matmul(xq, wq.t(), s_ch, s_tok, b, torch.bfloat16)
    dwq, dsc, db = wq.to(dev), s_ch.to(dev), b.to(dev)
    dscales, dzeros, dbias, dsmooth = scales.to(dev), zeros.to(dev), bias.to(dev), smooth.to(dev)
    for M in BOUNDARY_M:
        out = ops.gemm_w8a8(xq[:M].contiguous().to(dev), dwq, dsc, s_tok[:M].contiguous().to(dev), db)
        assert_bits_equal(out, want8[:M], "w8a8 M=%d" % M)
        for sm, dsm in ((None, None), (smooth, dsmooth)):
            xm = x[:M].contiguous()
            out = ops.gemm_w4a16(xm.to(dev), packed, dscales, dzeros, 64, dsm, dbias)
            w4a16_check(out, xm, codes, scales, zeros, 64, sm, bias, what=(M, sm is not None))


FULL_ROWS = [0, 1, 63, 64, 127, 128, 255, 256, 257, 511, 512, 1023, 1024, 1500, 2046, 2047]


@pytest.mark.parametrize("M", [2048, 16, 1])
def test_gemms_at_the_benchmark_size(dev, M):
    """N = 14336, K = 4096 (the size the metric is quoted on) for M = 2048 and the decode sizes: sampled rows of the W8A8
    output bit for bit and of the W4A16 output within its tolerance, every column."""
    N, K, grp = 14336, 4096, 128
    rows = [r for r in FULL_ROWS if r < M]
    xq, wq, s_ch, s_tok, b = w8a8_case(M, N, K, 311, True, 'float')
    out, acc = ops.gemm_w8a8(xq.to(dev), wq.to(dev), s_ch.to(dev), s_tok.to(dev), b.to(dev), want_acc=True)
    want_acc = od.int8_matmul_exact(xq[rows], wq.t())
    assert torch.equal(acc.cpu()[rows].to(torch.int64), want_acc), "accumulators"
    assert_bits_equal(out.cpu()[rows], od.quant_matmul(xq[rows], wq.t(), s_ch, s_tok[rows], b, torch.bfloat16), "w8a8 out")
    del out, acc
    x, codes, scales, zeros, smooth, bias = w4a16_case(M, N, K, grp, 312)
    packed = workloads.pack_nibbles(codes).to(dev)
    for sm in (None, smooth):
        out = ops.gemm_w4a16(x.to(dev), packed, scales.to(dev), zeros.to(dev), grp, None if sm is None else sm.to(dev),
                             bias.to(dev)).cpu()[rows]
        w4a16_check(out, x[rows], codes, scales, zeros, grp, sm, bias, rows=M, what=(M, sm is not None))


@pytest.mark.parametrize("M,N,K", [(2048, 14336, 4096), (520, 14336, 4096), (300, 14336, 4096), (130, 14336, 4096),
                                   (70, 14336, 4096), (200, 20000, 1024), (65, 72, 128), (17, 14336, 4096), (40, 14336, 4096),
                                   (64, 520, 1024), (33, 200, 512), (100, 1000, 768), (128, 20000, 256), (24, 72, 128),
                                   (32, 1000, 8192), (9, 520, 14336)])
def test_w4a16_fp16_at_the_benchmark_size(dev, M, N, K):
    """fp16 activations, more than 16 rows: the tile kernels with fp16 operands, every block shape the dispatch knows
    (256x256, 256x128, 128x256, 128x128, 128x64, 64x64; with specialised waves when K is a multiple of 256, the only
    tile kernels up to 64 rows; the dequantise-once form from 1025 rows on), with the lent workspace when the activations
    are smoothed (which ops.gemm_w4a16 lends); sampled rows against the exact anchor within the bound of the reading the
    library reports (fp16: u = 2^-11), every column; both factor dtypes."""
    grp = 128
    rows = [r for r in FULL_ROWS if r < M]
    for sdt in (torch.float16, torch.bfloat16):
        x, codes, scales, zeros, smooth, bias = w4a16_case(M, N, K, grp, 313, sdt)
        x, smooth = x.to(torch.float16), smooth.to(torch.float16)
        packed = workloads.pack_nibbles(codes).to(dev)
        for sm in (None, smooth):
            out = ops.gemm_w4a16(x.to(dev), packed, scales.to(dev), zeros.to(dev), grp, None if sm is None else sm.to(dev),
                                 bias.to(dev))
            assert out.dtype == torch.float16
            out = out.cpu()[rows]
            w4a16_check(out, x[rows], codes, scales, zeros, grp, sm, bias, rows=M, what=(M, sdt, sm is not None))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K,group", [(1025, 1000, 320, 32), (3584, 1000, 320, 32), (4100, 264, 64, 64), (1100, 16, 65536, 128),
                                         (1300, 1000, 4096, 128)])
def test_w4a16_very_many_rows_dequantise_once(dev, dtype, M, N, K, group):
    """From 1025 rows on, with the workspace the library asks for (the 16-bit weight and the smoothed activations), the
    int4 weight is dequantised once and the product is the plain 16-bit GEMM on the large tiles; with the smaller
    workspace of the fused kernels those run.  Same arithmetic (dt((u - z) * s), exact products, fp32 accumulation):
    sampled rows of both within the tolerance of the fp64 anchor; small integers bit for bit."""
    from amct_amd import _lib
    lib = _lib.load()
    # the 16-bit weight and the smoothed activations, plus the partial sums of a K-split GEMM when its tiles are few
    assert lib.amct_gemm_w4a16_workspace_bytes(M, N, K, group, 1) >= N * K * 2 + M * K * 2
    assert lib.amct_gemm_w4a16_workspace_bytes(M, N, K, group, 0) >= N * K * 2
    rows = sorted({r for r in FULL_ROWS + [M - 1, M - 2, 1023] if r < M})
    x, codes, scales, zeros, smooth, bias = w4a16_case(M, N, K, group, 333, torch.float16)
    x, smooth = x.to(dtype), smooth.to(dtype)
    xd, packed, sd, zd, smd, bd = x.to(dev), workloads.pack_nibbles(codes).to(dev), scales.to(dev), zeros.to(dev), smooth.to(dev), bias.to(dev)
    st = torch.cuda.current_stream(dev).cuda_stream
    for nbytes in (lib.amct_gemm_w4a16_workspace_bytes(M, N, K, group, 1), N * K * 2 + M * K * 2, M * K * 2):
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        out = torch.empty(M, N, dtype=dtype, device=dev)
        _lib.check(lib.amct_gemm_w4a16(xd.data_ptr(), smd.data_ptr(), packed.data_ptr(), sd.data_ptr(), _lib.F16, zd.data_ptr(),
                                       bd.data_ptr(), out.data_ptr(), M, N, K, group, _lib.BF16 if dtype == torch.bfloat16 else _lib.F16,
                                       ws.data_ptr(), ws.numel(), st))
        assert ops.gemm_w4a16_weight_rounded(M, N, K, group, dtype, nbytes)
        w4a16_check(out.cpu()[rows], x[rows], codes, scales, zeros, group, smooth, bias, rows=M, what=nbytes)
    g = torch.Generator().manual_seed(334)
    xi = torch.randint(-4, 5, (M, K), generator=g).to(dtype)
    ones = torch.ones(N, K // group, dtype=torch.float16)
    out = ops.gemm_w4a16(xi.to(dev), packed, ones.to(dev), zd, group)
    wi = codes.float() - zeros.float().repeat_interleave(group, dim=1)
    assert_bits_equal(out.cpu()[rows], torch.matmul(xi[rows].double(), wi.double().t()).to(dtype), "integer special case")


@pytest.mark.parametrize("seed", [1, 2])
def test_gemm_random_shapes(dev, seed):
    """Seeded random (M, N, K, group, scale dtype, smoothing) over the values at which the libraries switch kernels and
    over ragged ones: W8A8 bit for bit, W4A16 within its tolerance.  Every case is an ordinary supported call."""
    import random
    rng = random.Random(seed)
    done = 0
    while done < 40:
        M = rng.choice([1, 2, 3, 9, 16, 17, 24, 25, 31, 40, 41, 64, 65, 100, 128, 129, 200, 256, 257, 300, 511, 512, 513, 700])
        N = rng.choice([8, 16, 40, 64, 72, 128, 136, 200, 256, 520, 1000, 2056, 4104, 16392, 16400])
        K = rng.choice([64, 128, 192, 256, 320, 384, 512, 768, 1024, 2048, 4096, 8192, 8448])
        if M * N * K > 1.2e10:
            continue
        done += 1
        xq, wq, s_ch, s_tok, b = w8a8_case(M, N, K, 1000 * seed + done, True, 'float')
        out = ops.gemm_w8a8(xq.to(dev), wq.to(dev), s_ch.to(dev), s_tok.to(dev), b.to(dev))
        assert_bits_equal(out, od.quant_matmul(xq, wq.t(), s_ch, s_tok, b, torch.bfloat16), "w8a8 %d %d %d" % (M, N, K))
        group = rng.choice([g for g in (32, 64, 128, 256) if K % g == 0])
        sdt = rng.choice([torch.float16, torch.bfloat16])
        x, codes, scales, zeros, smooth, bias = w4a16_case(M, N, K, group, 1000 * seed + done, sdt)
        sm = smooth if rng.random() < 0.4 else None
        o4 = ops.gemm_w4a16(x.to(dev), workloads.pack_nibbles(codes).to(dev), scales.to(dev), zeros.to(dev), group,
                            None if sm is None else sm.to(dev), bias.to(dev)).cpu()
        w4a16_check(o4, x, codes, scales, zeros, group, sm, bias, what=(M, N, K, group, sdt, sm is not None))
