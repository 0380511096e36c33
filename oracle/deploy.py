"""Deploy-path oracle (CPU) -- test infrastructure only.

Restates how the reference builds the operands of its two quantized Linear
modules and what the device operators behind them compute.

Reference lines followed:

  w8a8_buffers      amct_pytorch/deploy_op/npu_quantization_linear.py:27-70,
                    72-87 (weight codes), 105-130 (bias)
  w8a8_forward      amct_pytorch/deploy_op/npu_quantization_linear.py:89-103
  w4a16_buffers     amct_pytorch/deploy_op/weight_npu_quant_module.py:29-100
  w4a16_forward     amct_pytorch/deploy_op/weight_npu_quant_module.py:102-121
  pack_int4_words   the call at weight_npu_quant_module.py:54-57
  pack_nibbles_k    this repo's own K-major nibble layout

The four device operators (activation quantise, int8 GEMM with rescale,
weight-only-quant GEMM, int4 packing) are implemented in the un-vendored
torch_npu package; the reference's tests replace them with mocks that neither
round, apply per-token scales, apply offsets nor pack
(tests/amct_pytorch/mock_torch_npu.py:21-90).  What is stated here is their
documented arithmetic.  Pin status:

  integer contraction   pinned: exact in fp64 (|acc| <= 4096*128*127 < 2^53);
                        tests also brute-force it with int64 loops on tiny
                        shapes.
  rescale epilogue      PARITY UNPINNED against torch_npu (order of the two
                        scale multiplies, where the float bias is added);
                        this repo fixes: fp32(acc+int_bias) * s_ch[n], then
                        * s_tok[m], then + float bias, then one rounding to
                        the output dtype.
  w4a16 dequant         PARITY UNPINNED against torch_npu (precision of the
                        dequantised weight); this repo fixes: (q - z) * s
                        exact in fp32, rounded once to x's dtype (every
                        kernel that feeds the matrix pipe a 16-bit weight)
                        or not rounded at all (the weight-streaming kernels
                        for M <= 16, as the reference's CPU stand-in
                        mock_torch_npu.py:33-55 does), fp32 accumulate.
                        The library says which reading a call takes
                        (amct_gemm_w4a16_weight_rounded); the tests compare
                        EVERY call with the exact anchor, the rounding ones
                        within weight_only_error_bounds().
                        Special case z=8 (unsigned), s=1 reduces to a plain
                        matmul -- tested against torch.matmul.
  int4 word packing     PARITY UNPINNED against torch_npu (nibble order);
                        this repo fixes little-endian: nibble j of word i
                        holds column 8*i+j.
"""
import torch

from . import int_quant as iq


# --------------------------------------------------------------------------
# W8A8
# --------------------------------------------------------------------------
def w8a8_buffers(weight, bias, scale_w, scale_d, offset_d=None, smooth=None, wts_type='int8'):
    """Returns dict with act_scale, act_offset, quantized_weight ([K,N] view of
    [N,K] storage), deq_scale, pertoken_scale, bias, scale_factor, granularity."""
    out_dtype = weight.dtype
    out = {}
    per_token = scale_d.dim() > 1
    off = offset_d if offset_d is not None else torch.tensor([0])
    off = off.repeat(scale_d.shape)
    out['act_scale'] = (1 / scale_d).reshape(-1).to(out_dtype)
    out['act_offset'] = off.reshape(-1).to(out_dtype)
    w = weight
    if smooth is not None:
        w = iq.smooth_weight(smooth, w)
        out['scale_factor'] = 1 / smooth
    sw = scale_w.reshape(-1)
    sdiv = sw.reshape(-1, 1) if sw.shape[0] > 1 else sw
    codes = iq.to_codes(w / sdiv, wts_type)                 # [N,K] int8
    wq = torch.transpose(codes, 1, 0)                       # [K,N] view
    out['quantized_weight'] = wq
    offset_bias = None
    if offset_d is not None:
        rep = offset_d.float().repeat(1, weight.shape[-1])
        offset_bias = rep.float() @ wq.float()
        offset_bias = -1 * offset_bias.round().to(torch.int32).reshape(-1)
    deq = scale_d * sw
    if not per_token:
        out['deq_scale'] = deq
        out['pertoken_scale'] = None
    else:
        out['deq_scale'] = sw
        out['pertoken_scale'] = scale_d.reshape(-1).to(torch.float32)
    b = None
    if bias is not None:
        if not per_token:
            b = (bias.data / (scale_d * sw)).round().to(torch.int32)
        else:
            b = bias
        if offset_bias is not None:
            b = b + offset_bias
    elif offset_bias is not None:
        b = offset_bias
    out['bias'] = b
    out['per_token'] = per_token
    out['output_dtype'] = out_dtype
    return out


def int8_matmul_exact(xq, wq_kn):
    """int8 x int8 -> exact integer accumulators as int64 ([M,K] @ [K,N])."""
    return (xq.double() @ wq_kn.double()).to(torch.int64)


def quant_matmul(xq, wq_kn, scale, pertoken_scale=None, bias=None, output_dtype=torch.bfloat16):
    """The int8 GEMM operator (npu_quantization_linear.py:100-102): integer
    accumulate, int32 bias joins the accumulator, fp32 rescale, float bias
    after the rescale, one rounding to the output dtype."""
    acc = int8_matmul_exact(xq.reshape(-1, xq.shape[-1]), wq_kn)
    fbias = None
    if bias is not None:
        if bias.dtype == torch.int32:
            acc = acc + bias.to(torch.int64)
        else:
            fbias = bias.float()
    # int32 -> fp32 conversion rounds to nearest even, as the device does
    f = acc.to(torch.int32).to(torch.float32)
    f = f * scale.reshape(1, -1).float()
    if pertoken_scale is not None:
        ps = pertoken_scale.reshape(-1).float()
        ps = ps.repeat(f.shape[0] // ps.numel())          # one scale per token, shared by leading batch dims
        f = f * ps.reshape(-1, 1)
    if fbias is not None:
        f = f + fbias
    return f.to(output_dtype).reshape(*xq.shape[:-1], -1)


def quant_matmul_f64(xq, wq_kn, scale, pertoken_scale=None, bias=None):
    """Same operator with the epilogue in fp64: the tolerance anchor."""
    acc = (xq.reshape(-1, xq.shape[-1]).double() @ wq_kn.double())
    fb = None
    if bias is not None:
        if bias.dtype == torch.int32:
            acc = acc + bias.double()
        else:
            fb = bias.double()
    f = acc * scale.reshape(1, -1).double()
    if pertoken_scale is not None:
        f = f * pertoken_scale.reshape(-1, 1).double()
    if fb is not None:
        f = f + fb
    return f


def w8a8_forward(buf, x):
    """Module forward (npu_quantization_linear.py:89-103)."""
    if buf.get('scale_factor') is not None:
        x = x * buf['scale_factor']
    xq = iq.static_quantize(x, buf['act_scale'], buf['act_offset'],
                            axis=-2 if buf['per_token'] else -1)
    return quant_matmul(xq, buf['quantized_weight'], buf['deq_scale'], buf['pertoken_scale'],
                        buf['bias'], buf['output_dtype'])


# --------------------------------------------------------------------------
# W4A16 / W8A16
# --------------------------------------------------------------------------
def pack_int4_words(codes_i32):
    """[K,N] int32 holding one int4 each -> [K,N/8] int32, column 8*i+j in
    bits 4j..4j+3 of word i (the operator called at
    weight_npu_quant_module.py:54-57; order is this repo's choice)."""
    k, n = codes_i32.shape
    u = (codes_i32.to(torch.int64) & 0xF).reshape(k, n // 8, 8)
    word = torch.zeros(k, n // 8, dtype=torch.int64)
    for j in range(8):
        word |= u[:, :, j] << (4 * j)
    word = torch.where(word >= 2 ** 31, word - 2 ** 32, word)
    return word.to(torch.int32)


def unpack_int4_words(words):
    k, n8 = words.shape
    w = words.to(torch.int64) & 0xFFFFFFFF
    out = torch.empty(k, n8, 8, dtype=torch.int64)
    for j in range(8):
        out[:, :, j] = (w >> (4 * j)) & 0xF
    out = torch.where(out >= 8, out - 16, out)
    return out.reshape(k, n8 * 8).to(torch.int32)


def pack_nibbles_k(codes_nk):
    """Signed int4 codes [N,K] -> this repo's deploy layout: uint8 [N,K/2],
    stored unsigned (code+8), low nibble = even k."""
    u = (codes_nk.to(torch.int64) + 8)
    return (u[:, 0::2] | (u[:, 1::2] << 4)).to(torch.uint8)


def unpack_nibbles_k(packed):
    p = packed.to(torch.int64)
    out = torch.empty(p.shape[0], p.shape[1] * 2, dtype=torch.int64)
    out[:, 0::2] = p & 0xF
    out[:, 1::2] = p >> 4
    return (out - 8).to(torch.int32)


def w4a16_buffers(weight, bias, scale_w, offset_w, wts_type, group_size=None, awq_scale=None):
    """Reference-layout deploy buffers (weight_npu_quant_module.py:29-100):
    quantized_weight [K,N] (int8, or int4 packed to [K,N/8] int32), scale_w and
    offset_w (= -offset) in the weight dtype, [K/g,N]."""
    out = {}
    w = weight
    shape = w.shape
    if awq_scale is not None:
        w = iq.awq_weight(w, awq_scale)
        out['scale_factor'] = awq_scale
    else:
        out['scale_factor'] = None
    codes = iq.quant_codes(w, wts_type, scale_w, offset_w, group_size)
    if group_size is not None:
        sw = scale_w.reshape(scale_w.shape[0], scale_w.shape[1])
        ow = offset_w.reshape(offset_w.shape[0], offset_w.shape[1]) if offset_w is not None else None
        codes = codes.reshape(codes.shape[0], -1)[:, :shape[1]] if codes.dim() == 3 else codes
        g = group_size
    else:
        sw = scale_w.reshape(-1, 1) if scale_w.dim() == 1 else scale_w
        sw = sw.repeat(shape[0], 1) if sw.shape[0] == 1 else sw
        ow = offset_w
        if ow is not None:
            ow = ow.reshape(-1, 1) if ow.dim() == 1 else ow
            ow = ow.repeat(shape[0], 1) if ow.shape[0] == 1 else ow
        g = 0
    out['codes_nk'] = codes                                   # signed, [N,K]
    qw = codes.transpose(-1, -2).contiguous()
    if wts_type == 'int4':
        qw = pack_int4_words(qw)
    out['quantized_weight'] = qw
    out['scale_w'] = sw.to(weight.dtype).transpose(-1, -2).contiguous()
    out['offset_w'] = (ow * -1).to(weight.dtype).transpose(-1, -2).contiguous() if ow is not None else None
    b = None
    if bias is not None:
        b = bias.to(torch.float32) if weight.dtype == torch.bfloat16 else bias
    out['bias'] = b
    out['group_size'] = g
    return out


def dequant_weight(codes_nk, scale_nk_g, antioffset_nk_g, group_size, dtype):
    """(q + antiquant_offset) * antiquant_scale, exact in fp32, rounded once to `dtype` -- or, with dtype None, left
    exact (fp64).  scale/offset are [N,G] (G=1 for per-channel).
    Both readings of the un-vendored operator are kept: the matrix pipe takes 16-bit operands, so the tile kernels
    round the dequantised weight to the activation dtype; the reference's CPU stand-in for the operator
    (tests/amct_pytorch/mock_torch_npu.py:33-55) multiplies in fp32 and rounds nothing, which is what the
    weight-streaming kernel for a few rows reproduces (integer weights in the matrix pipe, scale applied per group)."""
    n, k = codes_nk.shape
    g = group_size if group_size else k
    if dtype is None:
        q = iq.group_view(codes_nk.double(), g)
        s = scale_nk_g.double().reshape(n, -1, 1)
        if antioffset_nk_g is not None:
            q = q + antioffset_nk_g.double().reshape(n, -1, 1)
        return (q * s).reshape(n, -1)[:, :k]
    q = iq.group_view(codes_nk.float(), g)                    # [N,G,g]
    s = scale_nk_g.float().reshape(n, -1, 1)
    if antioffset_nk_g is not None:
        q = q + antioffset_nk_g.float().reshape(n, -1, 1)
    return (q * s).reshape(n, -1)[:, :k].to(dtype)


def weight_quant_matmul_f64(x2d, wdq_nk, bias=None):
    """fp64 anchor of x @ Wdq^T (+ bias)."""
    y = x2d.double() @ wdq_nk.double().t()
    if bias is not None:
        y = y + bias.double()
    return y


def w4a16_forward_f64(x, codes_nk, scale_ng, antioffset_ng, group_size, bias=None, scale_factor=None, round_weight=True):
    """Module forward (weight_npu_quant_module.py:102-121) with the contraction in fp64: x' = x*scale_factor rounded
    to x's dtype, weight dequantised (rounded to x's dtype, or exact with round_weight=False), exact products, fp64
    sum.  Returns fp64 [.., N]."""
    shp = x.shape
    x2 = x.reshape(-1, shp[-1])
    if scale_factor is not None:
        x2 = torch.mul(x2, scale_factor.to(x2.dtype))
    wdq = dequant_weight(codes_nk, scale_ng, antioffset_ng, group_size, x.dtype if round_weight else None)
    return weight_quant_matmul_f64(x2, wdq, bias).reshape(*shp[:-1], -1)


def smoothed_rows(x, scale_factor=None):
    """x' of the forward (weight_npu_quant_module.py:112-114): rows flattened, times scale_factor, rounded to x's dtype."""
    x2 = x.reshape(-1, x.shape[-1])
    if scale_factor is not None:
        x2 = torch.mul(x2, scale_factor.to(x2.dtype))
    return x2


def weight_only_error_bounds(x2d, w_exact_nk):
    """How far a kernel that rounds the dequantised weight to x's dtype may be from the exact result
    (w4a16_forward_f64 with round_weight=False), per output, derived from the arithmetic alone.  x2d: the smoothed
    activations [M, K] (smoothed_rows), w_exact_nk: dequant_weight(..., dtype=None).

    Rounding w to nearest in a format with p significand bits (hidden bit included) gives w(1 + d) with
    |d| <= u = 2^-p (bf16: p = 8, u = 2^-8; fp16: p = 11, u = 2^-11), so the output moves by sum_k x'_k w_k d_k:
      hard   u * sum_k |x'_k w_k|                       (every d_k at its limit with the worst sign)
      likely 7 u * sqrt(sum_k (x'_k w_k)^2)             (Hoeffding for independent bounded errors: exceeded with
                                                         probability < 2 exp(-24.5) = 5e-11 per output)
    Returns (hard, likely) as fp64 [M, N]."""
    u = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[x2d.dtype]
    xa, wa = x2d.double().abs(), w_exact_nk.double().abs()
    hard = u * (xa @ wa.t())
    likely = 7.0 * u * torch.sqrt((xa * xa) @ (wa * wa).t())
    return hard, likely


# --------------------------------------------------------------------------
# the reference's CPU stand-ins for the two matmul operators, as the timed CPU baseline of bench.py
# --------------------------------------------------------------------------
def cpu_standin_quant_matmul_f32(xq, wq_nk, scale, pertoken_scale=None, bias=None, output_dtype=torch.bfloat16):
    """What the reference's tests run for npu_quant_matmul when no NPU is present
    (tests/amct_pytorch/mock_torch_npu.py:58-67): operands upcast to fp32, one fp32 F.linear, the per-channel factor
    (plus the per-token factor, which the stand-in leaves out), cast.  fp32 accumulation is NOT exact at K = 4096,
    so this is a speed baseline only, never a checker."""
    out = torch.nn.functional.linear(xq.to(torch.float32), wq_nk.to(torch.float32), None)
    out *= scale.reshape(1, -1)
    if pertoken_scale is not None:
        out *= pertoken_scale.reshape(-1, 1)
    if bias is not None:
        out += bias.to(torch.float32)
    return out.to(output_dtype)


def cpu_standin_weight_quant_matmul_f32(x, codes_nk, scale_ng, antioffset_ng, group_size, bias=None, scale_factor=None):
    """mock_torch_npu.py:33-55 with the group-wise factors the operator takes: x * scale_factor in x's dtype
    (weight_npu_quant_module.py:113-114), fp32 dequantise, fp32 F.linear, cast to x's dtype.  Speed baseline only."""
    x2 = x.reshape(-1, x.shape[-1])
    if scale_factor is not None:
        x2 = torch.mul(x2, scale_factor.to(x2.dtype))
    wdq = dequant_weight(codes_nk, scale_ng, antioffset_ng, group_size, torch.float32)
    out = torch.nn.functional.linear(x2.float(), wdq, None if bias is None else bias.float())
    return out.to(x.dtype)


# --------------------------------------------------------------------------
# interchange formats of the checkpoint converter
# (amct_pytorch/experimental/quantization/DeepSeekV3.2/deploy.py)
# --------------------------------------------------------------------------
def fp8_block_dequant(weight, scale, block_size=128, out_dtype=torch.bfloat16):
    """weight_dequant :48-92 -- fp32(weight) * scale expanded per block, one rounding to out_dtype.
    Pinned by tests/test_oracle_int.py::test_interchange_known_answers (exact products of powers of two)."""
    m, n = weight.shape
    s = scale.repeat_interleave(block_size, dim=0).repeat_interleave(block_size, dim=1)[:m, :n]
    return (weight.to(torch.float32) * s).to(out_dtype)


def pack_4bit(x):
    """pack_4bit :110-127 -- pairs of output channels per byte, returned [n/2, k]."""
    x = x.T.contiguous()
    shape = x.shape
    x = x.view(-1, 2)
    y = torch.bitwise_or(x[:, 0] & 0b00001111, torch.bitwise_left_shift(x[:, 1], 4))
    return y.view(shape[0], shape[1] // 2).T.contiguous()


def scale_fp32_to_u64(weight_scale):
    """scale_fp32_to_u64 :95-107 -- the fp32 bits in the low half of a 64-bit word (as int64 here)."""
    import numpy as np
    bits = weight_scale.float().cpu().numpy().view(np.uint32).astype(np.uint64)
    return torch.from_numpy(bits.astype(np.int64))
