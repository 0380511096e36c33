"""Tensor-level wrappers around the C ABI: allocate outputs with torch, pass raw
device pointers and the current HIP stream, raise on error codes.  All
arithmetic happens in the HIP kernels; torch is used for memory only.
"""
import contextlib

import torch

from . import _lib
from ._lib import (BF16, CODES_I8, CODES_I32, CODES_NONE, COL_DIV, COL_MUL, COL_MUL_THEN_DIV, COL_NONE, F16, F32,
                   MX_E2M1, MX_E4M3, MX_FLOOR, MX_RCEIL, SCOPE_ABSMAX, SCOPE_AMCT, STAGE_COL, STAGE_DEQUANT,
                   STAGE_FULL, STAGE_SCALE)

_DT = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}


def dtype_code(dt):
    try:
        return _DT[dt]
    except KeyError:
        raise RuntimeError(
            "dtype {} not support now, only support float32/float16/bfloat16.".format(dt)) from None


def _dev(*tensors):
    """All tensors must live on one HIP device; there is no CPU path."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("amct_amd kernels run on the GPU only: got a tensor on '{}'".format(t.device))
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError("amct_amd: tensors on different devices ({} vs {})".format(dev, t.device))
    return dev


def _p(t):
    return None if t is None else t.data_ptr()


def _need(cond, msg, *args):
    """Host-side operand check: the kernels only see pointers, so every size they rely on is verified here,
    before anything is launched."""
    if not cond:
        raise RuntimeError(msg.format(*args))


def _segments(rows, cols, group):
    """Number of (scale, offset) entries for a [rows, cols] tensor: per group, per row (0) or per tensor (-1)."""
    if group > 0:
        return rows * ((cols + group - 1) // group)
    return rows if group == 0 else 1


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_SAME_DEVICE = contextlib.nullcontext()


def _stream(dev):
    """Handle of torch's current stream on dev (the raw getter skips building a Stream object per call)."""
    if _raw_stream is not None and dev.index is not None:
        return _raw_stream(dev.index)
    return torch.cuda.current_stream(dev).cuda_stream


def _on(dev):
    """Device guard for a launch: nothing to switch (the common case) when dev is already current."""
    if dev.index is None or dev.index == torch.cuda.current_device():
        return _SAME_DEVICE
    return torch.cuda.device(dev)


def _c(t):
    return t if t.is_contiguous() else t.contiguous()


# Scratch memory the GEMM wrappers lend to the library (it never allocates): ONE grow-only byte tensor per device and
# stream, shared by every call on that stream.  Calls on one stream run in order, so they can share it; a fresh
# torch.empty per forward would pass a dequantise-once call (the weight as 16 bits: N * K * 2 bytes) through the
# allocator every time.  `workspace_limit_bytes` caps what is lent: a call that asks for more gets the capped size and
# the library then takes the kernels that need less (documented per entry point: never an error), which bounds the
# memory a deployment pays for the faster many-row kernels.  None: no cap.
workspace_limit_bytes = None
_WORKSPACES = {}


def lent_workspace(dev, nbytes):
    """A uint8 tensor of at least min(nbytes, workspace_limit_bytes) bytes on dev for the current stream, or None."""
    if workspace_limit_bytes is not None:
        nbytes = min(nbytes, int(workspace_limit_bytes))
    if nbytes <= 0:
        return None
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), _stream(dev))
    ws = _WORKSPACES.get(key)
    if ws is None or ws.numel() < nbytes:
        _WORKSPACES.pop(key, None)                   # let the smaller one go before the larger one is allocated
        ws = None
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        _WORKSPACES[key] = ws
    return ws


def release_workspaces():
    """Drops the lent scratch tensors (they come back on the next call that needs one)."""
    _WORKSPACES.clear()


# ---------------------------------------------------------------------------
# A1 / A2
# ---------------------------------------------------------------------------
def minmax(w, group=0):
    """w [rows, cols] -> (min, max) fp32, shape [rows] (group=0) or [rows, ceil(cols/group)]."""
    dev = _dev(w)
    w = _c(w)
    rows, cols = w.shape
    n = rows if group == 0 else rows * ((cols + group - 1) // group)
    mn = torch.empty(n, dtype=torch.float32, device=dev)
    mx = torch.empty(n, dtype=torch.float32, device=dev)
    with _on(dev):
        _lib.check(_lib.load().amct_minmax(_p(w), _p(mn), _p(mx), rows, cols, group, dtype_code(w.dtype), _stream(dev)))
    if group:
        return mn.reshape(rows, -1), mx.reshape(rows, -1)
    return mn, mx


def col_minmax(x, col_max=None, col_min=None, absolute=False):
    """Per-column (input channel) max and min over all rows of x [rows, cols] -> fp32 [cols] each.
    With col_max / col_min given (fp32 [cols]) the running update `batch > old ? batch : old` is applied to
    them in place and they are returned; absolute=True reduces |x| and returns only the maximum."""
    _need(x.dim() == 2, "col_minmax expects a 2-D tensor, got {} dims", x.dim())
    rows, cols = x.shape
    for name, t in (("col_max", col_max), ("col_min", col_min)):
        _need(t is None or (t.dtype == torch.float32 and t.numel() == cols and t.is_contiguous()),
              "col_minmax: {} must be a contiguous fp32 tensor of {} elements", name, cols)
    dev = _dev(x, col_max, col_min)
    x = _c(x)
    accumulate = col_max is not None or col_min is not None
    # a running tensor the caller did not pass starts at the neutral element of its update, so that the
    # accumulating kernel never folds uninitialised memory into the result
    if col_max is None:
        col_max = torch.full((cols,), float('-inf'), dtype=torch.float32, device=dev) if accumulate else \
            torch.empty(cols, dtype=torch.float32, device=dev)
    if col_min is None and not absolute:
        col_min = torch.full((cols,), float('inf'), dtype=torch.float32, device=dev) if accumulate else \
            torch.empty(cols, dtype=torch.float32, device=dev)
    lib = _lib.load()
    nbytes = lib.amct_col_minmax_workspace_bytes(rows, cols)
    ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device=dev)
    with _on(dev):
        _lib.check(lib.amct_col_minmax(_p(x), _p(col_max), None if absolute else _p(col_min), rows, cols, int(absolute),
                                       int(accumulate), dtype_code(x.dtype), _p(ws), nbytes, _stream(dev)))
    return col_max if absolute else (col_max, col_min)


def awq_loss(y, yhat):
    """mean((y - yhat)^4) as a 0-d fp32 tensor on the device, the difference rounded to the tensors' dtype
    (algorithm/awq.py:96); one pass over both tensors."""
    dev = _dev(y, yhat)
    if y.dtype != yhat.dtype or y.shape != yhat.shape:
        raise RuntimeError("awq_loss: the two outputs must share dtype and shape")
    y, yhat = _c(y), _c(yhat)
    lib = _lib.load()
    nbytes = lib.amct_awq_loss_workspace_bytes()
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    loss = torch.empty((), dtype=torch.float32, device=dev)
    with _on(dev):
        _lib.check(lib.amct_awq_loss(_p(y), _p(yhat), y.numel(), dtype_code(y.dtype), _p(loss), _p(ws), nbytes, _stream(dev)))
    return loss


def hessian_update(hessian, x, beta, alpha):
    """hessian [C,C] fp32 <- beta * hessian + alpha * x^T x in place, x [tokens, C] bf16|f16 (gptq_module.py:176-181).
    beta == 0 does not read hessian."""
    dev = _dev(hessian, x)
    _need(hessian.dim() == 2 and hessian.shape[0] == hessian.shape[1] and hessian.dtype == torch.float32 and
          hessian.is_contiguous(), "hessian_update: the Hessian must be a contiguous square fp32 matrix")
    _need(x.dim() == 2 and x.shape[1] == hessian.shape[0], "hessian_update: x must be [tokens, {}]".format(hessian.shape[0]))
    _need(x.dtype in (torch.bfloat16, torch.float16), "hessian_update: 16-bit activations only")
    x = _c(x)
    lib = _lib.load()
    tokens, cols = x.shape
    nbytes = lib.amct_hessian_update_workspace_bytes(tokens, cols)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)
    with _on(dev):
        _lib.check(lib.amct_hessian_update(_p(hessian), _p(x), tokens, cols, float(beta), float(alpha), dtype_code(x.dtype),
                                           _p(ws), ws.numel(), _stream(dev)))
    return hessian


def scale_offset(vmax, vmin, bits, symmetric, scope_rule=SCOPE_AMCT, bad=None):
    """Elementwise (max, min) -> (scale fp32, offset int32 | None), same shape as the inputs."""
    dev = _dev(vmax, vmin, bad)
    if vmax.dtype != vmin.dtype or vmax.shape != vmin.shape:
        raise RuntimeError("max and min must share dtype and shape")
    vmax, vmin = _c(vmax), _c(vmin)
    scale = torch.empty(vmax.shape, dtype=torch.float32, device=dev)
    offset = None if symmetric else torch.empty(vmax.shape, dtype=torch.int32, device=dev)
    with _on(dev):
        _lib.check(_lib.load().amct_scale_offset(_p(vmax), _p(vmin), _p(scale), _p(offset), _p(bad), vmax.numel(), bits,
                                                 int(symmetric), scope_rule, dtype_code(vmax.dtype), _stream(dev)))
    return scale, offset


# ---------------------------------------------------------------------------
# A3..A6 with given factors
# ---------------------------------------------------------------------------
def quant_with_params(w, scale, offset, group, qmin, qmax, want_dq=True, codes_kind=CODES_NONE, col_scale=None,
                      col_mode=COL_NONE, via_src=False, stage=STAGE_FULL):
    """group: >0 per group, 0 per row, -1 per tensor.  Returns (dq | None, codes | None)."""
    _need(w.dim() == 2, "quantise expects a 2-D tensor, got {} dims", w.dim())
    rows, cols = w.shape
    nseg = _segments(rows, cols, group)
    _need(scale.numel() == nseg, "scale has {} entries, the tensor [{}, {}] with group {} needs {}", scale.numel(), rows,
          cols, group, nseg)
    _need(offset is None or offset.numel() == nseg, "offset has {} entries, {} expected",
          0 if offset is None else offset.numel(), nseg)
    _need(col_scale is None or col_scale.numel() == cols, "column scale has {} entries, {} columns",
          0 if col_scale is None else col_scale.numel(), cols)
    dev = _dev(w, scale, offset, col_scale)
    w = _c(w)
    scale = _c(scale.to(torch.float32))
    if offset is not None:
        offset = _c(offset.to(torch.int32))
    dq = torch.empty_like(w) if want_dq else None
    codes = None
    if codes_kind == CODES_I8:
        codes = torch.empty(w.shape, dtype=torch.int8, device=dev)
    elif codes_kind == CODES_I32:
        codes = torch.empty(w.shape, dtype=torch.int32, device=dev)
    if col_scale is not None:
        col_scale = _c(col_scale.to(w.dtype))
    with _on(dev):
        _lib.check(_lib.load().amct_quant_with_params(
            _p(w), _p(scale), _p(offset), _p(dq), _p(codes), codes_kind, _p(col_scale), col_mode, rows, cols, group,
            qmin, qmax, int(via_src), stage, dtype_code(w.dtype), _stream(dev)))
    return dq, codes


def col_scale(w, c, divide):
    """w * c[k] (or w / c[k]) rounded to w's dtype; c is [1,K] or [K]."""
    dev = _dev(w, c)
    one = torch.ones(1, dtype=torch.float32, device=dev)
    out, _ = quant_with_params(w, one, None, -1, -128, 127, col_scale=c.reshape(-1),
                               col_mode=COL_DIV if divide else COL_MUL, stage=STAGE_COL)
    return out


# ---------------------------------------------------------------------------
# K1 fused
# ---------------------------------------------------------------------------
def fakequant_int(w, bits, symmetric, group=0, want_dq=True, codes_kind=CODES_NONE, scope_rule=SCOPE_AMCT,
                  qmin=None, qmax=None, col_scale=None, col_mode=COL_NONE, via_src=False, bad=None):
    """One pass over w: min/max -> factors -> quantise.  Returns (dq, codes, scale, offset);
    scale/offset are flat [rows] (group=0) or [rows, cols/group]."""
    _need(w.dim() == 2, "quantise expects a 2-D tensor, got {} dims", w.dim())
    rows, cols = w.shape
    _need(group >= 0, "the fused kernel takes per-row (0) or per-group (> 0) factors, got group {}", group)
    _need(col_scale is None or col_scale.numel() == cols, "column scale has {} entries, {} columns",
          0 if col_scale is None else col_scale.numel(), cols)
    dev = _dev(w, col_scale, bad)
    w = _c(w)
    nseg = _segments(rows, cols, group)
    if qmin is None:
        qmin = -(1 << (bits - 1))
    if qmax is None:
        qmax = (1 << (bits - 1)) - 1
    scale = torch.empty(nseg, dtype=torch.float32, device=dev)
    offset = None if symmetric else torch.empty(nseg, dtype=torch.int32, device=dev)
    dq = torch.empty_like(w) if want_dq else None
    codes = None
    if codes_kind == CODES_I8:
        codes = torch.empty(w.shape, dtype=torch.int8, device=dev)
    elif codes_kind == CODES_I32:
        codes = torch.empty(w.shape, dtype=torch.int32, device=dev)
    if col_scale is not None:
        col_scale = _c(col_scale.to(w.dtype))
    with _on(dev):
        _lib.check(_lib.load().amct_fakequant_int(
            _p(w), _p(dq), _p(codes), codes_kind, _p(scale), _p(offset), _p(bad), _p(col_scale), col_mode, rows, cols,
            group, bits, int(symmetric), scope_rule, qmin, qmax, int(via_src), dtype_code(w.dtype), _stream(dev)))
    if group:
        scale = scale.reshape(rows, -1)
        offset = offset.reshape(rows, -1) if offset is not None else None
    return dq, codes, scale, offset


# ---------------------------------------------------------------------------
# K2
# ---------------------------------------------------------------------------
def quant_int4_group_pack(w, group, symmetric=False, scale_dtype=torch.float16, want_scales32=False, col_scale=None,
                          col_mode=COL_NONE, bad=None):
    """w [N,K] -> (packed uint8 [N,K/2], scales16 [N,K/g], zeros uint8 [N,K/g], scales32 | None)."""
    _need(w.dim() == 2, "quantise expects a 2-D tensor, got {} dims", w.dim())
    rows, cols = w.shape
    if group <= 0 or cols % group or group % 32:
        raise ValueError("int4 group pack needs cols % group == 0 and group % 32 == 0")
    _need(col_scale is None or col_scale.numel() == cols, "column scale has {} entries, {} columns",
          0 if col_scale is None else col_scale.numel(), cols)
    dev = _dev(w, col_scale, bad)
    w = _c(w)
    g = cols // group
    packed = torch.empty(rows, cols // 2, dtype=torch.uint8, device=dev)
    s16 = torch.empty(rows, g, dtype=scale_dtype, device=dev)
    s32 = torch.empty(rows, g, dtype=torch.float32, device=dev) if want_scales32 else None
    zeros = torch.empty(rows, g, dtype=torch.uint8, device=dev)
    if col_scale is not None:
        col_scale = _c(col_scale.to(w.dtype))
    with _on(dev):
        _lib.check(_lib.load().amct_quant_int4_group_pack(
            _p(w), _p(packed), _p(s16), dtype_code(scale_dtype), _p(s32), _p(zeros), _p(bad), _p(col_scale), col_mode,
            rows, cols, group, int(symmetric), dtype_code(w.dtype), _stream(dev)))
    return packed, s16, zeros, s32


def pack_int4_words(codes_i32):
    """int32 [k,n] (one signed int4 each) -> int32 [k,n/8]."""
    dev = _dev(codes_i32)
    codes_i32 = _c(codes_i32)
    if codes_i32.dtype != torch.int32 or codes_i32.dim() != 2:
        raise RuntimeError("int4 packing expects a 2-D int32 tensor")
    k, n = codes_i32.shape
    if n % 8:
        raise RuntimeError("int4 packing needs the last dim to be a multiple of 8")
    words = torch.empty(k, n // 8, dtype=torch.int32, device=dev)
    with _on(dev):
        _lib.check(_lib.load().amct_pack_int4_words(_p(codes_i32), _p(words), k, n, _stream(dev)))
    return words


def words_to_nibbles_nk(words, k, n):
    """int32 [k,n/8] -> uint8 [n,k/2] (code+8, even k in the low nibble)."""
    dev = _dev(words)
    words = _c(words)
    packed = torch.empty(n, k // 2, dtype=torch.uint8, device=dev)
    with _on(dev):
        _lib.check(_lib.load().amct_words_to_nibbles_nk(_p(words), _p(packed), k, n, _stream(dev)))
    return packed


def pack_nibbles_nk(codes_i8):
    """int8 [N,K] signed int4 codes -> uint8 [N,K/2] (code+8, even k in the low nibble)."""
    dev = _dev(codes_i8)
    codes_i8 = _c(codes_i8)
    if codes_i8.dtype != torch.int8 or codes_i8.shape[1] % 2:
        raise RuntimeError("nibble packing expects int8 codes with an even number of columns")
    n, k = codes_i8.shape
    packed = torch.empty(n, k // 2, dtype=torch.uint8, device=dev)
    with _on(dev):
        _lib.check(_lib.load().amct_pack_nibbles_nk(_p(codes_i8), _p(packed), n, k, _stream(dev)))
    return packed


def unpack_nibbles_to_i32_kn(packed):
    """uint8 [N,K/2] -> int32 [K,N] signed codes."""
    dev = _dev(packed)
    packed = _c(packed)
    n, k = packed.shape[0], packed.shape[1] * 2
    codes = torch.empty(k, n, dtype=torch.int32, device=dev)
    with _on(dev):
        _lib.check(_lib.load().amct_nibbles_nk_to_codes_kn(_p(packed), _p(codes), k, n, _stream(dev)))
    return codes


def bias_to_int32(bias, scale):
    """round_half_even(bias / scale) as int32 (amct_pytorch/deploy_op/npu_quantization_linear.py:117-120)."""
    scale = scale.reshape(-1)
    _, codes = quant_with_params(bias.reshape(-1, 1), scale, None, 0 if scale.numel() > 1 else -1,
                                 -2147483648, 2147483647, want_dq=False, codes_kind=CODES_I32)
    return codes.reshape(-1)


# ---------------------------------------------------------------------------
# K3
# ---------------------------------------------------------------------------
def act_quant_per_token_int8(x, smooth=None, mode=0):
    """x [..., K] -> (int8 same shape, scale fp32 [rows])."""
    dev = _dev(x, smooth)
    x = _c(x)
    K = x.shape[-1]
    M = x.numel() // K
    q = torch.empty(x.shape, dtype=torch.int8, device=dev)
    s = torch.empty(M, dtype=torch.float32, device=dev)
    if smooth is not None:
        smooth = _c(smooth.reshape(-1).to(x.dtype))
        if smooth.numel() != K:
            raise RuntimeError("smooth factor must have K elements")
    with _on(dev):
        _lib.check(_lib.load().amct_act_quant_per_token_int8(_p(x), _p(smooth), _p(q), _p(s), M, K, mode,
                                                             dtype_code(x.dtype), _stream(dev)))
    return q, s


def quantize_static(x, scales, zero_points, per_token, smooth=None):
    """q = sat_int8(rne(x * scales + zero_points)); x [..., M, K]."""
    dev = _dev(x, scales, zero_points, smooth)
    x = _c(x)
    K = x.shape[-1]
    rows = x.numel() // K
    scales = _c(scales.reshape(-1).to(x.dtype))
    if zero_points is not None:
        zero_points = _c(zero_points.reshape(-1).to(x.dtype))
    if smooth is not None:
        smooth = _c(smooth.reshape(-1).to(x.dtype))
    n_scales = scales.numel()
    if per_token:
        # one scale per row of the last-but-one dim, shared by every leading batch index
        m = x.shape[-2]
        if n_scales != m:
            raise RuntimeError("per-token quantize needs one scale per token ({} vs {})".format(n_scales, m))
        reps = rows // m
        if reps > 1:
            scales = scales.repeat(reps)
            zero_points = zero_points.repeat(reps) if zero_points is not None else None
            n_scales = rows
    q = torch.empty(x.shape, dtype=torch.int8, device=dev)
    with _on(dev):
        _lib.check(_lib.load().amct_quantize(_p(x), _p(smooth), _p(scales), _p(zero_points), _p(q), rows, K, n_scales,
                                             int(per_token), dtype_code(x.dtype), _stream(dev)))
    return q


# ---------------------------------------------------------------------------
# K4 / K5
# ---------------------------------------------------------------------------
def mx_quant(x, fmt, scale_mode=MX_FLOOR):
    dev = _dev(x)
    x = _c(x)
    cols = x.shape[-1]
    rows = x.numel() // cols
    if cols % 32:
        raise ValueError("MX quantisation needs the last dim to be a multiple of 32")
    el = torch.empty(*x.shape[:-1], cols if fmt == MX_E4M3 else cols // 2, dtype=torch.uint8, device=dev)
    e8 = torch.empty(*x.shape[:-1], cols // 32, dtype=torch.uint8, device=dev)
    with _on(dev):
        _lib.check(_lib.load().amct_mx_quant(_p(x), _p(el), _p(e8), rows, cols, fmt, scale_mode, dtype_code(x.dtype),
                                             _stream(dev)))
    return el, e8


def mx_dequant(el, e8, fmt, dtype=torch.bfloat16):
    cols = e8.shape[-1] * 32
    rows = e8.numel() // max(e8.shape[-1], 1)
    want = tuple(e8.shape[:-1]) + (cols if fmt == MX_E4M3 else cols // 2,)
    _need(el.dtype == torch.uint8 and e8.dtype == torch.uint8, "MX elements and shared exponents are uint8 tensors")
    _need(tuple(el.shape) == want, "MX elements have shape {}, the shared exponents {} imply {}", tuple(el.shape),
          tuple(e8.shape), want)
    dev = _dev(el, e8)
    el, e8 = _c(el), _c(e8)
    y = torch.empty(*e8.shape[:-1], cols, dtype=dtype, device=dev)
    with _on(dev):
        _lib.check(_lib.load().amct_mx_dequant(_p(el), _p(e8), _p(y), rows, cols, fmt, dtype_code(dtype), _stream(dev)))
    return y


def hif8_encode(x, saturate=False):
    dev = _dev(x)
    x = _c(x)
    y = torch.empty(x.shape, dtype=torch.uint8, device=dev)
    with _on(dev):
        _lib.check(_lib.load().amct_hif8_encode(_p(x), _p(y), x.numel(), dtype_code(x.dtype), int(saturate), _stream(dev)))
    return y


def hif8_decode(c, dtype=torch.bfloat16):
    dev = _dev(c)
    c = _c(c)
    y = torch.empty(c.shape, dtype=dtype, device=dev)
    with _on(dev):
        _lib.check(_lib.load().amct_hif8_decode(_p(c), _p(y), c.numel(), dtype_code(dtype), _stream(dev)))
    return y


# ---------------------------------------------------------------------------
# K6 / K7
# ---------------------------------------------------------------------------
def gemm_w8a8(xq, wq_nk, s_ch, s_tok=None, bias=None, out_dtype=torch.bfloat16, want_acc=False):
    """xq int8 [M,K], wq_nk int8 [N,K] (K contiguous) -> out [M,N] (and int32 accumulators)."""
    _need(xq.dim() == 2 and wq_nk.dim() == 2, "int8 GEMM expects 2-D operands")
    _need(xq.dtype == torch.int8 and wq_nk.dtype == torch.int8, "int8 GEMM expects int8 operands")
    M, K = xq.shape
    N = wq_nk.shape[0]
    if wq_nk.shape[1] != K:
        raise RuntimeError("int8 GEMM: K mismatch ({} vs {})".format(K, wq_nk.shape[1]))
    _need(s_ch.numel() in (1, N), "int8 GEMM: {} channel scales for {} output channels", s_ch.numel(), N)
    _need(s_tok is None or s_tok.numel() == M, "int8 GEMM: {} token scales for {} rows",
          0 if s_tok is None else s_tok.numel(), M)
    _need(bias is None or bias.numel() == N, "int8 GEMM: bias has {} entries, {} output channels",
          0 if bias is None else bias.numel(), N)
    dev = _dev(xq, wq_nk, s_ch, s_tok, bias)
    xq, wq_nk = _c(xq), _c(wq_nk)
    s_ch = _c(s_ch.reshape(-1).to(torch.float32))
    if s_ch.numel() == 1:
        s_ch = s_ch.expand(N).contiguous()
    if s_tok is not None:
        s_tok = _c(s_tok.reshape(-1).to(torch.float32))
    kind = 0
    if bias is not None:
        if bias.dtype == torch.int32:
            kind = 1
            bias = _c(bias)
        else:
            kind = 2
            bias = _c(bias.to(torch.float32))
    out = torch.empty(M, N, dtype=out_dtype, device=dev)
    acc = torch.empty(M, N, dtype=torch.int32, device=dev) if want_acc else None
    # the workspace the library asks for (partial sums, when it splits long rows over several blocks per tile)
    ws = lent_workspace(dev, _lib.load().amct_gemm_w8a8_workspace_bytes(M, N, K))
    with _on(dev):
        _lib.check(_lib.load().amct_gemm_w8a8_ws(_p(xq), _p(wq_nk), _p(s_tok), _p(s_ch), _p(bias), kind, _p(out), _p(acc),
                                                 M, N, K, dtype_code(out_dtype), _p(ws), 0 if ws is None else ws.numel(),
                                                 _stream(dev)))
    return (out, acc) if want_acc else out


def linear_w8a8(x, act_scale, act_offset, per_token, wq_nk, s_ch, s_tok=None, bias=None, out_dtype=torch.bfloat16,
                smooth=None):
    """quantize_static followed by gemm_w8a8 in one library call (the forward of the W8A8 deploy module): x [M,K]
    fp32|fp16|bf16; act_scale / act_offset one per tensor or (per_token) one per row, in x's dtype; the other operands as
    for gemm_w8a8.  Up to 16 rows the activations are quantised inside the weight-streaming kernel."""
    _need(x.dim() == 2 and wq_nk.dim() == 2 and wq_nk.dtype == torch.int8, "W8A8 Linear expects x [M,K] and an int8 weight [N,K]")
    M, K = x.shape
    N = wq_nk.shape[0]
    _need(wq_nk.shape[1] == K, "W8A8 Linear: K mismatch ({} vs {})", K, wq_nk.shape[1])
    _need(s_ch.numel() in (1, N), "W8A8 Linear: {} channel scales for {} output channels", s_ch.numel(), N)
    _need(s_tok is None or s_tok.numel() == M, "W8A8 Linear: {} token scales for {} rows",
          0 if s_tok is None else s_tok.numel(), M)
    _need(bias is None or bias.numel() == N, "W8A8 Linear: bias has {} entries, {} output channels",
          0 if bias is None else bias.numel(), N)
    n_scales = act_scale.numel()
    _need(n_scales == M if per_token else n_scales in (1, K), "W8A8 Linear: {} activation scales for x of shape {}",
          n_scales, tuple(x.shape))
    _need(act_offset is None or act_offset.numel() == n_scales, "W8A8 Linear: activation offsets do not match the scales")
    _need(smooth is None or smooth.numel() == K, "W8A8 Linear: smooth factor must have K elements")
    dev = _dev(x, act_scale, act_offset, wq_nk, s_ch, s_tok, bias, smooth)
    x, wq_nk = _c(x), _c(wq_nk)
    act_scale = _c(act_scale.reshape(-1).to(x.dtype))
    if act_offset is not None:
        act_offset = _c(act_offset.reshape(-1).to(x.dtype))
    if smooth is not None:
        smooth = _c(smooth.reshape(-1).to(x.dtype))
    s_ch = _c(s_ch.reshape(-1).to(torch.float32))
    if s_ch.numel() == 1:
        s_ch = s_ch.expand(N).contiguous()
    if s_tok is not None:
        s_tok = _c(s_tok.reshape(-1).to(torch.float32))
    kind = 0
    if bias is not None:
        if bias.dtype == torch.int32:
            kind, bias = 1, _c(bias)
        else:
            kind, bias = 2, _c(bias.to(torch.float32))
    out = torch.empty(M, N, dtype=out_dtype, device=dev)
    lib = _lib.load()
    # whatever the library asks for (the int8 activations of the two-kernel form, the GEMM's partial sums): which calls
    # quantise inside the weight-streaming kernel and need none of it is the library's rule, not restated here
    ws = lent_workspace(dev, lib.amct_linear_w8a8_workspace_bytes(M, N, K))
    with _on(dev):
        _lib.check(lib.amct_linear_w8a8(_p(x), dtype_code(x.dtype), _p(smooth), _p(act_scale), _p(act_offset), n_scales,
                                        int(bool(per_token)), _p(wq_nk), _p(s_tok), _p(s_ch), _p(bias), kind, _p(out), M, N, K,
                                        dtype_code(out_dtype), _p(ws), 0 if ws is None else ws.numel(), _stream(dev)))
    return out


def _check_weight_only(x, N, K, scales, zeros, group, smooth, bias, zeros_dtype, what):
    _need(x.dim() == 2 and x.shape[1] == K, "{}: activations must be [M, {}], got {}", what, K, tuple(x.shape))
    _need(x.dtype in (torch.bfloat16, torch.float16), "Not support tensor dtype {}, support dtypes {}.", x.dtype,
          [torch.bfloat16, torch.float16])
    _need(group > 0 and K % group == 0, "{}: K = {} is not a multiple of the group size {}", what, K, group)
    want = (N, K // group)
    _need(scales.dtype in (torch.float16, torch.bfloat16), "{}: scales must be fp16 or bf16, got {}", what, scales.dtype)
    _need(tuple(scales.shape) == want, "{}: scales have shape {}, expected {}", what, tuple(scales.shape), want)
    _need(zeros is None or (zeros.dtype == zeros_dtype and tuple(zeros.shape) == want),
          "{}: zero-points have shape {} / dtype {}, expected {} / {}", what,
          None if zeros is None else tuple(zeros.shape), None if zeros is None else zeros.dtype, want, zeros_dtype)
    _need(smooth is None or smooth.numel() == K, "{}: smooth factor has {} entries, K = {}", what,
          0 if smooth is None else smooth.numel(), K)
    _need(bias is None or bias.numel() == N, "{}: bias has {} entries, {} output channels", what,
          0 if bias is None else bias.numel(), N)


def gemm_w4a16_weight_rounded(M, N, K, group, dtype, workspace_bytes=None):
    """Whether amct_gemm_w4a16 rounds the dequantised weight to `dtype` for a call of this shape (True) or keeps it
    exact (False); workspace_bytes None: the workspace gemm_w4a16 lends."""
    lib = _lib.load()
    if workspace_bytes is None:
        workspace_bytes = lib.amct_gemm_w4a16_workspace_bytes(M, N, K, group, 0)
        if workspace_limit_bytes is not None:
            workspace_bytes = min(workspace_bytes, int(workspace_limit_bytes))
    r = lib.amct_gemm_w4a16_weight_rounded(M, N, K, group, dtype_code(dtype), workspace_bytes)
    if r < 0:
        _lib.check(r)
    return bool(r)


def gemm_w8a16_weight_rounded(M, N, K, group, dtype, workspace_bytes=None):
    """The same question for amct_gemm_w8a16_ws."""
    lib = _lib.load()
    if workspace_bytes is None:
        workspace_bytes = lib.amct_gemm_w8a16_workspace_bytes(M, N, K, group, 0)
        if workspace_limit_bytes is not None:
            workspace_bytes = min(workspace_bytes, int(workspace_limit_bytes))
    r = lib.amct_gemm_w8a16_weight_rounded(M, N, K, group, dtype_code(dtype), workspace_bytes)
    if r < 0:
        _lib.check(r)
    return bool(r)


def gemm_w4a16(x, wq_packed, scales, zeros, group, smooth=None, bias=None):
    """x [M,K] bf16|f16; wq_packed uint8 [N,K/2]; scales [N,K/g] f16|bf16; zeros uint8 [N,K/g]."""
    _need(wq_packed.dim() == 2 and wq_packed.dtype == torch.uint8, "int4 GEMM: the weight must be uint8 [N, K/2]")
    N, K = wq_packed.shape[0], wq_packed.shape[1] * 2
    if x.dim() == 2 and x.shape[1] != K:
        raise RuntimeError("int4 GEMM: K mismatch ({} vs {})".format(x.shape[1], K))
    _need(zeros is not None, "int4 GEMM: zero-points are required (8 everywhere for symmetric codes)")
    _check_weight_only(x, N, K, scales, zeros, group, smooth, bias, torch.uint8, "int4 GEMM")
    dev = _dev(x, wq_packed, scales, zeros, smooth, bias)
    x, wq_packed, scales, zeros = _c(x), _c(wq_packed), _c(scales), _c(zeros)
    M = x.shape[0]
    if smooth is not None:
        smooth = _c(smooth.reshape(-1).to(x.dtype))
    if bias is not None:
        bias = _c(bias.reshape(-1).to(torch.float32))
    out = torch.empty(M, N, dtype=x.dtype, device=dev)
    # the workspace the library asks for: the smoothed activations for the tile kernels, or the activation image the
    # weight-streaming kernel for a few rows fetches
    ws = lent_workspace(dev, _lib.load().amct_gemm_w4a16_workspace_bytes(M, N, K, group, int(smooth is not None)))
    with _on(dev):
        _lib.check(_lib.load().amct_gemm_w4a16(_p(x), _p(smooth), _p(wq_packed), _p(scales), dtype_code(scales.dtype),
                                               _p(zeros), _p(bias), _p(out), M, N, K, group, dtype_code(x.dtype),
                                               _p(ws), 0 if ws is None else ws.numel(), _stream(dev)))
    return out


def gemm_w8a16(x, wq_nk, scales, offsets, group, smooth=None, bias=None):
    """x [M,K] bf16|f16; wq_nk int8 [N,K] (K contiguous); scales [N,K/g] f16|bf16; offsets int8 [N,K/g] | None."""
    _need(wq_nk.dim() == 2 and wq_nk.dtype == torch.int8, "int8 weight-only GEMM: the weight must be int8 [N, K]")
    N, K = wq_nk.shape
    _check_weight_only(x, N, K, scales, offsets, group, smooth, bias, torch.int8, "int8 weight-only GEMM")
    dev = _dev(x, wq_nk, scales, offsets, smooth, bias)
    x, wq_nk, scales = _c(x), _c(wq_nk), _c(scales)
    offsets = None if offsets is None else _c(offsets)
    M = x.shape[0]
    if smooth is not None:
        smooth = _c(smooth.reshape(-1).to(x.dtype))
    if bias is not None:
        bias = _c(bias.reshape(-1).to(torch.float32))
    out = torch.empty(M, N, dtype=x.dtype, device=dev)
    # the workspace the library asks for: from 256 rows on, the dequantised weight (and the smoothed activations)
    ws = lent_workspace(dev, _lib.load().amct_gemm_w8a16_workspace_bytes(M, N, K, group, int(smooth is not None)))
    with _on(dev):
        _lib.check(_lib.load().amct_gemm_w8a16_ws(_p(x), _p(smooth), _p(wq_nk), _p(scales), dtype_code(scales.dtype),
                                                  _p(offsets), _p(bias), _p(out), M, N, K, group, dtype_code(x.dtype),
                                                  _p(ws), 0 if ws is None else ws.numel(), _stream(dev)))
    return out
