"""Operator-level drop-in for the four device operators the reference's deploy modules call
(torch_npu.npu_quantize, npu_quant_matmul, npu_weight_quant_batchmatmul,
npu_convert_weight_to_int4pack -- call sites amct_pytorch/deploy_op/npu_quantization_linear.py:98-102
and amct_pytorch/deploy_op/weight_npu_quant_module.py:54-57,116-117).  Same keyword names and operand
layouts as those calls; each runs HIP kernels only.

The weight operands arrive here in the reference's [K, N] layouts; their kernel layouts are computed on the
first call and cached per tensor and version for as long as the tensor lives (the deploy modules in
amct_amd.deploy_op convert once at construction instead).
"""
import torch

from . import ops


class _Npu:
    """Stand-in for the `torch_npu.npu` sub-namespace used at
    amct_pytorch/quantize_op/gptq_module.py:124-126."""

    @staticmethod
    def is_available():
        return torch.cuda.is_available()

    @staticmethod
    def empty_cache():
        torch.cuda.empty_cache()


npu = _Npu()


def npu_quantize(input, scales, zero_points=None, dtype=torch.int8, axis=-1, div_mode=False):
    """int8 = saturate(round_half_even(input * scales + zero_points)) with div_mode=False -- the call of
    amct_pytorch/deploy_op/npu_quantization_linear.py:98-99 -- or of input / scales + zero_points with div_mode=True
    (the operator's default; signature in tests/amct_pytorch/mock_torch_npu.py:69-70).  One scale per tensor, or one per
    index of `axis` (the last dim's neighbour, -2: per token).  The arithmetic inside torch_npu is not vendored:
    this library multiplies / divides and adds in fp32 (the division is the exactly rounded one of the weight
    quantiser, amct_quant_with_params) and rounds once.  Only dtype=torch.int8."""
    if dtype != torch.int8:
        raise RuntimeError("npu_quantize: only dtype=torch.int8 is supported")
    if axis not in (-1, -2, input.dim() - 1, input.dim() - 2):
        raise RuntimeError("npu_quantize: axis must address one of the last two dims")
    per_token = axis in (-2, input.dim() - 2)
    if not div_mode:
        return ops.quantize_static(input, scales, zero_points, per_token)
    if input.dim() < 2:
        raise RuntimeError("npu_quantize: the input must have at least two dims")
    K = input.shape[-1]
    x2 = input.reshape(-1, K)
    n = scales.numel()
    zp = None
    if zero_points is not None:
        zf = zero_points.reshape(-1).to(torch.float32)
        zp = zf.round().to(torch.int32)
        if not torch.equal(zp.to(torch.float32), zf):
            raise RuntimeError("npu_quantize: div_mode=True takes integer zero_points")
        if zp.numel() != n:
            raise RuntimeError("npu_quantize: {} zero_points for {} scales".format(zp.numel(), n))
    sc = scales.reshape(-1).to(torch.float32)
    if n == 1:
        group = -1                                   # one scale for the tensor
    elif per_token and n == input.shape[-2]:
        group = 0                                    # one per token, shared by every leading batch index
        reps = x2.shape[0] // n
        if reps > 1:
            sc = sc.repeat(reps)
            zp = None if zp is None else zp.repeat(reps)
    else:
        raise RuntimeError("npu_quantize: div_mode=True takes one scale per tensor or one per token, got {} scales "
                           "for an input of shape {}".format(n, tuple(input.shape)))
    _, codes = ops.quant_with_params(x2, sc, zp, group, -128, 127, want_dq=False, codes_kind=ops.CODES_I8)
    return codes.reshape(input.shape)


def _weight_nk(x2):
    """[K,N] int8 -> [N,K] K-contiguous; free when x2 is the transposed view the reference registers."""
    if x2.dim() != 2:
        raise RuntimeError("quantized weight must be 2-D")
    t = x2.t()
    return t if t.is_contiguous() else t.contiguous()


def npu_quant_matmul(x1, x2, scale, offset=None, bias=None, pertoken_scale=None, output_dtype=torch.bfloat16):
    """x1 int8 [..., M, K] @ x2 int8 [K, N] -> [..., M, N]: int32 accumulate (+ int32 bias),
    * scale[n] (* pertoken_scale[m]) (+ float bias), one rounding to output_dtype."""
    if offset is not None:
        raise RuntimeError("npu_quant_matmul: offset is not supported")
    if x1.dim() < 2 or x1.dim() > 6:
        raise RuntimeError("Linear quant only support dim from 2 to 6")
    lead = x1.shape[:-1]
    x2d = x1.reshape(-1, x1.shape[-1])
    s_tok = pertoken_scale
    if s_tok is not None and s_tok.numel() != x2d.shape[0]:
        # one scale per token of the last-but-one dim, shared by every leading batch index
        if s_tok.numel() == 0 or s_tok.numel() != x1.shape[-2]:
            raise RuntimeError("npu_quant_matmul: {} token scales for inputs of shape {}".format(
                s_tok.numel(), tuple(x1.shape)))
        s_tok = s_tok.reshape(-1).repeat(x2d.shape[0] // s_tok.numel())
    out = ops.gemm_w8a8(x2d, _weight_nk(x2), scale, s_tok, bias, output_dtype)
    return out.reshape(*lead, -1)


def npu_convert_weight_to_int4pack(weight, inner_k_tiles=0):
    """int32 [K, N] holding one signed int4 each -> int32 [K, N/8]."""
    return ops.pack_int4_words(weight)


class _LayoutCache:
    """Converted operands of npu_weight_quant_batchmatmul, keyed on the identity and version of the tensors the
    caller passed.  A deploy module calls the operator with the same registered buffers on every forward; their
    kernel layout ([N, K] weights, [N, K/g] factors) is computed on the first call only.

    Lifetime: an entry holds weak references to its source tensors and is dropped the moment one of them is freed
    (weakref.finalize), so the cache never outlives the model: at most one converted copy per live weight.  There
    is no entry count limit (a model of any number of layers hits on every forward after the first); `max_bytes`
    (None: unbounded) caps the converted bytes kept, evicting the least recently used entry first.
    Contract: a write that bumps the tensor's version counter (copy_, add_, ...) is seen and converts again; a
    write that does not (through `.data`, `set_()` onto the same storage, a kernel outside torch) is NOT seen --
    call clear_layout_cache() after such a write."""

    def __init__(self, max_bytes=None):
        import collections
        self.max_bytes = max_bytes
        self.entries = collections.OrderedDict()      # key -> (weakrefs, value, nbytes), least recently used first
        self.bytes = 0
        self.conversions = 0

    @staticmethod
    def _key(tensors, extra):
        return tuple((id(t), t.data_ptr(), t._version, tuple(t.shape), t.dtype) if t is not None else None
                     for t in tensors) + (extra,)

    def _drop(self, key):
        hit = self.entries.pop(key, None)
        if hit is not None:
            self.bytes -= hit[2]

    def get(self, tensors, extra, make):
        import weakref
        key = self._key(tensors, extra)
        hit = self.entries.get(key)
        if hit is not None and all((r is None and t is None) or (r is not None and r() is t)
                                   for r, t in zip(hit[0], tensors)):
            self.entries.move_to_end(key)
            return hit[1]
        self._drop(key)
        # an older version of the same source tensors is of no further use
        ids = tuple(None if t is None else id(t) for t in tensors)
        for k in [k for k in self.entries if tuple(None if e is None else e[0] for e in k[:-1]) == ids and k[-1] == extra]:
            self._drop(k)
        value = make()
        self.conversions += 1
        nbytes = sum(v.numel() * v.element_size() for v in value if isinstance(v, torch.Tensor))
        refs = []
        for t in tensors:
            if t is None:
                refs.append(None)
                continue
            refs.append(weakref.ref(t))
            weakref.finalize(t, self._drop, key)        # the source is gone: so is the converted copy
        self.entries[key] = (refs, value, nbytes)
        self.bytes += nbytes
        while self.max_bytes is not None and self.bytes > self.max_bytes and len(self.entries) > 1:
            self._drop(next(iter(self.entries)))
        return value

    def clear(self):
        self.entries.clear()
        self.bytes = 0


_layout_cache = _LayoutCache()


def clear_layout_cache():
    """Forgets every converted operand (needed after a write to a weight or factor tensor that torch's version
    counter does not see)."""
    _layout_cache.clear()


def set_layout_cache_limit(max_bytes):
    """Caps the converted bytes the operator keeps (None: no cap; entries always die with their source tensors)."""
    _layout_cache.max_bytes = max_bytes


def npu_weight_quant_batchmatmul(x, weight, antiquant_scale, antiquant_offset=None, quant_scale=None,
                                 quant_offset=None, bias=None, antiquant_group_size=0, inner_precise=0):
    """x [..., K] @ ((weight + antiquant_offset) * antiquant_scale) + bias.  weight: int8 [K, N], or int4 packed
    [K, N/8] int32; factors [K/g, N] (or broadcastable to [1, N] when antiquant_group_size == 0), in x's dtype.
    The kernels stream [N, K] weights and [N, K/g] factors: the conversion of the operands a caller passes is done
    once per (tensor, version) and cached."""
    if quant_scale is not None or quant_offset is not None:
        raise RuntimeError("npu_weight_quant_batchmatmul: output quantisation is not supported")
    if weight.dtype not in (torch.int32, torch.int8) or weight.dim() != 2:
        raise RuntimeError("npu_weight_quant_batchmatmul: the weight must be int8 [K, N] or packed int4 (int32 [K, N/8])")
    K = x.shape[-1]
    if weight.shape[0] != K:
        raise RuntimeError("npu_weight_quant_batchmatmul: weight must be [K, N] / [K, N/8]")
    int4 = weight.dtype == torch.int32
    N = weight.shape[1] * (8 if int4 else 1)
    group = antiquant_group_size if antiquant_group_size else K
    if K % group:
        raise RuntimeError("npu_weight_quant_batchmatmul: K is not a multiple of antiquant_group_size")

    def convert():
        if int4:
            wq = ops.words_to_nibbles_nk(weight, K, N)
        else:
            wq = weight.t().contiguous()
        return (wq,) + factors_to_native(antiquant_scale, antiquant_offset, N, K // group, int4)

    wq, scales, zeros = _layout_cache.get((weight, antiquant_scale, antiquant_offset), (group, x.dtype), convert)
    lead = x.shape[:-1]
    x2 = x.reshape(-1, K)
    out = ops.gemm_w4a16(x2, wq, scales, zeros, group, None, bias) if int4 else \
        ops.gemm_w8a16(x2, wq, scales, zeros, group, None, bias)
    return out.reshape(*lead, N)


def factors_to_native(antiquant_scale, antiquant_offset, N, G, int4=True):
    """Reference factor layout ([G, N], offset stored negated in the float dtype) -> kernel layout: scales [N, G]
    f16|bf16; int4: zeros uint8 [N, G] = 8 - antiquant_offset; int8: offsets int8 [N, G] = -antiquant_offset
    (None when there is no antiquant_offset)."""
    sc = antiquant_scale.reshape(-1, N) if antiquant_scale.dim() > 1 else antiquant_scale.reshape(1, -1)
    if sc.shape[0] not in (1, G):
        raise RuntimeError("antiquant_scale has {} groups, expected {}".format(sc.shape[0], G))
    sc = sc.expand(G, N).t().contiguous()
    if sc.dtype not in (torch.float16, torch.bfloat16):
        sc = sc.to(torch.bfloat16)
    lo, hi, base = (0, 15, 8) if int4 else (-128, 127, 0)
    if antiquant_offset is None:
        zeros = torch.full((N, G), 8, dtype=torch.uint8, device=sc.device) if int4 else None
    else:
        off = antiquant_offset.reshape(-1, N) if antiquant_offset.dim() > 1 else antiquant_offset.reshape(1, -1)
        if off.shape[0] not in (1, G):
            raise RuntimeError("antiquant_offset has {} groups, expected {}".format(off.shape[0], G))
        z = base - off.expand(G, N).t().to(torch.int32)
        if int(z.min()) < lo or int(z.max()) > hi:
            raise RuntimeError("antiquant_offset outside the {} range".format("int4" if int4 else "int8"))
        zeros = z.to(torch.uint8 if int4 else torch.int8).contiguous()
    return sc, zeros


# ---------------------------------------------------------------------------
# The same four operators in the dispatcher, as torch.ops.amct_hip.*, for callers that go through
# torch.ops (scripted or exported graphs).  Device implementations only: a CPU tensor finds no kernel.
# ---------------------------------------------------------------------------
_torch_lib = torch.library.Library("amct_hip", "DEF")
_torch_lib.define("quantize(Tensor input, Tensor scales, Tensor? zero_points=None, int axis=-1, "
                  "bool div_mode=False) -> Tensor")
_torch_lib.define("quant_matmul(Tensor x1, Tensor x2, Tensor scale, Tensor? pertoken_scale=None, "
                  "Tensor? bias=None, ScalarType? output_dtype=None) -> Tensor")
_torch_lib.define("weight_quant_batchmatmul(Tensor x, Tensor weight, Tensor antiquant_scale, "
                  "Tensor? antiquant_offset=None, Tensor? bias=None, int antiquant_group_size=0) -> Tensor")
_torch_lib.define("convert_weight_to_int4pack(Tensor weight) -> Tensor")


def _op_quantize(input, scales, zero_points=None, axis=-1, div_mode=False):
    return npu_quantize(input, scales, zero_points, torch.int8, axis, div_mode)


def _op_quant_matmul(x1, x2, scale, pertoken_scale=None, bias=None, output_dtype=None):
    return npu_quant_matmul(x1, x2, scale, bias=bias, pertoken_scale=pertoken_scale,
                            output_dtype=output_dtype if output_dtype is not None else torch.bfloat16)


def _op_weight_quant_batchmatmul(x, weight, antiquant_scale, antiquant_offset=None, bias=None,
                                 antiquant_group_size=0):
    return npu_weight_quant_batchmatmul(x, weight, antiquant_scale, antiquant_offset, bias=bias,
                                        antiquant_group_size=antiquant_group_size)


_torch_lib.impl("quantize", _op_quantize, "CUDA")
_torch_lib.impl("quant_matmul", _op_quant_matmul, "CUDA")
_torch_lib.impl("weight_quant_batchmatmul", _op_weight_quant_batchmatmul, "CUDA")
_torch_lib.impl("convert_weight_to_int4pack", npu_convert_weight_to_int4pack, "CUDA")
