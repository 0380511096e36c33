"""Operator-level drop-in for the four device operators the reference's deploy modules call
(torch_npu.npu_quantize, npu_quant_matmul, npu_weight_quant_batchmatmul,
npu_convert_weight_to_int4pack -- call sites amct_pytorch/deploy_op/npu_quantization_linear.py:98-102
and amct_pytorch/deploy_op/weight_npu_quant_module.py:54-57,116-117).  Same keyword names and operand
layouts as those calls; each runs HIP kernels only.

The weight operands arrive here in the reference's [K, N] layouts and are re-laid out for the kernels
on every call; the deploy modules in amct_amd.deploy_op do that once at construction instead.
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
    """int8 = saturate(round_half_even(input * scales + zero_points)) (div_mode=False) or
    input / scales (div_mode=True is not used by the reference's deploy path)."""
    if dtype != torch.int8:
        raise RuntimeError("npu_quantize: only dtype=torch.int8 is supported")
    if div_mode:
        raise RuntimeError("npu_quantize: div_mode=True is not supported")
    if axis not in (-1, -2, input.dim() - 1, input.dim() - 2):
        raise RuntimeError("npu_quantize: axis must address one of the last two dims")
    per_token = axis in (-2, input.dim() - 2)
    return ops.quantize_static(input, scales, zero_points, per_token)


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
        reps = x2d.shape[0] // s_tok.numel()
        s_tok = s_tok.reshape(-1).repeat(reps)
    out = ops.gemm_w8a8(x2d, _weight_nk(x2), scale, s_tok, bias, output_dtype)
    return out.reshape(*lead, -1)


def npu_convert_weight_to_int4pack(weight, inner_k_tiles=0):
    """int32 [K, N] holding one signed int4 each -> int32 [K, N/8]."""
    return ops.pack_int4_words(weight)


def npu_weight_quant_batchmatmul(x, weight, antiquant_scale, antiquant_offset=None, quant_scale=None,
                                 quant_offset=None, bias=None, antiquant_group_size=0, inner_precise=0):
    """x [M, K] @ ((weight + antiquant_offset) * antiquant_scale) + bias with weight int4 packed
    [K, N/8] int32, factors [K/g, N] (or [1|N-broadcast, N] when antiquant_group_size == 0)."""
    if quant_scale is not None or quant_offset is not None:
        raise RuntimeError("npu_weight_quant_batchmatmul: output quantisation is not supported")
    if weight.dtype != torch.int32:
        raise RuntimeError("npu_weight_quant_batchmatmul: only packed int4 weights (int32 words) are supported")
    K = x.shape[-1]
    if weight.shape[0] != K:
        raise RuntimeError("npu_weight_quant_batchmatmul: weight must be [K, N/8]")
    N = weight.shape[1] * 8
    group = antiquant_group_size if antiquant_group_size else K
    packed = ops.words_to_nibbles_nk(weight, K, N)
    scales, zeros = factors_to_native(antiquant_scale, antiquant_offset, N, K // group)
    lead = x.shape[:-1]
    out = ops.gemm_w4a16(x.reshape(-1, K), packed, scales, zeros, group, None, bias)
    return out.reshape(*lead, N)


def factors_to_native(antiquant_scale, antiquant_offset, N, G):
    """Reference factor layout ([G, N], offset stored negated in the float dtype) -> kernel layout
    (scales [N, G] f16|bf16, zeros uint8 [N, G] = 8 - antiquant_offset)."""
    sc = antiquant_scale.reshape(-1, N) if antiquant_scale.dim() > 1 else antiquant_scale.reshape(1, -1)
    if sc.shape[0] not in (1, G):
        raise RuntimeError("antiquant_scale has {} groups, expected {}".format(sc.shape[0], G))
    sc = sc.expand(G, N).t().contiguous()
    if sc.dtype not in (torch.float16, torch.bfloat16):
        sc = sc.to(torch.bfloat16)
    if antiquant_offset is None:
        zeros = torch.full((N, G), 8, dtype=torch.uint8, device=sc.device)
    else:
        off = antiquant_offset.reshape(-1, N) if antiquant_offset.dim() > 1 else antiquant_offset.reshape(1, -1)
        z = 8 - off.expand(G, N).t().to(torch.int32)
        if int(z.min()) < 0 or int(z.max()) > 15:
            raise RuntimeError("antiquant_offset outside the int4 range")
        zeros = z.to(torch.uint8).contiguous()
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
