"""Weight-only deploy Linear (W4A16 / W8A16): the MI355X counterpart of NpuWeightQuantizedLinear
(amct_pytorch/deploy_op/weight_npu_quant_module.py:29-121).  Same constructor argument and buffer
names (scale_factor, quantized_weight, scale_w, offset_w, bias); int4 and int8 weights, bf16 and fp16 models
(amct_pytorch/utils/vars.py:43-47).  The buffers are kept in the layout the GEMM kernels stream:
  int4: quantized_weight uint8 [N, K/2] (code + 8, even k in the low nibble), offset_w uint8 [N, K/g] (offset + 8)
  int8: quantized_weight int8 [N, K], offset_w int8 [N, K/g] (the quantiser's offset) or None
  scale_w [N, K/g] in the weight's dtype
and `reference_layout()` converts them to the reference's [K, N] (int8) / [K, N/8] (int4 words) / [K/g, N] form."""
import torch
from torch import nn

from .. import ops
from ..utils.quant_util import check_scale_offset_shape

_SUPPORTED = (torch.bfloat16, torch.float16)


class HipWeightQuantizedLinear(nn.Module):
    def __init__(self, quant_module):
        super().__init__()
        wts_type = quant_module.wts_type
        if wts_type not in ('int4', 'int8'):
            raise ValueError('Not supported quant_dtype {}'.format(wts_type))
        self.wts_type = wts_type
        bits = 4 if wts_type == 'int4' else 8
        qmin, qmax = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
        device = quant_module.weight.device
        weight = quant_module.weight.data
        if weight.dtype not in _SUPPORTED:
            raise RuntimeError('Not support tensor dtype {}, support dtypes {}.'.format(weight.dtype, list(_SUPPORTED)))
        self.group_size = quant_module.group_size
        N, K = weight.shape
        awq = None
        if hasattr(quant_module, 'scale') and quant_module.scale is not None:
            awq = quant_module.scale.to(device=device)
            if list(awq.shape) != [1, K]:
                raise RuntimeError("AWQ params scale.shape should be [1, {}] current shape is {}".format(
                    K, list(awq.shape)))
            self.register_buffer('scale_factor', awq)
        else:
            self.scale_factor = None
        scale_w = quant_module.scale_w.to(device)
        offset_w = quant_module.offset_w.to(device) if quant_module.offset_w is not None else None
        check_scale_offset_shape(weight, scale_w, offset_w, self.group_size)
        if self.group_size is not None:
            if K % self.group_size:
                raise RuntimeError("weight-only deploy needs cin to be a multiple of group_size")
            group, g = self.group_size, self.group_size
            sw = scale_w.reshape(N, -1)
            ow = offset_w.reshape(N, -1) if offset_w is not None else None
        else:
            # per channel / per tensor: one group spanning K (weight_npu_quant_module.py:91-98)
            group = 0 if scale_w.numel() > 1 else -1
            g = K
            sw = scale_w.reshape(-1, 1)
            sw = sw.repeat(N, 1) if sw.shape[0] == 1 else sw
            ow = None
            if offset_w is not None:
                ow = offset_w.reshape(-1, 1)
                ow = ow.repeat(N, 1) if ow.shape[0] == 1 else ow
            self.group_size = 0
        self._gemm_group = g
        self._symmetric = offset_w is None
        if ow is not None and (int(ow.min()) < qmin or int(ow.max()) > qmax):
            raise RuntimeError("offset_w outside the {} range".format(wts_type))
        # codes with the given factors (quant_weight, amct_pytorch/utils/quant_util.py:76-93)
        _, codes = ops.quant_with_params(weight, scale_w.reshape(-1), None if offset_w is None else offset_w.reshape(-1),
                                         group, qmin, qmax, want_dq=False, codes_kind=ops.CODES_I8, col_scale=awq,
                                         col_mode=ops.COL_DIV if awq is not None else ops.COL_NONE)
        self.register_buffer('scale_w', sw.to(weight.dtype).contiguous())
        if wts_type == 'int4':
            self.register_buffer('quantized_weight', ops.pack_nibbles_nk(codes))
            zeros = (ow.to(torch.int32) + 8).to(torch.uint8) if ow is not None else \
                torch.full(sw.shape, 8, dtype=torch.uint8, device=device)
            self.register_buffer('offset_w', zeros.contiguous())
        else:
            self.register_buffer('quantized_weight', codes)
            if ow is not None:
                self.register_buffer('offset_w', ow.to(torch.int8).contiguous())
            else:
                self.offset_w = None
        if quant_module.bias is not None:
            # the reference keeps an fp16 bias in fp16 and widens a bf16 one (:68-73); fp16 -> fp32 is exact, and the
            # kernels add the bias to the fp32 accumulator either way
            self.register_buffer('bias', quant_module.bias.to(device=device).to(torch.float32))
        else:
            self.bias = None

    def forward(self, inputs):
        ori_shape = inputs.shape
        if inputs.dim() < 2 or inputs.dim() > 6:
            raise RuntimeError("Linear quant only support dim from 2 to 6")
        inputs = inputs.to(self.quantized_weight.device).reshape(-1, ori_shape[-1])
        if self.wts_type == 'int4':
            out = ops.gemm_w4a16(inputs, self.quantized_weight, self.scale_w, self.offset_w, self._gemm_group,
                                 self.scale_factor, self.bias)
        else:
            out = ops.gemm_w8a16(inputs, self.quantized_weight, self.scale_w, self.offset_w, self._gemm_group,
                                 self.scale_factor, self.bias)
        return out.reshape(*ori_shape[:-1], -1)

    def reference_layout(self):
        """(quantized_weight, scale_w [K/g, N], offset_w [K/g, N] = -offset | None) as the reference registers them
        (weight_npu_quant_module.py:52-66): int8 [K, N] codes, or int32 [K, N/8] words for int4."""
        sw = self.scale_w.t().contiguous()
        if self.wts_type == 'int4':
            codes = ops.unpack_nibbles_to_i32_kn(self.quantized_weight)
            qw = ops.pack_int4_words(codes)
            ow = None if self._symmetric else \
                (8 - self.offset_w.to(torch.int32)).to(self.scale_w.dtype).t().contiguous()
        else:
            qw = self.quantized_weight.t().contiguous()
            ow = None if self.offset_w is None else \
                (self.offset_w.to(torch.int32) * -1).to(self.scale_w.dtype).t().contiguous()
        return qw, sw, ow
