"""W8A8 deploy Linear: the MI355X counterpart of NpuQuantizationLinear
(amct_pytorch/deploy_op/npu_quantization_linear.py:27-130).  Same constructor argument
(the calibrated quant module), same buffer names (act_scale, act_offset, scale_factor,
quantized_weight, deq_scale, pertoken_scale, bias) so state_dict keys match; forward runs the
HIP activation-quantise and int8 MFMA GEMM kernels."""
import torch

from .. import ops


class HipQuantizationLinear(torch.nn.Module):
    def __init__(self, quant_module, dynamic_act=False):
        """dynamic_act=True ignores the calibrated activation scale and quantises every token with
        its own live scale (symmetric, the per-token statistics of
        amct_pytorch/quantize_op/minmax_module.py:96-105 evaluated on the batch)."""
        super().__init__()
        self.output_dtype = quant_module.weight.dtype
        device = quant_module.weight.device
        self.offset_bias = None
        self.dynamic_act = dynamic_act
        self.act_type = quant_module.act_type
        self.act_granularity = 'PER_TENSOR'
        self.quantize_axis = -1
        scale_d = quant_module.scale_d.to(device=device)
        offset_d = quant_module.offset_d if quant_module.offset_d is not None else torch.tensor([0])
        offset_d = offset_d.to(device).repeat(scale_d.shape)
        if scale_d.dim() > 1:
            self.act_granularity = 'PER_TOKEN'
            self.quantize_axis = -2
        self.register_buffer('act_scale', (1 / scale_d).reshape(-1).to(self.output_dtype))
        self.register_buffer('act_offset', offset_d.reshape(-1).to(self.output_dtype))

        wts_type = quant_module.wts_type
        if wts_type != 'int8':
            raise ValueError('Not supported quant_dtype {}'.format(wts_type))
        weight = quant_module.weight.data
        smooth = None
        if quant_module.scale is not None:
            smooth = quant_module.scale.to(device=device, dtype=weight.dtype)
            if list(smooth.shape) != [1, weight.shape[1]]:
                raise RuntimeError("smooth_factor shape should be {} current shape is {}"
                                   .format([1, weight.shape[1]], list(smooth.shape)))
            self.register_buffer('scale_factor', (1 / quant_module.scale).to(device=device))
        scale_w = quant_module.scale_w.reshape(-1).to(device=device)
        codes = self.quant_wts(weight, scale_w, wts_type, smooth)          # [N,K] int8, K contiguous
        self.register_buffer('quantized_weight', torch.transpose(codes, 1, 0))
        if quant_module.offset_d is not None:
            # -(offset_d[1,K] @ Wq[K,N]) with the integer contraction done exactly by the int8 GEMM kernel.  The
            # reference forms the same sum with an fp32 matmul and rounds it (npu_quantization_linear.py:56-59): that
            # is exact while K * |offset_d| * 127 < 2^24 and otherwise carries the rounding of its library's summation
            # order; the exact integer is what that expression approximates, and is what is registered here.
            zrow = quant_module.offset_d.to(device).reshape(1, 1).to(torch.int8).repeat(1, weight.shape[-1])
            one = torch.ones(weight.shape[0], dtype=torch.float32, device=device)
            _, acc = ops.gemm_w8a8(zrow, codes, one, want_acc=True, out_dtype=torch.float32)
            self.offset_bias = (-acc.reshape(-1)).to(torch.int32)

        deq = scale_d * scale_w
        if self.act_granularity == 'PER_TENSOR':
            self.register_buffer('deq_scale', deq)
            self.pertoken_scale = None
        else:
            self.register_buffer('deq_scale', scale_w)
            self.register_buffer('pertoken_scale', quant_module.scale_d.reshape(-1).to(torch.float32).to(device=device))
        self._init_bias(quant_module, scale_d, scale_w)

    @staticmethod
    def quant_wts(weight, scale_w_tensor, wts_type, smooth=None):
        """(weight [* smooth]) / scale -> int8 codes [N,K] (npu_quantization_linear.py:49-53,72-87)."""
        group = 0 if scale_w_tensor.shape[0] > 1 else -1
        _, codes = ops.quant_with_params(weight, scale_w_tensor, None, group, -128, 127, want_dq=False,
                                         codes_kind=ops.CODES_I8, col_scale=smooth,
                                         col_mode=ops.COL_MUL if smooth is not None else ops.COL_NONE)
        return codes

    def forward(self, x):
        if x.dim() < 2 or x.dim() > 6:
            raise RuntimeError("Linear quant only support dim from 2 to 6")
        smooth = self.scale_factor if hasattr(self, 'scale_factor') else None
        lead = x.shape[:-1]
        if self.dynamic_act:
            xq, s_tok = ops.act_quant_per_token_int8(x, smooth)
            s_ch = self.deq_scale if self.act_granularity == 'PER_TOKEN' else self._scale_w()
            out = ops.gemm_w8a8(xq.reshape(-1, x.shape[-1]), self.quantized_weight.t(), s_ch, s_tok,
                                self._float_bias(), self.output_dtype)
            return out.reshape(*lead, -1)
        per_token = self.act_granularity == 'PER_TOKEN'
        x2 = x.reshape(-1, x.shape[-1])
        m = x2.shape[0]
        act_scale, act_offset, s_tok = self.act_scale, self.act_offset, self.pertoken_scale
        if per_token and act_scale.numel() != m:
            # one scale per token of the last-but-one dim, shared by every leading batch index
            if act_scale.numel() != x.shape[-2]:
                raise RuntimeError("per-token quantize needs one scale per token ({} vs {})".format(
                    act_scale.numel(), x.shape[-2]))
            act_scale, act_offset = act_scale.repeat(m // act_scale.numel()), act_offset.repeat(m // act_offset.numel())
        if s_tok is not None and s_tok.numel() != m:
            if s_tok.numel() != x.shape[-2]:
                raise RuntimeError("per-token scales were calibrated for {} tokens, the input has {}".format(
                    s_tok.numel(), x.shape[-2]))
            s_tok = s_tok.repeat(m // s_tok.numel())
        # npu_quantize and npu_quant_matmul (npu_quantization_linear.py:98-102) in one library call
        out = ops.linear_w8a8(x2, act_scale, act_offset, per_token, self.quantized_weight.t(), self.deq_scale, s_tok,
                              self.bias, self.output_dtype, smooth)
        return out.reshape(*lead, -1)

    def _scale_w(self):
        return self._dyn_scale_w

    def _float_bias(self):
        return self._dyn_bias

    def _init_bias(self, module, scale_d, scale_w):
        """npu_quantization_linear.py:105-130."""
        # operands of the dynamic_act path: buffers (so that .to(device) moves them) that stay out of state_dict
        self.register_buffer('_dyn_scale_w', scale_w, persistent=False)
        self.register_buffer('_dyn_bias', module.bias.data.float() if module.bias is not None else None,
                             persistent=False)
        if module.bias is not None:
            bias = module.bias
            if self.act_granularity == 'PER_TENSOR':
                b = ops.bias_to_int32(bias.data, scale_d * scale_w)
                self.register_buffer('bias', b)
            else:
                self.register_buffer('bias', bias)
            if self.offset_bias is not None:
                self.bias = self.bias + self.offset_bias
        else:
            self.bias = None if self.offset_bias is None else self.offset_bias
