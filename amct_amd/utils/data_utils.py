"""Host-side mirror of amct_pytorch/utils/data_utils.py for the hot path: same names, arguments
and errors; the arithmetic runs in the HIP kernels."""
import torch

from .. import ops

DATA_MAP = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def check_linear_input_dim(input_tensor):
    """Linear inputs must have 2..6 dims (amct_pytorch/utils/data_utils.py:26-34)."""
    if input_tensor.dim() < 2 or input_tensor.dim() > 6:
        raise RuntimeError("Linear quant only support dim from 2 to 6")


@torch.no_grad()
def convert_precision(ori_tensor, quant_dtype):
    """round-half-even then clamp to the integer range, dtype kept
    (amct_pytorch/utils/data_utils.py:48-66)."""
    if DATA_MAP.get(ori_tensor.dtype) is None:
        raise RuntimeError(
            "dtype {} not support now, only support float32/float16/bfloat16.".format(ori_tensor.dtype))
    bits = int(quant_dtype.replace('int', ''))
    shape = ori_tensor.shape
    flat = ori_tensor.reshape(-1, shape[-1]) if ori_tensor.dim() > 1 else ori_tensor.reshape(1, -1)
    one = torch.ones(1, dtype=torch.float32, device=ori_tensor.device)
    # scale 1, no offset: w/1 is exact, so dq == clamp(rne(w))
    dq, _ = ops.quant_with_params(flat, one, None, -1, -(1 << (bits - 1)), (1 << (bits - 1)) - 1)
    return dq.reshape(shape)
