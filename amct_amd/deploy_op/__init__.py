from .hip_quantization_linear import HipQuantizationLinear  # noqa: F401
from .weight_hip_quant_module import HipWeightQuantizedLinear  # noqa: F401
