"""Constants shared by the quantize / deploy path (values as in the reference's
amct_pytorch/utils/vars.py:19-29)."""
INT8_MAX = 127
INT8_MIN = -128
INT4_MAX = 7
INT4_MIN = -8
INT8 = 'int8'
INT4 = 'int4'
SUPPORT_WEIGHT_QUANT_DTYPE = [INT8, INT4]
SUPPORT_INPUT_QUANT_DTYPE = [INT8]
