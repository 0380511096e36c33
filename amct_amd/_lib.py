"""ctypes binding of libamct_hip.so (the C ABI declared in include/amct_hip.h).

There is no fallback: if the library is missing, loading raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# AMCT_HIP_LIB names another build of the same library (for comparing two builds on one machine)
LIB_PATH = os.environ.get("AMCT_HIP_LIB") or os.path.join(_HERE, "lib", "libamct_hip.so")

F32, F16, BF16 = 0, 1, 2
SCOPE_AMCT, SCOPE_ABSMAX = 0, 1
COL_NONE, COL_MUL, COL_DIV, COL_MUL_THEN_DIV = 0, 1, 2, 3
STAGE_FULL, STAGE_SCALE, STAGE_DEQUANT, STAGE_COL = 0, 1, 2, 3
CODES_NONE, CODES_I8, CODES_I32 = 0, 1, 2
MX_E4M3, MX_E2M1 = 0, 1
MX_FLOOR, MX_RCEIL = 0, 1
COL_MINMAX_NOALLOC_MAX_COLS = 8192

_P = ctypes.c_void_p
_I = ctypes.c_int
_L = ctypes.c_int64

# name -> (restype, argtypes); must list every function include/amct_hip.h declares
SIGNATURES = {
    "amct_hip_version": (_I, []),
    "amct_hip_strerror": (ctypes.c_char_p, [_I]),
    "amct_copy_bytes": (_I, [_P, _P, _L, _P]),
    "amct_mfma_yardstick": (_I, [_I, _I, _I, _P, _P, _P]),
    "amct_minmax": (_I, [_P, _P, _P, _L, _L, _I, _I, _P]),
    "amct_gptq_block": (_I, [_P, _L, _P, _L, _P, _L, _P, _P, _L, _P, _L, _I, _I, _I, _P]),
    "amct_hessian_update_workspace_bytes": (ctypes.c_size_t, [_L, _L]),
    "amct_hessian_update": (_I, [_P, _P, _L, _L, ctypes.c_float, ctypes.c_float, _I, _P, ctypes.c_size_t, _P]),
    "amct_fp8_block_dequant": (_I, [_P, _P, _P, _L, _L, _I, _I, _P]),
    "amct_pack_int4_pairs_n": (_I, [_P, _P, _L, _L, _P]),
    "amct_scale_f32_to_u64": (_I, [_P, _P, _L, _P]),
    "amct_col_minmax_workspace_bytes": (ctypes.c_size_t, [_L, _L]),
    "amct_col_minmax": (_I, [_P, _P, _P, _L, _L, _I, _I, _I, _P, ctypes.c_size_t, _P]),
    "amct_col_minmax_noalloc": (_I, [_P, _P, _P, _L, _L, _I, _I, _I, _P]),
    "amct_awq_loss_workspace_bytes": (ctypes.c_size_t, []),
    "amct_awq_loss": (_I, [_P, _P, _L, _I, _P, _P, ctypes.c_size_t, _P]),
    "amct_scale_offset": (_I, [_P, _P, _P, _P, _P, _L, _I, _I, _I, _I, _P]),
    "amct_quant_with_params": (_I, [_P, _P, _P, _P, _P, _I, _P, _I, _L, _L, _I, _I, _I, _I, _I, _I, _P]),
    "amct_fakequant_int": (_I, [_P, _P, _P, _I, _P, _P, _P, _P, _I, _L, _L, _I, _I, _I, _I, _I, _I, _I, _I, _P]),
    "amct_quant_int4_group_pack": (_I, [_P, _P, _P, _I, _P, _P, _P, _P, _I, _L, _L, _I, _I, _I, _P]),
    "amct_pack_int4_words": (_I, [_P, _P, _L, _L, _P]),
    "amct_words_to_nibbles_nk": (_I, [_P, _P, _L, _L, _P]),
    "amct_pack_nibbles_nk": (_I, [_P, _P, _L, _L, _P]),
    "amct_nibbles_nk_to_codes_kn": (_I, [_P, _P, _L, _L, _P]),
    "amct_act_quant_per_token_int8": (_I, [_P, _P, _P, _P, _L, _L, _I, _I, _P]),
    "amct_quantize": (_I, [_P, _P, _P, _P, _P, _L, _L, _L, _I, _I, _P]),
    "amct_mx_quant": (_I, [_P, _P, _P, _L, _L, _I, _I, _I, _P]),
    "amct_mx_dequant": (_I, [_P, _P, _P, _L, _L, _I, _I, _P]),
    "amct_hif8_encode": (_I, [_P, _P, _L, _I, _I, _P]),
    "amct_hif8_decode": (_I, [_P, _P, _L, _I, _P]),
    "amct_gemm_w8a8": (_I, [_P, _P, _P, _P, _P, _I, _P, _P, _L, _L, _L, _I, _P]),
    "amct_gemm_w8a8_workspace_bytes": (ctypes.c_size_t, [_L, _L, _L]),
    "amct_gemm_w8a8_ws": (_I, [_P, _P, _P, _P, _P, _I, _P, _P, _L, _L, _L, _I, _P, ctypes.c_size_t, _P]),
    "amct_linear_w8a8_workspace_bytes": (ctypes.c_size_t, [_L, _L, _L]),
    "amct_linear_w8a8": (_I, [_P, _I, _P, _P, _P, _L, _I, _P, _P, _P, _P, _I, _P, _L, _L, _L, _I, _P, ctypes.c_size_t, _P]),
    "amct_gemm_w8a16": (_I, [_P, _P, _P, _P, _I, _P, _P, _P, _L, _L, _L, _I, _I, _P]),
    "amct_gemm_w8a16_workspace_bytes": (ctypes.c_size_t, [_L, _L, _L, _I, _I]),
    "amct_gemm_w8a16_ws": (_I, [_P, _P, _P, _P, _I, _P, _P, _P, _L, _L, _L, _I, _I, _P, ctypes.c_size_t, _P]),
    "amct_gemm_w4a16_workspace_bytes": (ctypes.c_size_t, [_L, _L, _L, _I, _I]),
    "amct_gemm_w4a16_weight_rounded": (_I, [_L, _L, _L, _I, _I, ctypes.c_size_t]),
    "amct_gemm_w8a16_weight_rounded": (_I, [_L, _L, _L, _I, _I, ctypes.c_size_t]),
    "amct_gemm_w4a16": (_I, [_P, _P, _P, _P, _I, _P, _P, _P, _L, _L, _L, _I, _I, _P, ctypes.c_size_t, _P]),
}

_lib = None


def load():
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "amct_amd: {} is missing -- build it with `python -m amct_amd.build` "
            "(there is no CPU fallback)".format(LIB_PATH))
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc):
    if rc != 0:
        raise RuntimeError("amct_hip: " + load().amct_hip_strerror(rc).decode())
