"""ctypes binding of libsglamd.so, the C-ABI library holding every gfx950 kernel.

There is no fallback: if the library is missing or a symbol is absent, importing this
module raises, and so does every operator built on it.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# SGLAMD_LIBRARY selects another build of the same library (e.g. one compiled with different tuning macros)
LIB_PATH = os.environ.get("SGLAMD_LIBRARY") or os.path.join(_HERE, "libsglamd.so")

# element type tags (include/sglamd.h)
F32, F16, BF16, FP8_E4M3, I8, I32, I64 = range(7)
SCALE_ROW_MAJOR, SCALE_COL_MAJOR, SCALE_COL_MAJOR_UE8M0 = range(3)
FORM_DIVIDE, FORM_RECIPROCAL = 0, 1

_p, _i, _i64, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float

# name -> argtypes; the declarations of include/sglamd.h, in order
SIGNATURES = {
    "sglamd_per_token_group_quant_8bit": [_p, _i, _p, _i, _p, _i64, _i64, _i, _i, _i64, _f, _f, _f, _i, _p],
    "sglamd_per_token_quant_fp8": [_p, _i, _p, _p, _i64, _i64, _p],
    "sglamd_per_token_quant_int8": [_p, _i, _p, _p, _i64, _i64, _p],
    "sglamd_static_quant_fp8": [_p, _i, _p, _p, _p, _i64, _i64, _p],
    "sglamd_tensor_absmax_scale": [_p, _i, _i64, _f, _f, _p, _p, _p],
    "sglamd_fp8_blockwise_scaled_mm": [_p, _i64, _p, _i64, _p, _i64, _i64, _p, _i64, _i64, _p, _i64, _i, _i64, _i64,
                                       _i64, _p, _i64, _p],
    "sglamd_fp8_blockwise_scaled_mm_pow2": [_p, _i64, _p, _i64, _p, _i64, _i64, _p, _i64, _i64, _p, _i64, _i, _i64,
                                            _i64, _i64, _p, _i64, _p],
    "sglamd_int8_blockwise_scaled_mm": [_p, _i64, _p, _i64, _p, _i64, _i64, _p, _i64, _i64, _p, _i64, _i, _i64, _i64,
                                       _i64, _p, _i64, _p],
    "sglamd_fp8_scaled_mm": [_p, _i64, _p, _i64, _p, _p, _p, _p, _i64, _i, _i64, _i64, _i64, _p, _i64, _p],
    "sglamd_int8_scaled_mm": [_p, _i64, _p, _i64, _p, _p, _p, _p, _i64, _i, _i64, _i64, _i64, _p, _i64, _p],
    "sglamd_gemm_workspace_bytes": [_i64, _i64, _i64],
    "sglamd_last_gemm_kernel": [],
    "sglamd_last_streaming_shape": [],
    "sglamd_streaming_piece_offset": [_i, _i, _i64, _p],
    "sglamd_ue8m0_unpack": [_p, _i64, _i64, _i64, _p, _i64, _i64, _p],
    "sglamd_ceiling_mfma": [_i, _i, _i, _p, _p],
    "sglamd_ceiling_hbm": [_p, _p, _i64, _p, _p],
    "sglamd_ceiling_hbm_lds": [_p, _i64, _p],
    "sglamd_ceiling_l2_read": [_p, _i64, _i, _i, _p, _p],
    "sglamd_ceiling_gemm_l2_resident": [_p, _p, _p, _p, _p, _i64, _i64, _i64, _p],
    "sglamd_moe_align_block_size": [_p, _i, _i64, _i, _i, _p, _i64, _p, _p, _p, _i, _p],
    "sglamd_fused_moe_block_fp8_gemm": [_p, _i64, _p, _i64, _i64, _p, _i64, _i64, _p, _i64, _i64, _i64, _p, _i64, _i,
                                        _p, _p, _p, _p, _i64, _i, _i, _i, _i64, _i64, _i64, _p],
    "sglamd_fused_moe_block_int8_gemm": [_p, _i64, _p, _i64, _i64, _p, _i64, _i64, _p, _i64, _i64, _i64, _p, _i64, _i,
                                         _p, _p, _p, _p, _i64, _i, _i, _i, _i64, _i64, _i64, _p],
    "sglamd_topk_softmax": [_p, _p, _p, _i, _i64, _i64, _i64, _i, _f, _p, _p],
    "sglamd_topk_sigmoid": [_p, _p, _p, _i, _i64, _i64, _i64, _i, _p, _p],
    "sglamd_block_scaled_mm_any": [_p, _i64, _p, _i64, _p, _i64, _i64, _p, _i64, _i64, _p, _i64, _i, _i, _i64, _i64,
                                   _i64, _i, _i, _p],
    "sglamd_fused_moe_gemm_any": [_p, _i64, _p, _i64, _i64, _p, _i64, _i64, _p, _i64, _i64, _i64, _p, _i64, _p, _i64,
                                  _i, _i, _i, _i, _p, _p, _p, _p, _i64, _i, _i, _i, _i64, _i64, _i64, _p],
    "sglamd_silu_and_mul": [_p, _p, _i, _i64, _i64, _p],
    "sglamd_gelu_and_mul": [_p, _p, _i, _i64, _i64, _p],
    "sglamd_gelu_tanh_and_mul": [_p, _p, _i, _i64, _i64, _p],
    "sglamd_moe_sum_reduce": [_p, _p, _i, _i64, _i, _i64, _f, _p],
    "sglamd_silu_mul_group_quant_8bit": [_p, _i, _p, _i, _p, _i64, _i64, _i, _i, _i64, _f, _f, _f, _i, _p],
    "sglamd_silu_mul_group_quant_8bit_masked": [_p, _i, _p, _i, _p, _i64, _i64, _i64, _i, _i64, _i64, _p, _f, _f, _f,
                                                _p],
    "sglamd_fused_rms_fp8_group_quant": [_p, _i64, _p, _f, _p, _i64, _i64, _p, _p, _p, _p, _p, _i64, _p, _f, _i64, _p,
                                         _i, _i, _i, _p],
    "sglamd_prepare_moe_input": [_p, _i64, _i, _i, _i64, _i64, _p, _p, _p, _p, _p, _p, _p],
    "sglamd_shuffle_rows": [_p, _p, _p, _i64, _i64, _p],
    "sglamd_apply_shuffle_mul_sum": [_p, _p, _p, _p, _i, _i64, _i, _i64, _p],
    "sglamd_grouped_mm_workspace_bytes": [_i64, _i],
    "sglamd_fp8_blockwise_scaled_grouped_mm": [_p, _i, _p, _p, _p, _p, _p, _p, _i, _i64, _i64, _i64, _p, _i64, _p],
    "sglamd_fused_moe_block_fp8_workspace": [_i64, _i64, _i64, _i, _i, _i],
    "sglamd_fused_moe_block_fp8_static_max_bytes": [],
    "sglamd_fused_moe_block_fp8_static": [_p, _i, _i64, _i64, _i64, _i, _i, _p, _p, _p, _p, _p, _p, _i, _p, _f, _i, _p],
    "sglamd_fused_moe_block_fp8": [_p, _i, _i64, _i64, _i64, _i, _i, _p, _p, _p, _p, _p, _p, _i, _p, _f, _i, _p, _i64,
                                   _p],
}


class SglAmdError(RuntimeError):
    pass


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python sglang_amd/csrc/build.py` "
            "(hipcc, gfx950). sglang_amd has no CPU or eager fallback."
        )
    lib = ctypes.CDLL(LIB_PATH)
    lib.sglamd_last_error.restype = ctypes.c_char_p
    lib.sglamd_last_error.argtypes = []
    lib.sglamd_abi_version.restype = _i
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.argtypes = args
        fn.restype = _i64 if ("workspace" in name or name.endswith("_bytes")) else _i
    return lib


lib = _load()


def check(rc: int) -> None:
    """Raises RuntimeError with the library's message for a non-zero status."""
    if rc != 0:
        msg = lib.sglamd_last_error().decode("utf-8", "replace")
        if rc == -2:
            raise NotImplementedError(msg)
        raise SglAmdError(msg)
