"""Linear-layer wrappers over the quantise + GEMM pair, with the reference's signatures
(python/sglang/srt/layers/quantization/fp8_utils.py:350-365,612-642,758-811,814-834,1458-1560)."""
from typing import Callable, List, Optional

import torch

from ..gemm import fp8_blockwise_scaled_mm, fp8_scaled_mm
from .fp8_kernel import (
    per_token_group_quant_fp8,
    sglang_per_token_quant_fp8,
    w8a8_block_fp8_matmul,
)


def _rows(input: torch.Tensor) -> torch.Tensor:
    """Collapse the leading dimensions of an activation into one row dimension."""
    return input.reshape(-1, input.shape[-1]) if input.dim() != 2 else input


def _finish(out_2d: torch.Tensor, input: torch.Tensor, bias, dtype: torch.dtype) -> torch.Tensor:
    """Add the bias in place and restore the activation's leading dimensions."""
    if bias is not None:
        out_2d += bias
    return out_2d.to(dtype).view(*input.shape[:-1], out_2d.shape[-1])


def triton_w8a8_block_fp8_linear(input, weight, block_size: List[int], weight_scale, input_scale=None, bias=None):
    """Row-major-scale variant (fp8_utils.py:814-834); accepts N, K that are not multiples of 128."""
    assert input_scale is None
    x = _rows(input)
    x_q, x_scale = per_token_group_quant_fp8(x, block_size[1], column_major_scales=False)
    out = w8a8_block_fp8_matmul(x_q, weight, x_scale, weight_scale, block_size, output_dtype=x.dtype)
    return _finish(out, input, bias, x.dtype)


def cutlass_w8a8_block_fp8_linear_with_fallback(input, weight, block_size: List[int], weight_scale,
                                                input_scale=None, bias=None):
    """Column-major-scale variant feeding fp8_blockwise_scaled_mm (fp8_utils.py:612-642); weights whose
    N or K is not a multiple of 128 go to the row-major variant."""
    assert input_scale is None
    n, k = weight.shape
    if n % 128 or k % 128:
        return triton_w8a8_block_fp8_linear(input, weight, block_size, weight_scale, input_scale, bias)
    x = _rows(input)
    x_q, x_scale = per_token_group_quant_fp8(x, block_size[1], column_major_scales=True)
    out = fp8_blockwise_scaled_mm(x_q, weight.T, x_scale, weight_scale.T, out_dtype=x.dtype)
    return _finish(out, input, bias, x.dtype)


def aiter_w8a8_block_fp8_linear(input, weight, block_size: List[int], weight_scale, input_scale=None, bias=None):
    """The ROCm variant's contract (fp8_utils.py:758-811): with `input_scale` the input is already quantised
    (e4m3fn with row-major 1x128 scales, as fused_rms_fp8_group_quant returns it) and the result is bfloat16;
    without it the input is quantised here like in the other variants."""
    if input_scale is None:
        return cutlass_w8a8_block_fp8_linear_with_fallback(input, weight, block_size, weight_scale, None, bias)
    assert input.dtype == torch.float8_e4m3fn, "a pre-quantised input must be float8_e4m3fn"
    x_q = _rows(input)
    out = w8a8_block_fp8_matmul(x_q, weight, input_scale.view(x_q.shape[0], -1), weight_scale, block_size,
                                output_dtype=torch.bfloat16)
    return _finish(out, input, bias, torch.bfloat16)


def dispatch_w8a8_block_fp8_linear() -> Callable:
    """fp8_utils.py:350-365: on this backend there is one implementation."""
    return cutlass_w8a8_block_fp8_linear_with_fallback


def apply_fp8_linear(input, weight, weight_scale, input_scale=None, input_scale_ub=None, bias=None,
                     cutlass_fp8_supported: bool = True, use_per_token_if_dynamic: bool = True,
                     pad_output=None, compressed_tensor_quant: bool = False):
    """Per-token dynamic activation quant + per-channel weight scale GEMM (fp8_utils.py:1458-1560,
    dynamic per-token branch :1527-1559).  `weight` is the [K, N] column-major view of the
    [N, K] parameter (w8a8_fp8.py:120,137); `weight_scale` has N elements."""
    assert input_scale is None, "static activation scales are not implemented"
    x = _rows(input)
    x_q, x_scale = sglang_per_token_quant_fp8(x)
    out = fp8_scaled_mm(x_q, weight, x_scale, weight_scale.reshape(-1).contiguous(), out_dtype=input.dtype, bias=bias)
    return out.view(*input.shape[:-1], weight.shape[1])
