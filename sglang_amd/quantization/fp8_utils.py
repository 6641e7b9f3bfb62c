"""Linear-layer wrappers over the quantise + GEMM pair, with the reference's signatures
(python/sglang/srt/layers/quantization/fp8_utils.py:350-365,612-642,645-696,758-811,814-834,1458-1560)."""
from typing import Callable, List, Optional

import torch

from ..gemm import fp8_blockwise_scaled_mm, fp8_scaled_mm
from .fp8_kernel import (
    per_token_group_quant_fp8,
    sglang_per_token_group_quant_fp8,
    sglang_per_token_quant_fp8,
    static_quant_fp8,
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


def _dynamic_block_quant_only(input_scale, block_size) -> None:
    """Configurations of the block linears that are valid in the reference and not built here are refused
    before any work, with the exception a caller's fall-through catches."""
    if input_scale is not None:
        raise NotImplementedError("a static activation scale is not implemented for the block-FP8 linear")
    if not all(b in (64, 128) for b in block_size):
        raise NotImplementedError("scale blocks of 64 or 128 in each direction are implemented")


def triton_w8a8_block_fp8_linear(input, weight, block_size: List[int], weight_scale, input_scale=None, bias=None):
    """Row-major-scale variant (fp8_utils.py:814-834); accepts N, K that are not multiples of 128."""
    _dynamic_block_quant_only(input_scale, block_size)
    x = _rows(input)
    x_q, x_scale = per_token_group_quant_fp8(x, block_size[1], column_major_scales=False)
    out = w8a8_block_fp8_matmul(x_q, weight, x_scale, weight_scale, block_size, output_dtype=x.dtype)
    return _finish(out, input, bias, x.dtype)


def cutlass_w8a8_block_fp8_linear_with_fallback(input, weight, block_size: List[int], weight_scale,
                                                input_scale=None, bias=None):
    """Column-major-scale variant feeding fp8_blockwise_scaled_mm (fp8_utils.py:612-642); weights whose
    N or K is not a multiple of 128 go to the row-major variant."""
    _dynamic_block_quant_only(input_scale, block_size)
    if weight_scale.dtype == torch.int32:
        return deepgemm_w8a8_block_fp8_linear_with_fallback(input, weight, block_size, weight_scale, None, bias)
    n, k = weight.shape
    if n % 128 or k % 128 or list(block_size) != [128, 128]:
        return triton_w8a8_block_fp8_linear(input, weight, block_size, weight_scale, input_scale, bias)
    x = _rows(input)
    x_q, x_scale = per_token_group_quant_fp8(x, block_size[1], column_major_scales=True)
    out = fp8_blockwise_scaled_mm(x_q, weight.T, x_scale, weight_scale.T, out_dtype=x.dtype)
    return _finish(out, input, bias, x.dtype)


def deepgemm_w8a8_block_fp8_linear_with_fallback(input, weight, block_size: List[int], weight_scale,
                                                 input_scale=None, bias=None):
    """The UE8M0 variant (fp8_utils.py:645-696): weight scales are packed power-of-two exponents (int32 words, one
    row of words per weight row), the activations are quantised to the same format (column-major, rows aligned to
    4), and the GEMM applies both inside its MFMAs.  Float weight scales take the ordinary variant, as the
    reference falls back to its Triton kernel."""
    _dynamic_block_quant_only(input_scale, block_size)
    if weight_scale.dtype != torch.int32:
        return cutlass_w8a8_block_fp8_linear_with_fallback(input, weight, block_size, weight_scale, None, bias)
    x = _rows(input)
    x_q, x_scale = sglang_per_token_group_quant_fp8(x, block_size[1], column_major_scales=True,
                                                    scale_tma_aligned=True, scale_ue8m0=True)
    out = w8a8_block_fp8_matmul(x_q, weight, x_scale, weight_scale, block_size, output_dtype=x.dtype)
    return _finish(out, input, bias, x.dtype)


def aiter_w8a8_block_fp8_linear(input, weight, block_size: List[int], weight_scale, input_scale=None, bias=None):
    """The ROCm variant's contract (fp8_utils.py:758-811): with `input_scale` the input is already quantised
    (e4m3fn with row-major 1x128 scales, as fused_rms_fp8_group_quant returns it) and the result is bfloat16;
    without it the input is quantised here like in the other variants."""
    if input_scale is None:
        return cutlass_w8a8_block_fp8_linear_with_fallback(input, weight, block_size, weight_scale, None, bias)
    if input.dtype != torch.float8_e4m3fn or list(block_size) != [128, 128]:
        raise NotImplementedError("an input scale is only accepted with a pre-quantised float8_e4m3fn input "
                                  "and block_size [128, 128]")
    x_q = _rows(input)
    if input_scale.numel() != x_q.shape[0] * (-(-x_q.shape[1] // 128)):
        raise NotImplementedError("the input scale must hold one value per row and 128 columns")
    out = w8a8_block_fp8_matmul(x_q, weight, input_scale.view(x_q.shape[0], -1), weight_scale, block_size,
                                output_dtype=torch.bfloat16)
    return _finish(out, input, bias, torch.bfloat16)


def dispatch_w8a8_block_fp8_linear() -> Callable:
    """fp8_utils.py:350-365: on this backend there is one implementation."""
    return cutlass_w8a8_block_fp8_linear_with_fallback


def apply_fp8_linear(input, weight, weight_scale, input_scale=None, input_scale_ub=None, bias=None,
                     cutlass_fp8_supported: bool = True, use_per_token_if_dynamic: bool = False,
                     pad_output=None, compressed_tensor_quant: bool = False):
    """Activation quant + row-scaled GEMM (fp8_utils.py:1458-1560): per-token dynamic scales (:1527-1559), a
    dynamic per-tensor scale (use_per_token_if_dynamic=False), or a static per-tensor `input_scale` broadcast to
    the rows (:1518-1524, static_quant_fp8).  `weight` is the [K, N]
    column-major view of the [N, K] parameter (w8a8_fp8.py:120,137); `weight_scale` has N elements, or one that
    is then used for every column."""
    # `input_scale_ub` is accepted and unused, as in the reference's function body; `pad_output` pads the rows of
    # the quantised input for torch._scaled_mm there and narrows the result again, so the output is the same with or
    # without it and nothing is padded here.
    if input_scale is not None and input_scale.numel() != 1:
        raise NotImplementedError("a static input_scale must be per tensor")
    n_out = weight.shape[1]
    if weight_scale.numel() not in (1, n_out):
        raise NotImplementedError("weight scales must be per channel (one per output column) or per tensor")
    if input.dtype not in (torch.float16, torch.bfloat16):
        raise NotImplementedError("the output dtype must be float16 or bfloat16")
    x = _rows(input)
    # Which activation scale (fp8_utils.py:1488-1547): a static one when given; with compressed_tensor_quant the
    # flag decides between per token and per tensor; otherwise dynamic scales are per token (the reference's CUDA
    # branch, :1527-1529) except for per-tensor weights without the flag (its ROCm branch, :1534-1540).
    per_tensor_dynamic = input_scale is None and not use_per_token_if_dynamic and \
        (compressed_tensor_quant or weight_scale.numel() == 1)
    if input_scale is not None:
        x_q, x_scale = static_quant_fp8(x, input_scale, repeat_scale=True)
    elif per_tensor_dynamic:
        # max|x| / 448 computed on the device, then broadcast to the rows like a static scale
        from ..ops import tensor_absmax_scale_

        scale = torch.empty(1, device=x.device, dtype=torch.float32)
        tensor_absmax_scale_(x if x.is_contiguous() else x.contiguous(), scale)
        x_q, x_scale = static_quant_fp8(x, scale, repeat_scale=True)
    else:
        x_q, x_scale = sglang_per_token_quant_fp8(x)
    w_scale = weight_scale.reshape(-1).to(torch.float32)
    if w_scale.numel() == 1:
        w_scale = w_scale.expand(n_out)
    out = fp8_scaled_mm(x_q, weight, x_scale, w_scale.contiguous(), out_dtype=input.dtype, bias=bias)
    return out.view(*input.shape[:-1], weight.shape[1])
