"""Python shims over ``torch.ops.sgl_kernel`` with the reference's names, argument order
and defaults (sgl-kernel/python/sgl_kernel/gemm.py:13-42,99-147)."""
from typing import Optional

import torch

from . import ops  # noqa: F401

_K = torch.ops.sgl_kernel
_V2_GROUP_SIZES = (16, 32, 64, 128)


def int8_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias=None):
    """[M, K] int8 x column-major [K, N] int8, one scale per row of A and per column of B, optional [N] bias."""
    return _K.int8_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias)


def fp8_blockwise_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype):
    """[M, K] e4m3 x column-major [K, N] e4m3 with 1x128 activation and 128x128 weight scales."""
    return _K.fp8_blockwise_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype)


def fp8_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias=None):
    """The e4m3 sibling of int8_scaled_mm."""
    return _K.fp8_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias)


def sgl_per_token_group_quant_8bit(
    input: torch.Tensor,
    output_q: torch.Tensor,
    output_s: torch.Tensor,
    group_size: int,
    eps: float,
    fp8_min: float,
    fp8_max: float,
    scale_ue8m0: bool = False,
    fuse_silu_and_mul: bool = False,
    masked_m: Optional[torch.Tensor] = None,
    enable_v2: Optional[bool] = None,
) -> None:
    """Quantise `input` per group of `group_size` into `output_q`, scales into `output_s`.  Two arithmetics
    exist (sgl_kernel/gemm.py:112-147): the second one is the default for the group sizes it supports and
    the only one that takes the SiLU*mul fusion and the masked layout."""
    use_v2 = enable_v2 if enable_v2 is not None else group_size in _V2_GROUP_SIZES
    common = (input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0)
    if use_v2:
        _K.sgl_per_token_group_quant_8bit_v2(*common, fuse_silu_and_mul, masked_m)
        return
    assert not fuse_silu_and_mul, "only v2 support fuse_silu_and_mul"
    assert masked_m is None, "only v2 support masked_m"
    _K.sgl_per_token_group_quant_8bit(*common)


# older names of the same function
sgl_per_token_group_quant_fp8 = sgl_per_token_group_quant_8bit
sgl_per_token_group_quant_int8 = sgl_per_token_group_quant_8bit


def sgl_per_token_quant_fp8(input: torch.Tensor, output_q: torch.Tensor, output_s: torch.Tensor) -> None:
    """One scale per row: output_s[i] = max|input[i, :]| / 448."""
    _K.sgl_per_token_quant_fp8(input, output_q, output_s)
