"""Activation-quantisation callers and the block-FP8 matmul entry, with the reference's
names, arguments and scale-buffer layouts
(python/sglang/srt/layers/quantization/fp8_kernel.py:454-678,1135-1300)."""
from typing import List, Optional, Tuple

import torch

from ..gemm import (
    sgl_per_token_group_quant_8bit,
    sgl_per_token_quant_fp8,
)

fp8_dtype = torch.float8_e4m3fn
fp8_max = 448.0
fp8_min = -448.0


def ceil_align(x: int, y: int) -> int:
    return (x + y - 1) // y * y


def create_per_token_group_quant_fp8_output_scale(
    x_shape, device, group_size, column_major_scales: bool, scale_tma_aligned: bool, scale_ue8m0: bool
):
    """The four scale layouts (fp8_kernel.py:454-495): UE8M0 packed int32 (column-major,
    rows padded to 4), column-major fp32 with/without row padding, row-major fp32."""
    if scale_ue8m0:
        assert column_major_scales and scale_tma_aligned
        *x_batch, x_q_mn, x_q_k = x_shape
        x_s_mn, x_s_k = x_q_mn, x_q_k // 128
        aligned_mn = ceil_align(x_s_mn, 4)
        aligned_k = ceil_align(x_s_k, 4)
        return torch.empty((*x_batch, aligned_k // 4, aligned_mn), device=device, dtype=torch.int).transpose(-1, -2)[
            ..., :x_s_mn, :
        ]
    elif column_major_scales:
        if scale_tma_aligned:
            aligned_size = (x_shape[-2] + 3) // 4 * 4
            return torch.empty(
                tuple(x_shape[:-2]) + (x_shape[-1] // group_size, aligned_size), device=device, dtype=torch.float32
            ).transpose(-1, -2)[: x_shape[-2], :]
        else:
            return torch.empty(
                (x_shape[-1] // group_size,) + tuple(x_shape[:-1]), device=device, dtype=torch.float32
            ).permute(-1, -2)
    else:
        return torch.empty(tuple(x_shape[:-1]) + (x_shape[-1] // group_size,), device=device, dtype=torch.float32)


def sglang_per_token_group_quant_fp8(
    x: torch.Tensor,
    group_size: int,
    eps: float = 1e-10,
    column_major_scales: bool = False,
    scale_tma_aligned: bool = False,
    scale_ue8m0: bool = False,
    fuse_silu_and_mul: bool = False,
    masked_m: Optional[torch.Tensor] = None,
    enable_v2: Optional[bool] = None,
):
    """fp8_kernel.py:498-565."""
    assert x.shape[-1] % group_size == 0, "the last dimension of `x` cannot be divisible by `group_size`"
    assert x.is_contiguous(), "`x` is not contiguous"
    out_shape = (*x.shape[:-1], x.shape[-1] // (2 if fuse_silu_and_mul else 1))
    x_q = torch.empty(out_shape, device=x.device, dtype=fp8_dtype)
    x_s = create_per_token_group_quant_fp8_output_scale(
        x_shape=out_shape,
        device=x.device,
        group_size=group_size,
        column_major_scales=column_major_scales,
        scale_tma_aligned=scale_tma_aligned,
        scale_ue8m0=scale_ue8m0,
    )
    if enable_v2 is None:
        enable_v2 = group_size in (16, 32, 64, 128)
    if x.shape[0] > 0:
        sgl_per_token_group_quant_8bit(
            x, x_q, x_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0, fuse_silu_and_mul, masked_m,
            enable_v2=enable_v2,
        )
    return x_q, x_s


def sglang_per_token_group_quant_fp8_ue8m0(x: torch.Tensor, group_size: int, eps: float = 1e-10):
    """fp8_kernel.py:568-610."""
    assert x.shape[-1] % group_size == 0, f"hidden ({x.shape[-1]}) must be divisible by group_size ({group_size})"
    assert x.is_contiguous(), "x must be contiguous"
    *x_batch, x_q_mn, x_q_k = x.shape
    x_q = torch.empty(x.shape, device=x.device, dtype=fp8_dtype)
    aligned_mn = ceil_align(x_q_mn, 4)
    aligned_k = ceil_align(x_q_k // group_size, 4)
    x_s = torch.empty((*x_batch, aligned_k // 4, aligned_mn), device=x.device, dtype=torch.int).transpose(-1, -2)[
        ..., :x_q_mn, :
    ]
    if x.shape[0] > 0:
        sgl_per_token_group_quant_8bit(
            x, x_q, x_s, group_size, eps, fp8_min, fp8_max, True, False, None, enable_v2=True
        )
    return x_q, x_s


def sglang_per_token_group_quant_int8(x: torch.Tensor, group_size: int, eps: float = 1e-10,
                                      dtype: torch.dtype = torch.int8, enable_v2: Optional[bool] = None):
    """int8 sibling (python/sglang/srt/layers/quantization/int8_kernel.py:184-225): row-major fp32 scales."""
    assert x.shape[-1] % group_size == 0
    assert x.is_contiguous()
    x_q = torch.empty_like(x, dtype=dtype)
    x_s = torch.empty(x.shape[:-1] + (x.shape[-1] // group_size,), device=x.device, dtype=torch.float32)
    if x.numel() > 0:
        sgl_per_token_group_quant_8bit(x, x_q, x_s, group_size, eps, -128.0, 127.0, False, enable_v2=enable_v2)
    return x_q, x_s


def sglang_per_token_group_quant_8bit(
    x: torch.Tensor,
    group_size: int,
    dst_dtype: torch.dtype,
    eps: float = 1e-10,
    column_major_scales: bool = False,
    scale_tma_aligned: bool = False,
    scale_ue8m0: bool = False,
    fuse_silu_and_mul: bool = False,
    masked_m: Optional[torch.Tensor] = None,
    enable_v2: Optional[bool] = None,
):
    """fp8_kernel.py:614-653."""
    if dst_dtype == torch.int8:
        assert not column_major_scales
        assert not scale_tma_aligned
        assert not fuse_silu_and_mul
        assert masked_m is None
        return sglang_per_token_group_quant_int8(x=x, group_size=group_size, eps=eps, dtype=dst_dtype,
                                                 enable_v2=enable_v2)
    return sglang_per_token_group_quant_fp8(
        x=x, group_size=group_size, eps=eps, column_major_scales=column_major_scales,
        scale_tma_aligned=scale_tma_aligned, scale_ue8m0=scale_ue8m0, fuse_silu_and_mul=fuse_silu_and_mul,
        masked_m=masked_m, enable_v2=enable_v2,
    )


def sglang_per_token_quant_fp8(x: torch.Tensor, dtype: torch.dtype = fp8_dtype):
    """fp8_kernel.py:656-672."""
    assert x.is_contiguous(), "`x` is not contiguous"
    x_q = torch.empty_like(x, device=x.device, dtype=dtype)
    x_s = torch.empty(x.shape[0], 1, device=x.device, dtype=torch.float32)
    sgl_per_token_quant_fp8(x, x_q, x_s)
    return x_q, x_s


# on this backend the operator is always the sgl_kernel one (fp8_kernel.py:675-678)
per_token_group_quant_fp8 = sglang_per_token_group_quant_fp8


def _cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def prepare_block_fp8_matmul_inputs(A, B, As, Bs, block_size: List[int], output_dtype: torch.dtype = torch.float16):
    """Shape checks and output allocation of fp8_kernel.py:1135-1180 (fp32 scales only)."""
    assert len(block_size) == 2
    block_n, block_k = block_size[0], block_size[1]
    assert A.shape[-1] == B.shape[-1]
    assert A.shape[:-1] == As.shape[:-1]
    assert A.is_contiguous()
    if As.dtype == torch.float:
        assert _cdiv(A.shape[-1], block_k) == As.shape[-1]
    else:
        raise NotImplementedError("packed UE8M0 activation scales are not accepted by this matmul yet")
    M = A.numel() // A.shape[-1]
    assert B.ndim == 2
    assert B.is_contiguous()
    assert Bs.ndim == 2
    N, K = B.shape
    if Bs.dtype == torch.float:
        assert _cdiv(N, block_n) == Bs.shape[0]
        assert _cdiv(K, block_k) == Bs.shape[1]
    else:
        raise NotImplementedError("packed UE8M0 weight scales are not accepted by this matmul yet")
    C = A.new_empty(A.shape[:-1] + (N,), dtype=output_dtype)
    return M, N, K, C


def w8a8_block_fp8_matmul(A, B, As, Bs, block_size: List[int], output_dtype: torch.dtype = torch.float16):
    """Block-wise W8A8 matmul with row-major scales (fp8_kernel.py:1201-1300): A [..., K] e4m3fn,
    B [N, K] e4m3fn, As [..., ceil(K/128)], Bs [ceil(N/128), ceil(K/128)] -> [..., N]."""
    from ..ops import w8a8_block_fp8_matmul_

    M, N, K, C = prepare_block_fp8_matmul_inputs(A, B, As, Bs, block_size, output_dtype)
    if list(block_size) != [128, 128]:
        raise NotImplementedError("only block_size [128, 128] is implemented")
    assert output_dtype in (torch.float16, torch.bfloat16)
    if not As.is_contiguous():
        As = As.contiguous()
    w8a8_block_fp8_matmul_(A.view(M, K), B, As.view(M, -1), Bs, C.view(M, N))
    return C


w8a8_block_fp8_matmul_triton = w8a8_block_fp8_matmul  # same contract; there is no Triton here
