"""INT8 activation quantisation callers and the block-scaled INT8 matmul
(python/sglang/srt/layers/quantization/int8_kernel.py:59-89, :134-226, :355-425)."""
from typing import List

import torch

from ..ops import per_token_quant_int8_, w8a8_block_int8_matmul_
from .fp8_kernel import sglang_per_token_group_quant_int8


def per_token_quant_int8(x: torch.Tensor, scale_dtype=torch.float32, cal_sum: bool = False):
    """Returns (x_q int8 like x, scales [..., 1]); cal_sum additionally returns the row sums."""
    assert x.is_contiguous()
    assert scale_dtype == torch.float32, "only fp32 scales are produced"
    x_q = torch.empty_like(x, dtype=torch.int8)
    scales = torch.empty(x.shape[:-1] + (1,), device=x.device, dtype=torch.float32)
    per_token_quant_int8_(x, x_q, scales)
    if cal_sum:
        return x_q, scales, x.to(torch.float32).sum(dim=-1).to(x.dtype)
    return x_q, scales


def per_token_group_quant_int8(x: torch.Tensor, group_size: int, eps: float = 1e-10, dtype: torch.dtype = torch.int8):
    """Per-token-group INT8 quantisation (int8_kernel.py:134-190): x [..., hidden] contiguous ->
    (x_q int8 like x, x_s fp32 [..., hidden // group_size]); scale = max(absmax, eps) / 127."""
    assert x.shape[-1] % group_size == 0, "the last dimension of `x` cannot be divisible by `group_size`"
    assert x.is_contiguous(), "`x` is not contiguous"
    x_q, x_s = sglang_per_token_group_quant_int8(x.view(-1, x.shape[-1]), group_size, eps=eps, dtype=dtype)
    return x_q.view(x.shape), x_s.view(x.shape[:-1] + (x.shape[-1] // group_size,))


def w8a8_block_int8_matmul(A, B, As, Bs, block_size: List[int], output_dtype: torch.dtype = torch.float16):
    """Block-wise W8A8 INT8 matmul (int8_kernel.py:355-425): A [..., K] int8, B [N, K] int8,
    As [..., ceil(K/block_k)], Bs [ceil(N/block_n), ceil(K/block_k)] fp32 -> [..., N].  Each block_k-deep partial
    dot product is exact in int32 and is folded into an fp32 accumulator with As * Bs.  block_size [128, 128] runs
    the specialised kernels, 64 in either direction the generic one."""
    assert len(block_size) == 2
    block_n, block_k = block_size[0], block_size[1]
    if not all(b in (64, 128) for b in block_size):
        raise NotImplementedError("scale blocks of 64 or 128 in each direction are implemented")
    assert A.shape[-1] == B.shape[-1]
    assert A.shape[:-1] == As.shape[:-1] and A.is_contiguous()
    assert -(-A.shape[-1] // block_k) == As.shape[-1]
    M = A.numel() // A.shape[-1]
    assert B.ndim == 2 and B.is_contiguous() and Bs.ndim == 2
    N, K = B.shape
    assert -(-N // block_n) == Bs.shape[0]
    assert -(-K // block_k) == Bs.shape[1]
    assert A.dtype == torch.int8 and B.dtype == torch.int8
    assert As.dtype == torch.float32 and Bs.dtype == torch.float32
    assert output_dtype in (torch.float16, torch.bfloat16)
    C = A.new_empty(A.shape[:-1] + (N,), dtype=output_dtype)
    if not As.is_contiguous():
        As = As.contiguous()
    if list(block_size) != [128, 128]:
        from ..ops import block_scaled_mm_any_

        block_scaled_mm_any_(A.view(M, K), B, As.view(M, -1), Bs, C.view(M, N), block_n, block_k)
        return C
    w8a8_block_int8_matmul_(A.view(M, K), B, As.view(M, -1), Bs, C.view(M, N))
    return C
