"""Python shims for the MoE-side operators (sgl-kernel/python/sgl_kernel/moe.py:6-25,
sgl-kernel/python/sgl_kernel/elementwise.py silu_and_mul)."""
from typing import Optional

import torch

from . import ops  # noqa: F401


def moe_align_block_size(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids, num_tokens_post_pad,
                         cumsum_buffer, pad_sorted_token_ids=False):
    torch.ops.sgl_kernel.moe_align_block_size.default(
        topk_ids, num_experts, block_size, sorted_token_ids, experts_ids, num_tokens_post_pad, cumsum_buffer,
        pad_sorted_token_ids,
    )


def moe_sum_reduce(input_tensor, output_tensor, routed_scaling_factor=0):
    torch.ops.sgl_kernel.moe_sum_reduce.default(input_tensor, output_tensor, routed_scaling_factor)


def silu_and_mul(input: torch.Tensor, out: torch.Tensor = None) -> torch.Tensor:
    if input.shape[-1] * input.dtype.itemsize % 16 != 0:
        raise ValueError("The pointers must be multiple of 16 bytes.")
    if out is not None:
        assert input.shape[:-1] == out.shape[:-1] and input.shape[-1] == 2 * out.shape[-1]
    else:
        out = torch.empty(input.shape[:-1] + (input.shape[-1] // 2,), device=input.device, dtype=input.dtype)
    torch.ops.sgl_kernel.silu_and_mul.default(out, input)
    return out


def topk_softmax(topk_weights: torch.Tensor, topk_ids: torch.Tensor, gating_output: torch.Tensor,
                 renormalize: bool = False, moe_softcapping: float = 0.0,
                 correction_bias: Optional[torch.Tensor] = None) -> None:
    """sgl-kernel/python/sgl_kernel/moe.py:28-54."""
    torch.ops.sgl_kernel.topk_softmax.default(topk_weights, topk_ids, gating_output, renormalize, moe_softcapping,
                                              correction_bias)
