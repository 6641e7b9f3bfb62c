"""Python shims for the MoE-side operators (sgl-kernel/python/sgl_kernel/moe.py:6-25,175-251,
sgl-kernel/python/sgl_kernel/gemm.py:213-220, sgl-kernel/python/sgl_kernel/elementwise.py silu_and_mul)."""
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


def _act_and_mul(op, input: torch.Tensor, out: torch.Tensor = None) -> torch.Tensor:
    if input.shape[-1] * input.dtype.itemsize % 16 != 0:
        raise ValueError("The pointers must be multiple of 16 bytes.")
    if out is not None:
        assert input.shape[:-1] == out.shape[:-1] and input.shape[-1] == 2 * out.shape[-1]
    else:
        out = torch.empty(input.shape[:-1] + (input.shape[-1] // 2,), device=input.device, dtype=input.dtype)
    op(out, input)
    return out


def silu_and_mul(input: torch.Tensor, out: torch.Tensor = None) -> torch.Tensor:
    """sgl-kernel/python/sgl_kernel/elementwise.py:258-270."""
    return _act_and_mul(torch.ops.sgl_kernel.silu_and_mul.default, input, out)


def gelu_tanh_and_mul(input: torch.Tensor, out: torch.Tensor = None) -> torch.Tensor:
    """sgl-kernel/python/sgl_kernel/elementwise.py:273-285."""
    return _act_and_mul(torch.ops.sgl_kernel.gelu_tanh_and_mul.default, input, out)


def gelu_and_mul(input: torch.Tensor, out: torch.Tensor = None) -> torch.Tensor:
    """sgl-kernel/python/sgl_kernel/elementwise.py:288-300."""
    return _act_and_mul(torch.ops.sgl_kernel.gelu_and_mul.default, input, out)


def topk_softmax(topk_weights: torch.Tensor, topk_ids: torch.Tensor, gating_output: torch.Tensor,
                 renormalize: bool = False, moe_softcapping: float = 0.0,
                 correction_bias: Optional[torch.Tensor] = None) -> None:
    """sgl-kernel/python/sgl_kernel/moe.py:28-54."""
    torch.ops.sgl_kernel.topk_softmax.default(topk_weights, topk_ids, gating_output, renormalize, moe_softcapping,
                                              correction_bias)


def topk_sigmoid(topk_weights: torch.Tensor, topk_ids: torch.Tensor, gating_output: torch.Tensor,
                 renormalize: bool = False, correction_bias: Optional[torch.Tensor] = None) -> None:
    """sgl-kernel/python/sgl_kernel/moe.py:57-80."""
    torch.ops.sgl_kernel.topk_sigmoid.default(topk_weights, topk_ids, gating_output, renormalize, correction_bias)


def prepare_moe_input(topk_ids, expert_offsets, problem_sizes1, problem_sizes2, input_permutation, output_permutation,
                      num_experts, n, k, blockscale_offsets: Optional[torch.Tensor] = None):
    """sgl-kernel/python/sgl_kernel/moe.py:217-240."""
    torch.ops.sgl_kernel.prepare_moe_input.default(
        topk_ids, expert_offsets, blockscale_offsets, problem_sizes1, problem_sizes2, input_permutation,
        output_permutation, num_experts, n, k,
    )


def shuffle_rows(input_tensor, dst2src_map, output_tensor_shape):
    """sgl-kernel/python/sgl_kernel/gemm.py:213-220."""
    output_tensor = torch.empty(output_tensor_shape, device=input_tensor.device, dtype=input_tensor.dtype)
    torch.ops.sgl_kernel.shuffle_rows.default(input_tensor, dst2src_map, output_tensor)
    return output_tensor


def apply_shuffle_mul_sum(input, output, permutation, factors):
    """sgl-kernel/python/sgl_kernel/moe.py:243-251."""
    torch.ops.sgl_kernel.apply_shuffle_mul_sum.default(input, output, permutation, factors)


def fp8_blockwise_scaled_grouped_mm(output, a_ptrs, b_ptrs, out_ptrs, a_scales_ptrs, b_scales_ptrs, a, b, scales_a,
                                    scales_b, stride_a, stride_b, stride_c, layout_sfa, layout_sfb, problem_sizes,
                                    expert_offsets, workspace):
    """sgl-kernel/python/sgl_kernel/moe.py:175-214."""
    torch.ops.sgl_kernel.fp8_blockwise_scaled_grouped_mm.default(
        output, a_ptrs, b_ptrs, out_ptrs, a_scales_ptrs, b_scales_ptrs, a, b, scales_a, scales_b, stride_a, stride_b,
        stride_c, layout_sfa, layout_sfb, problem_sizes, expert_offsets, workspace,
    )


def es_fp8_blockwise_scaled_grouped_mm(output, a, b, scales_a, scales_b, stride_a, stride_b, stride_d, problem_sizes,
                                       expert_offsets, workspace):
    """sgl-kernel/python/sgl_kernel/expert_specialization.py:4-29."""
    torch.ops.sgl_kernel.es_fp8_blockwise_scaled_grouped_mm.default(
        output, a, b, scales_a, scales_b, stride_a, stride_b, stride_d, problem_sizes, expert_offsets, workspace,
    )
