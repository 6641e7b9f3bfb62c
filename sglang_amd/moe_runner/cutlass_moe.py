"""Expert-major block-FP8 fused MoE with the argument list of the reference's grouped-GEMM backend
(python/sglang/srt/layers/moe/cutlass_moe.py:29-341): rows are physically permuted into one contiguous
span per expert (prepare_moe_input + shuffle_rows), both GEMMs run as one grouped launch each over those
spans, and apply_shuffle_mul_sum un-permutes, weights and sums the top-k rows.

Only the block-scaled FP8 configuration is implemented: the expert-specialised and MXFP8 variants of the
reference are Hopper/Blackwell launch variants of the same math and raise NotImplementedError here."""
from typing import Optional, Tuple

import torch

from ..moe import apply_shuffle_mul_sum, fp8_blockwise_scaled_grouped_mm, prepare_moe_input, shuffle_rows, silu_and_mul
from ..quantization.fp8_kernel import sglang_per_token_group_quant_fp8


def cutlass_fused_experts_fp8(
    a: torch.Tensor,
    w1_q: torch.Tensor,
    w2_q: torch.Tensor,
    w1_scale: torch.Tensor,
    w2_scale: torch.Tensor,
    topk_weights: torch.Tensor,
    topk_ids: torch.Tensor,
    a1_strides: torch.Tensor,
    c1_strides: torch.Tensor,
    a2_strides: torch.Tensor,
    c2_strides: torch.Tensor,
    workspace: torch.Tensor,
    a_ptrs: torch.Tensor,
    b_ptrs: torch.Tensor,
    out_ptrs: torch.Tensor,
    a_scales_ptrs: torch.Tensor,
    b_scales_ptrs: torch.Tensor,
    expert_offsets: torch.Tensor,
    problem_sizes1: torch.Tensor,
    problem_sizes2: torch.Tensor,
    use_fp8_blockscale: bool = True,
    use_mxfp8: bool = False,
    output: Optional[torch.Tensor] = None,
    enable_es: Tuple[bool, bool] = (False, False),
) -> torch.Tensor:
    """a [m, k] half/bfloat16; w1_q [E, k, 2n] and w2_q [E, n, k] e4m3fn as column-major views of the
    [E, 2n, k] / [E, k, n] checkpoints; w1_scale [E, k/128, 2n/128] and w2_scale [E, n/128, k/128] as the
    matching views; topk_weights / topk_ids [m, topk] (ids int32).  Returns [m, k] in a's dtype.
    Sequence of cutlass_moe.py:185-341: quantise a per 1x128 group, gather rows and their scales into
    expert-major order, grouped GEMM 1, SiLU*mul, quantise, grouped GEMM 2, weighted top-k sum."""
    assert use_fp8_blockscale, "Only support fp8 blockscale for now"
    if use_mxfp8 or any(enable_es):
        raise NotImplementedError("the MXFP8 and expert-specialised launch variants are not implemented")
    assert topk_weights.shape == topk_ids.shape, "topk shape mismatch"
    assert w1_q.dtype == torch.float8_e4m3fn
    assert w2_q.dtype == torch.float8_e4m3fn
    assert a.shape[1] == w1_q.shape[1], "Hidden size mismatch w1"
    assert w1_q.shape[2] == w2_q.shape[1] * 2, "Hidden size mismatch w2"
    assert w1_q.shape[0] == w2_q.shape[0], "Expert number mismatch"
    assert w1_q.shape[0] == w1_scale.shape[0], "w1 scales expert number mismatch"
    assert w1_q.shape[0] == w2_scale.shape[0], "w2 scales expert number mismatch"
    assert a.dtype in [torch.half, torch.bfloat16], "Invalid output dtype"

    out_dtype = a.dtype
    num_experts = w1_q.size(0)
    m = a.size(0)
    k = w1_q.size(1)
    n = w2_q.size(1)
    topk = topk_ids.size(1)
    device = a.device

    a_map = torch.empty((topk_ids.numel()), dtype=torch.int32, device=device)
    c_map = torch.empty((topk_ids.numel()), dtype=torch.int32, device=device)
    prepare_moe_input(topk_ids, expert_offsets, problem_sizes1, problem_sizes2, a_map, c_map, num_experts, n, k)

    a_q, a1_scale = sglang_per_token_group_quant_fp8(a, 128)
    rep_a_q = shuffle_rows(a_q, a_map, (m * topk, k))
    rep_a1_scales = shuffle_rows(a1_scale, a_map, (m * topk, k // 128))

    c1 = torch.empty((m * topk, n * 2), device=device, dtype=out_dtype)
    c2 = torch.empty((m * topk, k), device=device, dtype=out_dtype)
    a_sf_layout = torch.empty((num_experts, 5), device=device, dtype=torch.int)
    w_sf_layout = torch.empty((num_experts, 5), device=device, dtype=torch.int)

    fp8_blockwise_scaled_grouped_mm(c1, a_ptrs, b_ptrs, out_ptrs, a_scales_ptrs, b_scales_ptrs, rep_a_q, w1_q,
                                    rep_a1_scales, w1_scale, a1_strides, a1_strides, c1_strides, a_sf_layout,
                                    w_sf_layout, problem_sizes1, expert_offsets[:-1], workspace)

    intermediate = torch.empty((m * topk, n), device=device, dtype=out_dtype)
    silu_and_mul(c1, intermediate)
    intermediate_q, a2_scale = sglang_per_token_group_quant_fp8(intermediate, 128)

    fp8_blockwise_scaled_grouped_mm(c2, a_ptrs, b_ptrs, out_ptrs, a_scales_ptrs, b_scales_ptrs, intermediate_q, w2_q,
                                    a2_scale, w2_scale, a2_strides, a2_strides, c2_strides, a_sf_layout, w_sf_layout,
                                    problem_sizes2, expert_offsets[:-1], workspace)

    if output is None:
        output = torch.empty((m, k), device=device, dtype=out_dtype)
    apply_shuffle_mul_sum(c2, output, c_map, topk_weights.to(out_dtype))
    return output
