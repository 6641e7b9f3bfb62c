"""Expert-major block-FP8 fused MoE with the argument list of the reference's grouped-GEMM backend
(python/sglang/srt/layers/moe/cutlass_moe.py:29-341): rows are physically permuted into one contiguous
span per expert (prepare_moe_input + shuffle_rows), both GEMMs run as one grouped launch each over those
spans, and apply_shuffle_mul_sum un-permutes, weights and sums the top-k rows.

The block-scaled FP8 configuration is implemented, including `enable_es` (the reference's "expert specialisation"
operator es_fp8_blockwise_scaled_grouped_mm is a launch variant of the same arithmetic and runs the same kernels
here); the MXFP8 variant (Blackwell kernels with their own quantiser) raises NotImplementedError."""
from typing import Optional, Tuple

import torch

from ..moe import (
    apply_shuffle_mul_sum,
    es_fp8_blockwise_scaled_grouped_mm,
    fp8_blockwise_scaled_grouped_mm,
    prepare_moe_input,
    shuffle_rows,
    silu_and_mul,
)
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
    if use_mxfp8:
        raise NotImplementedError("the MXFP8 variant (SM100 expert-specialisation kernels) is not implemented")
    es_up, es_down = enable_es
    assert topk_weights.shape == topk_ids.shape, "topk shape mismatch"
    assert a.dtype in [torch.half, torch.bfloat16], "Invalid output dtype"
    for w in (w1_q, w2_q):
        assert w.dtype == torch.float8_e4m3fn
    E, k, two_n = w1_q.shape
    n = w2_q.shape[1]
    assert a.shape[1] == k, "Hidden size mismatch w1"
    assert two_n == 2 * n, "Hidden size mismatch w2"
    assert w2_q.shape[0] == E, "Expert number mismatch"
    assert w1_scale.shape[0] == E, "w1 scales expert number mismatch"
    assert w2_scale.shape[0] == E, "w2 scales expert number mismatch"

    m, topk = topk_ids.shape
    rows = m * topk

    # row maps: src_of[r] is the token behind expert-major row r, dst_of[j] the expert-major row of pair j
    src_of = topk_ids.new_empty(rows, dtype=torch.int32)
    dst_of = topk_ids.new_empty(rows, dtype=torch.int32)
    prepare_moe_input(topk_ids, expert_offsets, problem_sizes1, problem_sizes2, src_of, dst_of, E, n, k)
    first_row = expert_offsets[:-1]
    # scale-layout scratch that the operator's argument list asks for; this backend leaves it untouched
    sf_layouts = [a.new_empty((E, 5), dtype=torch.int32) for _ in range(2)]

    def grouped(x, w_q, w_scale, width, ab_strides, c_strides, sizes, es):
        """Quantise x per 1x128 group and multiply every expert's span by that expert's weight; `es` picks the
        operator the reference calls with enable_es (cutlass_moe.py:224-237,290-303): same arithmetic."""
        x_q, x_scale = x if isinstance(x, tuple) else sglang_per_token_group_quant_fp8(x, 128)
        out = a.new_empty((rows, width))
        if es:
            es_fp8_blockwise_scaled_grouped_mm(out, x_q, w_q, x_scale, w_scale, ab_strides, ab_strides, c_strides,
                                               sizes, first_row, workspace)
        else:
            fp8_blockwise_scaled_grouped_mm(out, a_ptrs, b_ptrs, out_ptrs, a_scales_ptrs, b_scales_ptrs, x_q, w_q,
                                            x_scale, w_scale, ab_strides, ab_strides, c_strides, *sf_layouts, sizes,
                                            first_row, workspace)
        return out

    # the tokens are quantised once and their bytes and scales gathered, rather than quantised per copy
    a_q, a_scale = sglang_per_token_group_quant_fp8(a, 128)
    gathered = (shuffle_rows(a_q, src_of, (rows, k)), shuffle_rows(a_scale, src_of, (rows, k // 128)))
    gate_up = grouped(gathered, w1_q, w1_scale, two_n, a1_strides, c1_strides, problem_sizes1, es_up)
    # silu_and_mul (cutlass_moe.py:271-272) and the group quantisation of its result in front of the second grouped
    # GEMM, as the one kernel that writes the same bytes and scales without the 16-bit activation rows in between
    if n % 128 == 0:
        act = sglang_per_token_group_quant_fp8(gate_up, 128, fuse_silu_and_mul=True)
    else:
        act = a.new_empty((rows, n))
        silu_and_mul(gate_up, act)
    down = grouped(act, w2_q, w2_scale, k, a2_strides, c2_strides, problem_sizes2, es_down)

    if output is None:
        output = a.new_empty((m, k))
    apply_shuffle_mul_sum(down, output, dst_of, topk_weights.to(a.dtype))
    return output
