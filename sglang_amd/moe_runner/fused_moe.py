"""Block-quantised fused MoE: align -> grouped GEMM 1 -> SiLU*mul -> grouped GEMM 2 (x routing weight)
-> top-k sum, with the reference's entry points and argument names
(python/sglang/srt/layers/moe/moe_runner/triton_utils/fused_moe.py:218-306,339-398,401-785,788-998).
The use_fp8_w8a8 and use_int8_w8a8 configurations (block-scaled with 64 or 128 wide scale blocks, per-channel, FP8
per-tensor with static activation scales; optional biases) with the gated SiLU activation are implemented; every
other flag combination raises NotImplementedError."""
from typing import Any, Dict, List, Optional

import torch

from ..moe import gelu_and_mul, moe_sum_reduce, silu_and_mul
from ..ops import fused_moe_block_fp8_, fused_moe_block_fp8_gemm_, fused_moe_gemm_any_
from ..quantization.fp8_kernel import (
    sglang_per_token_group_quant_fp8,
    sglang_per_token_group_quant_int8,
    scaled_fp8_quant,
    sglang_per_token_quant_fp8,
    static_quant_fp8,
)
from ..quantization.int8_kernel import per_token_quant_int8
from .base import MoeRunnerConfig
from .moe_align_block_size import moe_align_block_size


def get_default_config(M: int, E: int, topk: int) -> Dict[str, Any]:
    """Sorted-block height for the grouped GEMM, by expected rows per expert (the role of
    fused_moe_triton_config.py:183-192; the tile shapes themselves are fixed in the kernel)."""
    rows_per_expert = M * topk / max(E, 1)
    # the library's own choice for block_m == 0: the streaming kernel while an expert's rows fit one MFMA row
    # group, then the smallest tile-kernel block that still holds a whole expert (its weights are read once)
    if rows_per_expert <= 10:
        bm = 16
    elif rows_per_expert <= 56:
        bm = 64
    elif rows_per_expert <= 112:
        bm = 128
    else:
        bm = 192
    return {"BLOCK_SIZE_M": bm}


def _quantise_activations(A, A_scale, use_int8_w8a8: bool, per_channel_quant: bool, block_shape):
    """The activation quantisation step of invoke_fused_moe_kernel (fused_moe_triton_kernels.py:737-783): per
    1 x block_k group for the block configurations; per token when the weights are per channel; otherwise (FP8) per
    tensor, with the static scale when one is given and max|A| / 448 when not."""
    if block_shape is not None:
        quant = sglang_per_token_group_quant_int8 if use_int8_w8a8 else sglang_per_token_group_quant_fp8
        return quant(A, block_shape[1])
    if use_int8_w8a8:
        assert per_channel_quant, \
            "int8 quantization only supports channel-wise quantization except for block-wise quantization"
        return per_token_quant_int8(A)
    if A_scale is not None:
        assert A_scale.numel() == 1, f"Expected scalar scale, got numel={A_scale.numel()}"
        Aq, _ = static_quant_fp8(A, A_scale.reshape(1).to(torch.float32))
        return Aq, A_scale.reshape(1).to(torch.float32)
    if per_channel_quant:
        return sglang_per_token_quant_fp8(A)
    return scaled_fp8_quant(A, None)  # dynamic per-tensor: one scale, max|A| / 448


def _swiglu_silu_clamp_mul(x: torch.Tensor, gemm1_limit: float) -> torch.Tensor:
    """fused_moe.py:315-321.  A torch.compile'd pointwise function there: evaluated in fp32, rounded once."""
    gate, up = x.float().chunk(2, dim=-1)
    gate = torch.nn.functional.silu(gate).clamp(min=None, max=gemm1_limit)
    return (gate * up.clamp(min=-gemm1_limit, max=gemm1_limit)).to(x.dtype)


def swiglu_gpt_oss_sigmoid_alpha(x: torch.Tensor, gemm1_alpha: float, gemm1_limit: float) -> torch.Tensor:
    """fused_moe.py:324-331 (GPT-OSS: gate and up interleaved).  Evaluated in fp32 and rounded once, like the
    compiled function there."""
    gate, up = x[..., ::2].float(), x[..., 1::2].float()
    gate = gate.clamp(min=None, max=gemm1_limit)
    up = up.clamp(min=-gemm1_limit, max=gemm1_limit)
    return (gate * torch.sigmoid(gate * gemm1_alpha) * (up + 1)).to(x.dtype)


def invoke_fused_moe_kernel(A, B, C, B_scale, topk_weights, sorted_token_ids, expert_ids, num_tokens_post_padded,
                            mul_routed_weight: bool, top_k: int, config: Dict[str, Any], block_shape: Optional[List[int]],
                            use_int8_w8a8: bool = False, per_channel_quant: bool = False, A_scale=None, bias=None):
    """Quantises A and runs the grouped GEMM (fused_moe_triton_kernels.py:702-930; fp8 branches :737-763, int8
    branches :764-783).  Block shape [128, 128] without bias runs the specialised kernels, everything else the
    generic one."""
    assert topk_weights is None or topk_weights.stride(1) == 1
    assert sorted_token_ids.stride(0) == 1
    Aq, Aq_scale = _quantise_activations(A, A_scale, use_int8_w8a8, per_channel_quant, block_shape)
    if block_shape is not None and list(block_shape) == [128, 128] and bias is None:
        fused_moe_block_fp8_gemm_(Aq, Aq_scale, B, B_scale, C, topk_weights, sorted_token_ids, expert_ids,
                                  num_tokens_post_padded, mul_routed_weight, top_k, config["BLOCK_SIZE_M"])
        return
    fused_moe_gemm_any_(Aq, Aq_scale, B, B_scale, C, topk_weights, sorted_token_ids, expert_ids,
                        num_tokens_post_padded, mul_routed_weight, top_k, config["BLOCK_SIZE_M"],
                        block_shape=block_shape, bias=bias)


def fused_experts_impl(
    hidden_states: torch.Tensor,
    w1: torch.Tensor,
    w2: torch.Tensor,
    topk_weights: torch.Tensor,
    topk_ids: torch.Tensor,
    b1: Optional[torch.Tensor] = None,
    b2: Optional[torch.Tensor] = None,
    inplace: bool = False,
    activation: str = "silu",
    is_gated: bool = True,
    apply_router_weight_on_input: bool = False,
    use_fp8_w8a8: bool = False,
    use_int8_w8a8: bool = False,
    use_int8_w8a16: bool = False,
    use_int4_w4a16: bool = False,
    per_channel_quant: bool = False,
    w1_scale: Optional[torch.Tensor] = None,
    w2_scale: Optional[torch.Tensor] = None,
    w1_zp: Optional[torch.Tensor] = None,
    w2_zp: Optional[torch.Tensor] = None,
    a1_scale: Optional[torch.Tensor] = None,
    a2_scale: Optional[torch.Tensor] = None,
    block_shape: Optional[List[int]] = None,
    no_combine: bool = False,
    routed_scaling_factor: Optional[float] = None,
    gemm1_alpha: Optional[float] = None,
    gemm1_limit: Optional[float] = None,
    filter_expert: bool = True,
    swiglu_limit: Optional[float] = None,
    config: Optional[Dict[str, Any]] = None,
):
    """fused_moe.py:788-893 + the kernel sequence :401-785.  Implemented: use_fp8_w8a8 / use_int8_w8a8 with
    block_shape [bn, bk] (64 or 128 each), with per_channel_quant (per-token activation and per-channel weight
    scales), and FP8 with per-tensor activation scales (static a1_scale / a2_scale, or dynamic) and per-expert
    weight scales; biases b1 / b2;
    apply_router_weight_on_input; the activations of fused_moe.py:530-647 (gated SiLU and GELU, plain SiLU, GELU and
    squared ReLU, the clamped SwiGLU forms).  Everything else raises NotImplementedError before any work."""
    if use_fp8_w8a8 == use_int8_w8a8:
        raise NotImplementedError("only the use_fp8_w8a8 and use_int8_w8a8 configurations are implemented")
    if use_int8_w8a16 or use_int4_w4a16:
        raise NotImplementedError("weight-only MoE variants are not implemented")
    if (activation, is_gated) not in (("silu", True), ("gelu", True), ("silu", False), ("gelu", False),
                                      ("relu2", False)):
        raise ValueError(f"Unsupported activation: {activation=}, with {is_gated=}")
    if block_shape is not None:
        if len(block_shape) != 2 or not all(b in (64, 128) for b in block_shape):
            raise NotImplementedError("scale blocks of 64 or 128 in each direction are implemented")
    elif use_int8_w8a8:
        assert per_channel_quant, \
            "int8 quantization only supports channel-wise quantization except for block-wise quantization"
    # a1_scale / a2_scale only matter for FP8 without block_shape; the block and int8 configurations quantise the
    # activations themselves and, as in the reference, never look at them (fused_moe_triton_kernels.py:752-783)
    assert hidden_states.shape[1] == w1.shape[2], "Hidden size mismatch"
    assert topk_weights.shape == topk_ids.shape, "topk shape mismatch"
    assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert w1.is_contiguous(), "Expert weights1 must be contiguous"
    assert w2.is_contiguous(), "Expert weights2 must be contiguous"
    assert hidden_states.dtype in (torch.float16, torch.bfloat16)
    assert w1_scale is not None and w2_scale is not None

    num_tokens = hidden_states.shape[0]
    E, N, _ = w1.shape
    topk = topk_ids.shape[1]
    dev, dt = hidden_states.device, hidden_states.dtype

    wdt = torch.int8 if use_int8_w8a8 else torch.float8_e4m3fn
    assert w1.dtype == wdt and w2.dtype == wdt, "expert weights do not have the dtype the flags name"
    plain = (block_shape is not None and list(block_shape) == [128, 128] and b1 is None and b2 is None
             and not apply_router_weight_on_input)
    clamped = gemm1_alpha is not None or gemm1_limit is not None or swiglu_limit is not None
    fusable = (plain and activation == "silu" and is_gated and not clamped and use_fp8_w8a8 and not no_combine
               and hidden_states.shape[1] % 128 == 0 and N % 256 == 0
               and num_tokens > 0 and w1_scale.is_contiguous() and w2_scale.is_contiguous())
    if fusable:
        # whole sequence from one host call: its (at most five) launches are issued back to back from C
        out = hidden_states if inplace else torch.empty_like(hidden_states)
        tw = topk_weights if topk_weights.dtype == torch.float32 else topk_weights.to(torch.float32)
        fused_moe_block_fp8_(hidden_states, w1, w2, w1_scale, w2_scale, tw.contiguous(), topk_ids.contiguous(), out,
                             1.0 if routed_scaling_factor is None else routed_scaling_factor,
                             block_m=0 if config is None else config["BLOCK_SIZE_M"])
        return out
    if config is None:
        config = get_default_config(num_tokens, E, topk)
    if not plain and config["BLOCK_SIZE_M"] > 128:
        config = dict(config, BLOCK_SIZE_M=128)  # the generic kernel's tallest sorted block

    if no_combine:
        assert not inplace
        out_hidden_states = torch.empty((num_tokens, topk, w2.shape[1]), device=dev, dtype=dt)
    elif inplace:
        out_hidden_states = hidden_states
    else:
        out_hidden_states = torch.empty_like(hidden_states)
    if num_tokens == 0:
        return out_hidden_states
    if topk_weights.dtype != torch.float32:
        topk_weights = topk_weights.to(torch.float32)
    topk_weights = topk_weights.contiguous()

    sorted_token_ids, expert_ids, num_tokens_post_padded = moe_align_block_size(
        topk_ids.contiguous(), config["BLOCK_SIZE_M"], E)

    total_tokens = num_tokens * topk
    intermediate_cache1 = torch.empty((total_tokens, N), device=dev, dtype=dt)
    invoke_fused_moe_kernel(hidden_states, w1, intermediate_cache1, w1_scale, topk_weights, sorted_token_ids,
                            expert_ids, num_tokens_post_padded, apply_router_weight_on_input, topk, config, block_shape,
                            use_int8_w8a8=use_int8_w8a8, per_channel_quant=per_channel_quant, A_scale=a1_scale,
                            bias=b1)
    # fused_moe.py:530-647
    if is_gated and activation == "silu" and gemm1_alpha is not None:
        assert gemm1_limit is not None
        intermediate_cache2 = swiglu_gpt_oss_sigmoid_alpha(intermediate_cache1.view(-1, N), gemm1_alpha, gemm1_limit)
    elif is_gated and activation == "silu" and gemm1_limit is not None:
        intermediate_cache2 = _swiglu_silu_clamp_mul(intermediate_cache1.view(-1, N), gemm1_limit)
    elif is_gated:
        if activation == "gelu":
            assert gemm1_alpha is None, "gemm1_alpha is not supported for gelu"
            assert gemm1_limit is None, "gemm1_limit is not supported for gelu"
        elif swiglu_limit is not None:
            # the explicit clamp in front of silu_and_mul (fused_moe.py:565-569; the fused clamp kernels are CUDA-only)
            assert swiglu_limit == 10
            half = N // 2
            intermediate_cache1[:, :half].clamp_(max=swiglu_limit)
            intermediate_cache1[:, half:].clamp_(min=-swiglu_limit, max=swiglu_limit)
        intermediate_cache2 = torch.empty((total_tokens, N // 2), device=dev, dtype=dt)
        (silu_and_mul if activation == "silu" else gelu_and_mul)(intermediate_cache1.view(-1, N), intermediate_cache2)
    elif activation == "silu":
        intermediate_cache2 = torch.nn.functional.silu(intermediate_cache1.view(-1, N))
    elif activation == "gelu":
        intermediate_cache2 = torch.nn.functional.gelu(intermediate_cache1.view(-1, N))
    else:
        intermediate_cache2 = torch.square(torch.nn.functional.relu(intermediate_cache1.view(-1, N)))

    intermediate_cache3 = (out_hidden_states if no_combine
                           else torch.empty((num_tokens, topk, w2.shape[1]), device=dev, dtype=dt))
    invoke_fused_moe_kernel(intermediate_cache2, w2, intermediate_cache3, w2_scale, topk_weights, sorted_token_ids,
                            expert_ids, num_tokens_post_padded, not apply_router_weight_on_input and not no_combine, 1,
                            config, block_shape, use_int8_w8a8=use_int8_w8a8, per_channel_quant=per_channel_quant,
                            A_scale=a2_scale, bias=b2)
    if no_combine:
        return out_hidden_states
    if routed_scaling_factor is None:
        routed_scaling_factor = 1.0
    moe_sum_reduce(intermediate_cache3, out_hidden_states, routed_scaling_factor)
    return out_hidden_states


def _register_custom_op(fn, mutates_args):
    """Registers `fn` as torch.ops.sglang_amd.<name>, so that callers under torch.compile see one opaque node
    (the reference does the same for its own functions in the `sglang` namespace through register_custom_op,
    python/sglang/srt/utils/custom_op.py:57-165).  The namespace is this library's own on purpose: SGLang's
    registration skips a name that already exists under torch.ops.sglang (custom_op.py:152-165) and would then
    call this library's operator, which has no fall-through for the configurations it does not implement."""
    op = torch.library.custom_op(f"sglang_amd::{fn.__name__}", fn, mutates_args=mutates_args)
    if not mutates_args:
        op.register_fake(lambda hidden_states, *a, **k: torch.empty_like(hidden_states))
    return op


def inplace_fused_experts(
    hidden_states: torch.Tensor,
    w1: torch.Tensor,
    w2: torch.Tensor,
    topk_weights: torch.Tensor,
    topk_ids: torch.Tensor,
    b1: Optional[torch.Tensor] = None,
    b2: Optional[torch.Tensor] = None,
    activation: str = "silu",
    is_gated: bool = True,
    apply_router_weight_on_input: bool = False,
    use_fp8_w8a8: bool = False,
    use_int8_w8a8: bool = False,
    use_int8_w8a16: bool = False,
    use_int4_w4a16: bool = False,
    per_channel_quant: bool = False,
    w1_scale: Optional[torch.Tensor] = None,
    w2_scale: Optional[torch.Tensor] = None,
    w1_zp: Optional[torch.Tensor] = None,
    w2_zp: Optional[torch.Tensor] = None,
    a1_scale: Optional[torch.Tensor] = None,
    a2_scale: Optional[torch.Tensor] = None,
    block_shape: Optional[List[int]] = None,
    routed_scaling_factor: Optional[float] = None,
    gemm1_alpha: Optional[float] = None,
    gemm1_limit: Optional[float] = None,
    filter_expert: bool = True,
    swiglu_limit: Optional[float] = None,
) -> None:
    """fused_moe.py:91-151: the layer written over `hidden_states`."""
    fused_experts_impl(hidden_states, w1, w2, topk_weights, topk_ids, b1, b2, True, activation, is_gated,
                       apply_router_weight_on_input, use_fp8_w8a8, use_int8_w8a8, use_int8_w8a16, use_int4_w4a16,
                       per_channel_quant, w1_scale, w2_scale, w1_zp, w2_zp, a1_scale, a2_scale, block_shape, False,
                       routed_scaling_factor, gemm1_alpha, gemm1_limit, filter_expert, swiglu_limit=swiglu_limit)


def outplace_fused_experts(
    hidden_states: torch.Tensor,
    w1: torch.Tensor,
    w2: torch.Tensor,
    topk_weights: torch.Tensor,
    topk_ids: torch.Tensor,
    b1: Optional[torch.Tensor] = None,
    b2: Optional[torch.Tensor] = None,
    activation: str = "silu",
    is_gated: bool = True,
    apply_router_weight_on_input: bool = False,
    use_fp8_w8a8: bool = False,
    use_int8_w8a8: bool = False,
    use_int8_w8a16: bool = False,
    use_int4_w4a16: bool = False,
    per_channel_quant: bool = False,
    w1_scale: Optional[torch.Tensor] = None,
    w2_scale: Optional[torch.Tensor] = None,
    w1_zp: Optional[torch.Tensor] = None,
    w2_zp: Optional[torch.Tensor] = None,
    a1_scale: Optional[torch.Tensor] = None,
    a2_scale: Optional[torch.Tensor] = None,
    block_shape: Optional[List[int]] = None,
    no_combine: bool = False,
    routed_scaling_factor: Optional[float] = None,
    gemm1_alpha: Optional[float] = None,
    gemm1_limit: Optional[float] = None,
    filter_expert: bool = True,
    swiglu_limit: Optional[float] = None,
) -> torch.Tensor:
    """fused_moe.py:154-215: the layer into a fresh tensor ([tokens, topk, hidden] with no_combine)."""
    return fused_experts_impl(hidden_states, w1, w2, topk_weights, topk_ids, b1, b2, False, activation, is_gated,
                              apply_router_weight_on_input, use_fp8_w8a8, use_int8_w8a8, use_int8_w8a16,
                              use_int4_w4a16, per_channel_quant, w1_scale, w2_scale, w1_zp, w2_zp, a1_scale, a2_scale,
                              block_shape, no_combine=no_combine, routed_scaling_factor=routed_scaling_factor,
                              gemm1_alpha=gemm1_alpha, gemm1_limit=gemm1_limit, filter_expert=filter_expert,
                              swiglu_limit=swiglu_limit)


_inplace_op = _register_custom_op(inplace_fused_experts, ["hidden_states"])
_outplace_op = _register_custom_op(outplace_fused_experts, [])


def fused_experts(
    hidden_states: torch.Tensor,
    w1: torch.Tensor,
    w2: torch.Tensor,
    topk_output,
    moe_runner_config: MoeRunnerConfig,
    b1: Optional[torch.Tensor] = None,
    b2: Optional[torch.Tensor] = None,
    use_fp8_w8a8: bool = False,
    use_int8_w8a8: bool = False,
    use_int8_w8a16: bool = False,
    use_int4_w4a16: bool = False,
    per_channel_quant: bool = False,
    w1_scale: Optional[torch.Tensor] = None,
    w2_scale: Optional[torch.Tensor] = None,
    w1_zp: Optional[torch.Tensor] = None,
    w2_zp: Optional[torch.Tensor] = None,
    a1_scale: Optional[torch.Tensor] = None,
    a2_scale: Optional[torch.Tensor] = None,
    block_shape: Optional[List[int]] = None,
):
    """fused_moe.py:218-306: `topk_output` is (topk_weights, topk_ids, router_logits-or-None); the runner
    configuration picks the in-place or the out-of-place operator."""
    topk_weights, topk_ids, _ = topk_output
    c = moe_runner_config
    filter_expert = c.num_experts is None or c.num_experts != c.num_local_experts
    if c.inplace:
        assert not c.no_combine, "no combine + inplace makes no sense"
        _inplace_op(hidden_states, w1, w2, topk_weights, topk_ids, b1, b2, c.activation, c.is_gated,
                    c.apply_router_weight_on_input, use_fp8_w8a8, use_int8_w8a8, use_int8_w8a16, use_int4_w4a16,
                    per_channel_quant, w1_scale, w2_scale, w1_zp, w2_zp, a1_scale, a2_scale, block_shape,
                    c.routed_scaling_factor, c.gemm1_alpha, c.gemm1_clamp_limit, filter_expert,
                    swiglu_limit=c.swiglu_limit)
        return hidden_states
    return _outplace_op(hidden_states, w1, w2, topk_weights, topk_ids, b1, b2, c.activation, c.is_gated,
                        c.apply_router_weight_on_input, use_fp8_w8a8, use_int8_w8a8, use_int8_w8a16, use_int4_w4a16,
                        per_channel_quant, w1_scale, w2_scale, w1_zp, w2_zp, a1_scale, a2_scale, block_shape,
                        no_combine=c.no_combine, routed_scaling_factor=c.routed_scaling_factor,
                        gemm1_alpha=c.gemm1_alpha, gemm1_limit=c.gemm1_clamp_limit, filter_expert=filter_expert,
                        swiglu_limit=c.swiglu_limit)


def fused_moe(
    hidden_states: torch.Tensor,
    w1: torch.Tensor,
    w2: torch.Tensor,
    topk_output,
    moe_runner_config: MoeRunnerConfig = MoeRunnerConfig(),
    b1: Optional[torch.Tensor] = None,
    b2: Optional[torch.Tensor] = None,
    use_fp8_w8a8: bool = False,
    use_int8_w8a8: bool = False,
    use_int8_w8a16: bool = False,
    use_int4_w4a16: bool = False,
    per_channel_quant: bool = False,
    w1_scale: Optional[torch.Tensor] = None,
    w2_scale: Optional[torch.Tensor] = None,
    w1_zp: Optional[torch.Tensor] = None,
    w2_zp: Optional[torch.Tensor] = None,
    a1_scale: Optional[torch.Tensor] = None,
    a2_scale: Optional[torch.Tensor] = None,
    block_shape: Optional[List[int]] = None,
) -> torch.Tensor:
    """fused_moe.py:896-998.  The default runner configuration works in place, as in the reference."""
    return fused_experts(hidden_states, w1, w2, topk_output, moe_runner_config=moe_runner_config, b1=b1, b2=b2,
                         use_fp8_w8a8=use_fp8_w8a8, use_int8_w8a8=use_int8_w8a8, use_int8_w8a16=use_int8_w8a16,
                         use_int4_w4a16=use_int4_w4a16, per_channel_quant=per_channel_quant, w1_scale=w1_scale,
                         w2_scale=w2_scale, w1_zp=w1_zp, w2_zp=w2_zp, a1_scale=a1_scale, a2_scale=a2_scale,
                         block_shape=block_shape)
