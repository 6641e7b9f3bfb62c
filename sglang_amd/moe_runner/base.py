"""Records that carry a fused-MoE call between SGLang's layers and a runner backend, and the fused function this
library offers to the runner pool.

Field for field the reference's types: ``MoeRunnerConfig`` (python/sglang/srt/layers/moe/moe_runner/base.py:45-67),
``TritonMoeQuantInfo`` (moe_runner/triton.py:52-69), ``StandardTopKOutput`` (layers/moe/topk.py:252-262),
``StandardDispatchOutput`` / ``StandardCombineInput`` (layers/moe/token_dispatcher/standard.py:59-82).  A running
SGLang hands its own instances to ``fused_experts_none_to_triton``; only attribute names are relied on, so either
set of classes works, and these let the path run and be tested where SGLang is not installed."""
from dataclasses import dataclass
from typing import Any, List, NamedTuple, Optional

import torch


@dataclass
class MoeRunnerConfig:
    # MoE parameters
    num_experts: Optional[int] = None
    num_local_experts: Optional[int] = None
    hidden_size: Optional[int] = None
    intermediate_size_per_partition: Optional[int] = None
    layer_id: Optional[int] = None
    top_k: Optional[int] = None
    num_fused_shared_experts: Optional[int] = None
    params_dtype: Optional[torch.dtype] = None
    routing_method_type: Optional[Any] = None

    # Runner configuration
    activation: str = "silu"
    is_gated: bool = True
    apply_router_weight_on_input: bool = False
    inplace: bool = True
    no_combine: bool = False
    routed_scaling_factor: Optional[float] = None
    gemm1_alpha: Optional[float] = None
    gemm1_clamp_limit: Optional[float] = None
    swiglu_limit: Optional[float] = None


@dataclass
class TritonMoeQuantInfo:
    w13_weight: torch.Tensor
    w2_weight: torch.Tensor
    b13: Optional[torch.Tensor] = None
    b2: Optional[torch.Tensor] = None
    use_fp8_w8a8: bool = False
    use_int8_w8a8: bool = False
    use_int8_w8a16: bool = False
    use_int4_w4a16: bool = False
    per_channel_quant: bool = False
    w13_scale: Optional[torch.Tensor] = None
    w2_scale: Optional[torch.Tensor] = None
    w13_zp: Optional[torch.Tensor] = None
    w2_zp: Optional[torch.Tensor] = None
    a13_scale: Optional[torch.Tensor] = None
    a2_scale: Optional[torch.Tensor] = None
    block_shape: Optional[List[int]] = None


class StandardTopKOutput(NamedTuple):
    topk_weights: torch.Tensor
    topk_ids: torch.Tensor
    router_logits: Optional[torch.Tensor]

    @property
    def format(self) -> str:
        return "standard"


class StandardDispatchOutput(NamedTuple):
    hidden_states: torch.Tensor
    hidden_states_scale: Optional[torch.Tensor]
    topk_output: Any

    @property
    def format(self) -> str:
        return "standard"


class StandardCombineInput(NamedTuple):
    hidden_states: torch.Tensor

    @property
    def format(self) -> str:
        return "standard"


def _combine_input_type():
    """SGLang's own StandardCombineInput when it is importable (its combine step checks the format enum)."""
    try:
        from sglang.srt.layers.moe.token_dispatcher.standard import StandardCombineInput as theirs

        return theirs
    except ImportError:
        return StandardCombineInput


def fused_experts_none_to_triton(dispatch_output, quant_info, runner_config):
    """The fused function of the ("none", "triton") slot of the runner pool (moe_runner/triton.py:139-172;
    looked up by MoeRunner, moe_runner/runner.py:67-76, and called as fused_func(dispatch_output, quant_info,
    config), :97-98).  Raises NotImplementedError before any work for configurations this library does not
    implement, so that a caller can fall back."""
    from .fused_moe import fused_experts

    output = fused_experts(
        hidden_states=dispatch_output.hidden_states,
        w1=quant_info.w13_weight,
        w2=quant_info.w2_weight,
        topk_output=dispatch_output.topk_output,
        moe_runner_config=runner_config,
        b1=quant_info.b13,
        b2=quant_info.b2,
        use_fp8_w8a8=quant_info.use_fp8_w8a8,
        use_int8_w8a8=quant_info.use_int8_w8a8,
        use_int8_w8a16=quant_info.use_int8_w8a16,
        use_int4_w4a16=quant_info.use_int4_w4a16,
        per_channel_quant=quant_info.per_channel_quant,
        w1_scale=quant_info.w13_scale,
        w2_scale=quant_info.w2_scale,
        w1_zp=quant_info.w13_zp,
        w2_zp=quant_info.w2_zp,
        a1_scale=quant_info.a13_scale,
        a2_scale=quant_info.a2_scale,
        block_shape=quant_info.block_shape,
    )
    return _combine_input_type()(hidden_states=output)
