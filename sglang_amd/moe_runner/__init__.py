"""Host side of the fused MoE, mirroring
python/sglang/srt/layers/moe/moe_runner/{base,triton}.py and moe_runner/triton_utils/{moe_align_block_size,fused_moe}.py."""
from .base import (  # noqa: F401
    MoeRunnerConfig,
    StandardCombineInput,
    StandardDispatchOutput,
    StandardTopKOutput,
    TritonMoeQuantInfo,
    fused_experts_none_to_triton,
)
from .fused_moe import (  # noqa: F401
    fused_experts,
    fused_experts_impl,
    fused_moe,
    get_default_config,
    inplace_fused_experts,
    outplace_fused_experts,
)
from .moe_align_block_size import moe_align_block_size  # noqa: F401
