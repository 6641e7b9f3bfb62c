"""Host side of the fused MoE, mirroring
python/sglang/srt/layers/moe/moe_runner/triton_utils/{moe_align_block_size,fused_moe}.py."""
from .fused_moe import fused_experts, fused_experts_impl, fused_moe, get_default_config  # noqa: F401
from .moe_align_block_size import moe_align_block_size  # noqa: F401
