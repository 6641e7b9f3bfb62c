"""Allocating wrapper around the moe_align_block_size operator
(python/sglang/srt/layers/moe/moe_runner/triton_utils/moe_align_block_size.py:19-87)."""
from typing import Tuple

import torch

from ..moe import moe_align_block_size as sgl_moe_align_block_size


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int) -> Tuple[torch.Tensor, ...]:
    """Returns (sorted_token_ids, expert_ids, num_tokens_post_padded) for `topk_ids` [tokens, top_k].
    One extra bucket is passed to the operator so that id -1 (expert not on this rank) gets
    expert_ids == -1 blocks."""
    if topk_ids.numel() < num_experts + 1:
        max_num_tokens_padded = topk_ids.numel() * block_size
    else:
        max_num_tokens_padded = topk_ids.numel() + (num_experts + 1) * (block_size - 1)
    sorted_ids = torch.empty((max_num_tokens_padded,), dtype=torch.int32, device=topk_ids.device)
    max_num_m_blocks = (max_num_tokens_padded + block_size - 1) // block_size
    expert_ids = torch.empty((max_num_m_blocks,), dtype=torch.int32, device=topk_ids.device)
    num_tokens_post_pad = torch.empty((1), dtype=torch.int32, device=topk_ids.device)
    cumsum_buffer = torch.empty((num_experts + 2,), dtype=torch.int32, device=topk_ids.device)
    sgl_moe_align_block_size(topk_ids, num_experts + 1, block_size, sorted_ids, expert_ids, num_tokens_post_pad,
                             cumsum_buffer, True)
    return sorted_ids, expert_ids, num_tokens_post_pad
