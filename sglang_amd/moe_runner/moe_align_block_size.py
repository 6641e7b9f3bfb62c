"""Allocating wrapper around the moe_align_block_size operator
(python/sglang/srt/layers/moe/moe_runner/triton_utils/moe_align_block_size.py:19-87)."""
from typing import Tuple

import torch

from ..moe import moe_align_block_size as sgl_moe_align_block_size


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int) -> Tuple[torch.Tensor, ...]:
    """Returns (sorted_token_ids, expert_ids, num_tokens_post_padded) for `topk_ids` [tokens, top_k].
    One extra bucket is passed to the operator so that id -1 (expert not on this rank) gets
    expert_ids == -1 blocks."""
    pairs = topk_ids.numel()
    buckets = num_experts + 1
    # every non-empty bucket pads by at most block_size - 1 slots, and at most `pairs` buckets are non-empty
    slots = pairs + min(pairs, buckets) * (block_size - 1)
    i32 = dict(dtype=torch.int32, device=topk_ids.device)
    sorted_ids = torch.empty(slots, **i32)
    expert_ids = torch.empty(-(-slots // block_size), **i32)
    num_tokens_post_pad = torch.empty(1, **i32)
    cumsum_buffer = torch.empty(buckets + 1, **i32)
    sgl_moe_align_block_size(topk_ids, buckets, block_size, sorted_ids, expert_ids, num_tokens_post_pad,
                             cumsum_buffer, True)
    return sorted_ids, expert_ids, num_tokens_post_pad
