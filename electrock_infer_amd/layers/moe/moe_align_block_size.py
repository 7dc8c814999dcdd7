"""Host wrapper of the expert sort, mirroring
electrock_infer/layers/moe/moe_align_block_size.py:6-61 of the reference:
same signature, same buffer sizes, same return triple."""
from typing import Tuple

import torch

from ... import _C


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int,
                         num_experts: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Sort the flat (token, k) slots by expert and pad every expert segment to
    a multiple of ``block_size``.

    Returns ``(sorted_token_ids, expert_ids, num_tokens_post_pad)`` with the
    reference's worst-case lengths ``numel + E*(block_size-1)`` and
    ``cdiv(that, block_size)``; pads are -1, unused ``expert_ids`` are 0.
    The kernel defines every element itself, so the buffers are not pre-filled.
    """
    max_num_tokens_padded = topk_ids.numel() + num_experts * (block_size - 1)
    sorted_ids = torch.empty((max_num_tokens_padded,), dtype=torch.int32, device=topk_ids.device)
    max_num_m_blocks = (max_num_tokens_padded + block_size - 1) // block_size
    expert_ids = torch.empty((max_num_m_blocks,), dtype=torch.int32, device=topk_ids.device)
    num_tokens_post_pad = torch.empty((1,), dtype=torch.int32, device=topk_ids.device)
    _C.moe_align_block_size(topk_ids, num_experts, block_size, sorted_ids, expert_ids, num_tokens_post_pad)
    return sorted_ids, expert_ids, num_tokens_post_pad
