"""Chooses the attention kernel for a step by dtype and the step's shape."""

from __future__ import annotations

import torch

from . import ops


def paged_attention(qkv: torch.Tensor, num_heads: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    block_table: torch.Tensor, step, *, window: int, scale: float) -> torch.Tensor:
    """Attention of every token of the step over its request's cache pages -> [N, nq * D].

    ``qkv`` holds each token's query heads first in its row (rotated already).
    """
    return ops.paged_attention_plain(qkv, qkv.shape[1], k_cache, v_cache, block_table,
                                     step.token_entry, step.positions, num_heads, window, scale)
