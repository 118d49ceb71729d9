"""Chooses the attention kernel for a step by dtype and the step's shape."""

from __future__ import annotations

import torch

from . import ops

# The decode kernel aims at two workgroups per compute unit, more for small heads (a workgroup keeps three 32-key tiles
# in flight, whose bytes go with the head size): whole decode steps at 4,096 keys, 7B sizes, 256 units, take 4.05 / 5.28 /
# 6.28 ms at 16 / 32 / 48 requests against 4.13 / 5.35 / 6.32 with one per unit; at 64 requests one workgroup each
# (no split) is 2.5 % slower than two, from 128 on the requests alone give two per unit and nothing is split (the
# merge kernel goes: 128 requests 4.9 % faster than with a forced split).
MIN_SPLIT = 64                  # keys per split at least (a multiple of the 16-key tile)
MAX_SPLITS = 1024               # what the merge kernel holds
DECODE_PORTION = 8              # portions of at most this many tokens take the decode kernel; the attention part
                                # declares it as its entry_split, so the step lists long entries and short tokens by it
UNIT_HEAD_DIM = 128             # workgroups per compute unit: UNIT_HEAD_DIM / head size, at least MIN_PER_UNIT
MIN_PER_UNIT = 2


def decode_splits(num_tokens: int, groups: int, max_context: int, page_size: int = 0,
                  head_dim: int = 128) -> tuple[int, int]:
    """(split_len, num_splits): how the keys of a request are cut over workgroups so that
    ``num_tokens * groups * num_splits`` is about MIN_PER_UNIT times the number of compute units.  Boundaries are multiples of
    MIN_SPLIT in absolute positions.  With ``page_size`` a split is no longer than what the kernel that stages
    tiles through LDS takes (its list of a split's pages is in LDS): contexts beyond that are cut further instead
    of falling to the slower kernel (64 requests at 4,1xx tokens in tables 512 pages wide: 8.2 ms a step before,
    against 6.8 at 3,9xx tokens)."""
    max_context = max(1, max_context)
    most = (max_context + MIN_SPLIT - 1) // MIN_SPLIT
    workgroups = ops.compute_units() * max(MIN_PER_UNIT, UNIT_HEAD_DIM // max(1, head_dim))
    splits = max(1, min(workgroups // max(1, num_tokens * groups), most, MAX_SPLITS))
    split_len = ((max_context + splits - 1) // splits + MIN_SPLIT - 1) // MIN_SPLIT * MIN_SPLIT
    if page_size > 0:
        longest = ops.library().somi_attention_decode_lds_split(int(page_size))
        if MIN_SPLIT <= longest < split_len and (max_context + longest - 1) // longest <= MAX_SPLITS:
            split_len = longest
    return split_len, (max_context + split_len - 1) // split_len


def mfma_attention_supported(q: torch.Tensor, k_cache: torch.Tensor) -> bool:
    head_dim, page_size = k_cache.shape[3], k_cache.shape[2]
    return (q.dtype == torch.bfloat16 and head_dim % 16 == 0 and head_dim <= 256 and page_size % 4 == 0
            and q.data_ptr() % 16 == 0 and (q.shape[1] * 2) % 16 == 0)


def paged_attention(qkv: torch.Tensor, num_heads: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    block_table: torch.Tensor, step, *, window: int, scale: float) -> torch.Tensor:
    """Attention of every token of the step over its request's cache pages -> [N, nq * D].

    ``qkv`` holds each token's query heads first in its row (rotated already).  float32, and shapes the
    MFMA kernels do not take (head sizes that are no multiple of 16, page sizes that are no multiple
    of 4), run the plain kernel.
    """
    if not mfma_attention_supported(qkv, k_cache):
        return ops.paged_attention_plain(qkv, qkv.shape[1], k_cache, v_cache, block_table,
                                         step.token_entry, step.positions, num_heads, window, scale)
    nkv, head_dim = k_cache.shape[1], k_cache.shape[3]
    groups = nkv * ((num_heads // nkv + 15) // 16)
    out = torch.empty((qkv.shape[0], num_heads * head_dim), dtype=qkv.dtype, device=qkv.device)
    if step.max_entry_len > DECODE_PORTION:
        # portions of prompts: query tiles against key tiles.  Single tokens (and portions of a few) in the same
        # batch keep the kernel that splits a request's keys over workgroups: as a query tile with one live row
        # one workgroup would walk the whole context.
        split = step.split(DECODE_PORTION)
        short = split.num_short_tokens
        if split.num_long_tokens + short != step.num_tokens or short != split.short_tokens.numel():
            raise ValueError(f"the step's split at {DECODE_PORTION} tokens covers {split.num_long_tokens} + {short} "
                             f"of its {step.num_tokens} tokens: rows of the output would stay unwritten")
        ops.attention_prefill(qkv, qkv.shape[1], k_cache, v_cache, block_table, step.entry_start,
                              step.entry_first_position, step.max_entry_len, num_heads, window, scale, out,
                              max_context=step.max_context, entry_len=split.long_entry_len if short else None)
        if short:
            split_len, num_splits = decode_splits(short, groups, step.max_context, k_cache.shape[2], head_dim)
            ops.attention_decode(qkv, qkv.shape[1], k_cache, v_cache, block_table, step.token_entry, step.positions,
                                 num_heads, window, scale, split_len, num_splits, out, token_list=split.short_tokens)
        return out
    split_len, num_splits = decode_splits(step.num_tokens, groups, step.max_context, k_cache.shape[2], head_dim)
    ops.attention_decode(qkv, qkv.shape[1], k_cache, v_cache, block_table, step.token_entry, step.positions,
                         num_heads, window, scale, split_len, num_splits, out)
    return out
