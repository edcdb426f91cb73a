"""Chooses the differential-attention kernel for a step by dtype and the step's shape."""

from __future__ import annotations

import torch

from . import ops

DECODE_PORTION = 8      # portions of at most this many tokens count as decoded tokens; the part declares it as its
                        # entry_split, so the step lists long entries and short tokens by it


def diff_attention(qkv: torch.Tensor, num_heads: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                   block_table: torch.Tensor, step, *, window: int, keep_first: int, scale: float, lam: float,
                   eps: float, out_scale: float) -> torch.Tensor:
    """Differential attention of every token of the step over its request's cache pages -> [N, heads * value_dim].
    ``qkv`` holds each token's 2 * heads query maps first in its row (rotated already)."""
    return ops.diff_attention_plain(qkv, k_cache, v_cache, block_table, step.token_entry, step.positions, num_heads,
                                    window, keep_first, scale, lam, eps, out_scale)
