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
    ``qkv`` holds each token's 2 * heads query maps first in its row (rotated already).  float32, and sizes the
    matrix-core kernel is not built for, run the plain kernel.  Portions of more than DECODE_PORTION tokens are cut
    into query tiles of consecutive tokens; the tokens of the other entries (decoded tokens, portions of a few) each
    get a tile of their own, so that their workgroups' four wavefronts share the token's keys."""
    if not ops.diff_attention_mfma_supported(qkv, k_cache, v_cache):
        return ops.diff_attention_plain(qkv, k_cache, v_cache, block_table, step.token_entry, step.positions, num_heads,
                                        window, keep_first, scale, lam, eps, out_scale)
    out = torch.empty((qkv.shape[0], num_heads * v_cache.shape[2]), dtype=qkv.dtype, device=qkv.device)
    common = (qkv, k_cache, v_cache, block_table, num_heads, window, keep_first, scale, lam, eps, out_scale, out)
    if step.max_entry_len > DECODE_PORTION:
        split = step.split(DECODE_PORTION)
        short = split.num_short_tokens
        if split.num_long_tokens + short != step.num_tokens or short != split.short_tokens.numel():
            raise ValueError(f"the step's split at {DECODE_PORTION} tokens covers {split.num_long_tokens} + {short} "
                             f"of its {step.num_tokens} tokens: rows of the output would stay unwritten")
        ops.diff_attention_mfma(*common, entry_start=step.entry_start, entry_first_position=step.entry_first_position,
                                entry_len=split.long_entry_len if short else None, max_entry_len=step.max_entry_len)
        if short:
            ops.diff_attention_mfma(*common, token_list=split.short_tokens, token_entry=step.token_entry,
                                    positions=step.positions)
        return out
    ops.diff_attention_mfma(*common, token_entry=step.token_entry, positions=step.positions)
    return out
