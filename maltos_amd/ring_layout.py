"""Zigzag context-parallel token layout.

Counterpart of the reference's runtime/layers/ring_layout.py:6-43 and of the planner at
parallel/context_token_planner.py:78-103: with W ranks the sequence is cut into 2W half-chunks of
`half = local_seq_len / 2` tokens and rank r owns half-chunks r and 2W-1-r, which gives every rank
the same causal work per ring step.
"""
from __future__ import annotations

import torch


def expected_zigzag_ring_positions(local_seq_len: int, *, rank: int, world_size: int, device: torch.device) -> torch.Tensor:
    """Global positions (int64 [local_seq_len]) of the tokens rank `rank` holds."""
    if local_seq_len % 2:
        raise ValueError(f"zigzag ring attention requires an even local sequence length, got local_seq_len={local_seq_len}")
    half = local_seq_len // 2
    local = torch.arange(local_seq_len, device=device, dtype=torch.long)
    in_back_half = local >= half
    chunk = torch.where(in_back_half, 2 * world_size - 1 - rank, rank)
    return chunk * half + (local - in_back_half.long() * half)


def has_zigzag_ring_layout(position_ids: torch.Tensor, *, rank: int, world_size: int) -> bool:
    """True iff every row of a [batch, seq] position tensor is exactly this rank's zigzag layout."""
    if position_ids.dim() != 2 or position_ids.size(1) % 2:
        return False
    want = expected_zigzag_ring_positions(position_ids.size(1), rank=rank, world_size=world_size, device=position_ids.device)
    return bool((position_ids == want).all())
