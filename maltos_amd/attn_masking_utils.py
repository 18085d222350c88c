"""Canonical [batch, seq] position / sequence ids and the example-aware visibility rule.

Host-side counterpart of the reference's runtime/layers/attn_masking_utils.py:6-87: same public
names, argument meaning and ValueError conditions.  The HIP kernels evaluate the rule
(`k_pos <= q_pos` and equal sequence ids) in registers per score and never materialise the boolean
tensor; `build_example_causal_mask` is kept for callers and tests that want the tensor itself.
"""
from __future__ import annotations

import torch


def _as_batch_rows(ids: torch.Tensor, what: str, batch_size: int, seq_len: int, device: torch.device) -> torch.Tensor:
    """Rank-1 ids are shared by every row of the batch, rank-2 ids must already be [batch, seq]."""
    rank = ids.dim()
    if rank not in (1, 2):
        raise ValueError(f"{what} must have rank 1 or 2, got shape={tuple(ids.shape)}")
    ids = ids.to(device=device, dtype=torch.long)
    if rank == 1:
        if ids.numel() != seq_len:
            raise ValueError(f"{what} length must match seq_len, got {ids.numel()} vs {seq_len}")
        return ids.repeat(batch_size, 1)
    if tuple(ids.shape) != (batch_size, seq_len):
        raise ValueError(f"{what} shape must match [batch, seq], got {tuple(ids.shape)} vs ({batch_size}, {seq_len})")
    return ids.contiguous()


def canonical_position_ids(position_ids: torch.Tensor | None, *, batch_size: int, seq_len: int, position_offset: int,
                           device: torch.device) -> torch.Tensor:
    """int64 [batch, seq]; without ids the positions are position_offset .. position_offset + seq_len - 1."""
    if position_ids is None:
        position_ids = torch.arange(seq_len, device=device, dtype=torch.long) + int(position_offset)
    return _as_batch_rows(position_ids, "position_ids", batch_size, seq_len, device)


def canonical_sequence_ids(sequence_ids: torch.Tensor | None, *, batch_size: int, seq_len: int,
                           device: torch.device) -> torch.Tensor | None:
    """int64 [batch, seq], or None when the batch carries no document ids."""
    if sequence_ids is None:
        return None
    return _as_batch_rows(sequence_ids, "sequence_ids", batch_size, seq_len, device)


def build_example_causal_mask(*, q_positions: torch.Tensor, k_positions: torch.Tensor,
                              q_sequence_ids: torch.Tensor | None = None,
                              k_sequence_ids: torch.Tensor | None = None) -> torch.Tensor:
    """bool [batch, q, k]: key visible iff its position does not exceed the query's and, when ids are
    given, both belong to the same sequence."""
    for name, t in (("q_positions", q_positions), ("k_positions", k_positions)):
        if t.dim() != 2:
            raise ValueError(f"{name} must be a rank-2 [batch, seq] tensor, got {tuple(t.shape)}")
    if q_positions.size(0) != k_positions.size(0):
        raise ValueError(f"q_positions and k_positions must have same batch size, got {q_positions.size(0)} vs {k_positions.size(0)}")
    if (q_sequence_ids is None) != (k_sequence_ids is None):
        raise ValueError("q_sequence_ids and k_sequence_ids must both be provided or both be None")
    visible = q_positions[:, :, None] >= k_positions[:, None, :]
    if q_sequence_ids is None:
        return visible
    for name, ids, pos in (("q", q_sequence_ids, q_positions), ("k", k_sequence_ids, k_positions)):
        if ids.shape != pos.shape:
            raise ValueError(f"{name}_sequence_ids shape must match {name}_positions, got {tuple(ids.shape)} vs {tuple(pos.shape)}")
    return visible & (q_sequence_ids[:, :, None] == k_sequence_ids[:, None, :])
