"""One rank's side of the reference's all-gather context-parallel attention core.

`AllGatherKvAttentionCore.forward` (runtime/layers/all_gather_attention.py:18-71) gathers K, V, the positions and the
sequence ids of every rank along the sequence and runs one example-aware attention of the local queries over all of
them (`flash_varlen_mode="prefix"`: in the reference a Python loop packs query runs and key prefixes for the varlen
kernel).  Here the gathered tensors go to the document-mask kernel as they are: it takes positions and sequence ids
per token, in any order, and skips the 64-key tiles no query can see.  What gathers is a seam (one GPU here):
`kv_source(rank, k, v)` and `meta_source(rank, positions, sequence_ids)` return the per-rank lists.
"""
from __future__ import annotations

from typing import Callable, Sequence

import torch
import torch.nn as nn

from .attention_backend import AttentionBackend, causal_attention, validate_attention_backend
from .attn_masking_utils import canonical_position_ids, canonical_sequence_ids

KvChunk = tuple[torch.Tensor, torch.Tensor]


class HipAllGatherKvAttentionCore(nn.Module):
    """`attn_core` drop-in (q, k, v, position_offset, position_ids, sequence_ids) -> out."""

    preserves_native_gqa = True

    def __init__(self, *, rank: int, world_size: int,
                 kv_source: Callable[[int, torch.Tensor, torch.Tensor], Sequence[KvChunk]],
                 meta_source: Callable[[int, torch.Tensor, torch.Tensor | None], Sequence[tuple[torch.Tensor, torch.Tensor | None]]],
                 attention_backend: str = AttentionBackend.HIP) -> None:
        super().__init__()
        if not 0 <= rank < world_size:
            raise ValueError(f"bad rank {rank} for world_size {world_size}")
        self.rank, self.world_size, self.kv_source, self.meta_source = rank, world_size, kv_source, meta_source
        self.attention_backend = validate_attention_backend(attention_backend)

    def forward(self, q, k, v, position_offset: int, position_ids=None, sequence_ids=None) -> torch.Tensor:
        positions = canonical_position_ids(position_ids, batch_size=q.size(0), seq_len=q.size(-2),
                                           position_offset=position_offset, device=q.device)
        sequences = canonical_sequence_ids(sequence_ids, batch_size=q.size(0), seq_len=q.size(-2), device=q.device)
        chunks = self.kv_source(self.rank, k, v)
        meta = self.meta_source(self.rank, positions, sequences)
        if len(chunks) != self.world_size or len(meta) != self.world_size:
            raise ValueError(f"need K/V and positions of each of the {self.world_size} ranks")
        have_ids = [m[1] is not None for m in meta]
        if any(have_ids) != all(have_ids) or all(have_ids) != (sequences is not None):
            raise ValueError("sequence ids must be given by every rank or by none")
        return causal_attention(
            q, torch.cat([c[0] for c in chunks], dim=2), torch.cat([c[1] for c in chunks], dim=2),
            attention_backend=self.attention_backend, warning_prefix="HipAllGatherKvAttentionCore",
            q_positions=positions, k_positions=torch.cat([m[0] for m in meta], dim=1), q_sequence_ids=sequences,
            k_sequence_ids=torch.cat([m[1] for m in meta], dim=1) if sequences is not None else None,
            flash_varlen_mode="prefix")
