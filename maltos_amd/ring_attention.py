"""Zigzag ring (context-parallel) block attention: one rank's compute on one GPU.

Counterpart of the reference's flash ring path (runtime/layers/functional.py:619-645,751-820,
1012-1166 and RingAttentionCore, runtime/layers/ring_attention.py:21-113).  A rank holds the local
Q/K/V chunk in zigzag layout and, ring step by ring step, the K/V chunk of rank (rank - step) mod W:
    step 0        square causal block on the local chunk
    step <= rank  all local queries x the FRONT half of the remote chunk, no mask
    step >  rank  the TAIL half of the local queries x the whole remote chunk, no mask
Block outputs are merged in fp32 with a log-sum-exp merge; the backward pass re-runs the same
schedule with the GLOBAL out / LSE and accumulates dQ and the per-chunk dK/dV in fp32.

Packed documents (sequence ids given) take the other path of the reference
(_flash_packed_ring_forward/backward, functional.py:823-1009): every step attends all local queries to the whole
arriving chunk under the document mask "same sequence id, not PAD, k_pos <= q_pos", with the positions and sequence
ids travelling with the chunk.  The reference packs runs and key prefixes for flash_attn_varlen (flash_utils.py:
566-962, a Python loop with host reads per run); here the kernels take the ids directly and skip the 64-key tiles
no query can see, so there is no packing step and no host synchronisation.

What moves K/V between ranks is a separate concern (the reference uses P2P send/recv): here it is
the `kv_source` callable, which returns the chunk a step needs.  On one GPU the chunks are simply
resident; nothing in this module touches torch.distributed.
"""
from __future__ import annotations

from typing import Callable, Sequence

import torch
import torch.nn as nn

from . import ops
from .attention_backend import AttentionBackend, causal_attention, validate_attention_backend
from .attn_masking_utils import canonical_position_ids, canonical_sequence_ids
from .flash_utils import flash_attn_dense_with_lse

KvChunk = tuple[torch.Tensor, torch.Tensor]


def zigzag_ring_schedule(rank: int, world_size: int) -> list[tuple[int, str]]:
    """[(source rank of the K/V chunk, block kind)] for ring steps 0..W-1."""
    if not 0 <= rank < world_size:
        raise ValueError(f"rank {rank} outside world of {world_size}")
    plan = []
    for step in range(world_size):
        kind = "causal" if step == 0 else ("front_kv" if step <= rank else "tail_q")
        plan.append(((rank - step) % world_size, kind))
    return plan


def _first_block_state(blk) -> tuple[torch.Tensor, torch.Tensor]:
    """The running fp32 (out, lse) of a schedule whose first block covers every local query: that block itself (one
    conversion instead of clearing the state and merging the block into it)."""
    running_out = torch.empty(blk.out.shape, dtype=torch.float32, device=blk.out.device)
    running_out.copy_(blk.out)
    return running_out, blk.lse


class _ZigzagRingFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q: torch.Tensor, rank: int, world_size: int, *kv_flat: torch.Tensor):
        if len(kv_flat) != 2 * world_size:
            raise ValueError(f"expected {2 * world_size} K/V tensors, got {len(kv_flat)}")
        seq = q.size(-2)
        if seq % 2:
            raise ValueError(f"zigzag ring attention requires an even local sequence length, got {seq}")
        half = seq // 2
        running_out = running_lse = None
        for src, kind in zigzag_ring_schedule(rank, world_size):
            k, v = kv_flat[2 * src], kv_flat[2 * src + 1]
            if kind == "causal":  # step 0, all local queries
                running_out, running_lse = _first_block_state(flash_attn_dense_with_lse(q, k, v, causal=True))
            elif kind == "front_kv":
                blk = flash_attn_dense_with_lse(q, k[:, :, :half], v[:, :, :half], causal=False)
                ops.attention_merge_(running_out, running_lse, blk.out, blk.lse, 0)
            else:
                blk = flash_attn_dense_with_lse(q[:, :, half:], k, v, causal=False)
                ops.attention_merge_(running_out, running_lse, blk.out, blk.lse, half)
        out = running_out.to(dtype=kv_flat[1].dtype)
        ctx.save_for_backward(q, out, running_lse, *kv_flat)
        ctx.rank, ctx.world_size = rank, world_size
        ctx.mark_non_differentiable(running_lse)
        return out, running_lse

    @staticmethod
    def backward(ctx, dout: torch.Tensor, _dlse):
        q, out, lse, *kv_flat = ctx.saved_tensors
        rank, world_size = ctx.rank, ctx.world_size
        half = q.size(-2) // 2
        dout = dout.contiguous()
        # dq collects every step in fp32: the first step (causal, all local queries) overwrites it, the others add.
        # A chunk's dK / dV come from exactly one step, so that step writes them in their final dtype; only the half
        # of a chunk that a front_kv step does not touch is cleared.
        dq = torch.empty(q.shape, dtype=torch.float32, device=q.device)
        grads: list[torch.Tensor | None] = [None] * len(kv_flat)
        for step, (src, kind) in enumerate(zigzag_ring_schedule(rank, world_size)):
            k, v = kv_flat[2 * src], kv_flat[2 * src + 1]
            dk, dv = torch.empty_like(k), torch.empty_like(v)
            grads[2 * src], grads[2 * src + 1] = dk, dv
            if kind == "causal":
                ops.attention_backward_ring_block(dout, q, k, v, out, lse, dq, dk, dv, first=step == 0, mask_mode=ops.MASK_CAUSAL)
            elif kind == "front_kv":
                dk[:, :, half:].zero_()
                dv[:, :, half:].zero_()
                ops.attention_backward_ring_block(dout, q, k[:, :, :half], v[:, :, :half], out, lse, dq, dk[:, :, :half],
                                                  dv[:, :, :half], first=False, mask_mode=ops.MASK_NONE)
            else:
                ops.attention_backward_ring_block(dout[:, :, half:], q[:, :, half:], k, v, out[:, :, half:],
                                                  lse[:, :, half:].contiguous(), dq[:, :, half:], dk, dv, first=False,
                                                  mask_mode=ops.MASK_NONE)
        return (dq.to(q.dtype), None, None, *grads)


def flash_attn_dense_block(q, k, v, q_pos, k_pos, q_seq, k_seq):
    """One document-masked block without autograd: (out, lse) as flash_attn_dense_with_lse returns them."""
    from .flash_utils import FlashAttnBlockOutput

    out, lse = ops.attention_forward(q, k, v, mask_mode=ops.MASK_DOC, q_pos=q_pos, k_pos=k_pos, q_seq=q_seq, k_seq=k_seq)
    return FlashAttnBlockOutput(out=out, lse=lse)


class _PackedRingFunction(torch.autograd.Function):
    """flat = (k, v, positions, sequence_ids) of rank 0, of rank 1, ...; ids are int [B, S_chunk]."""

    @staticmethod
    def forward(ctx, q: torch.Tensor, q_pos: torch.Tensor, q_seq: torch.Tensor, rank: int, world_size: int, *flat):
        if len(flat) != 4 * world_size:
            raise ValueError(f"expected {4 * world_size} chunk tensors, got {len(flat)}")
        running_out = running_lse = None
        for step in range(world_size):
            k, v, k_pos, k_seq = flat[4 * ((rank - step) % world_size):][:4]
            blk = flash_attn_dense_block(q, k, v, q_pos, k_pos, q_seq, k_seq)
            if step == 0:
                running_out, running_lse = _first_block_state(blk)
            else:
                ops.attention_merge_(running_out, running_lse, blk.out, blk.lse, 0)  # a block nobody sees into is (0, -inf)
        out = running_out.to(dtype=flat[1].dtype)
        ctx.save_for_backward(q, q_pos, q_seq, out, running_lse, *flat)
        ctx.rank, ctx.world_size = rank, world_size
        ctx.mark_non_differentiable(running_lse)
        return out, running_lse

    @staticmethod
    def backward(ctx, dout: torch.Tensor, _dlse):
        q, q_pos, q_seq, out, lse, *flat = ctx.saved_tensors
        rank, world_size = ctx.rank, ctx.world_size
        dout = dout.contiguous()
        dq = torch.empty(q.shape, dtype=torch.float32, device=q.device)  # the first step overwrites it, the others add
        grads: list[torch.Tensor | None] = [None] * (4 * world_size)
        for step in range(world_size):
            src = (rank - step) % world_size
            k, v, k_pos, k_seq = flat[4 * src:][:4]
            dk, dv = torch.empty_like(k), torch.empty_like(v)  # every step sees the whole chunk: written once, in place
            grads[4 * src], grads[4 * src + 1] = dk, dv
            ops.attention_backward_ring_block(dout, q, k, v, out, lse, dq, dk, dv, first=step == 0, mask_mode=ops.MASK_DOC,
                                              q_pos=q_pos, k_pos=k_pos, q_seq=q_seq, k_seq=k_seq)
        return (dq.to(q.dtype), None, None, None, None, *grads)


def packed_ring_attention(q: torch.Tensor, kv_chunks: Sequence[KvChunk], *, q_positions: torch.Tensor,
                          q_sequence_ids: torch.Tensor, kv_positions: Sequence[torch.Tensor],
                          kv_sequence_ids: Sequence[torch.Tensor], rank: int, world_size: int, return_lse: bool = False):
    """Rank `rank`'s attention output for packed documents: kv_chunks[r], kv_positions[r], kv_sequence_ids[r] describe
    rank r's chunk ([batch, kv_heads, s_r, head_dim] and [batch, s_r]); q_positions / q_sequence_ids are this rank's.
    Any token order inside a chunk (zigzag included) is fine: the mask is evaluated per (query, key) pair."""
    if not (len(kv_chunks) == len(kv_positions) == len(kv_sequence_ids) == world_size):
        raise ValueError(f"need K/V, positions and sequence ids for each of the {world_size} ranks")
    flat: list[torch.Tensor] = []
    for (k, v), pos, seq in zip(kv_chunks, kv_positions, kv_sequence_ids):
        flat += [k, v, pos, seq]
    out, lse = _PackedRingFunction.apply(q, q_positions, q_sequence_ids, rank, world_size, *flat)
    return (out, lse) if return_lse else out


def zigzag_ring_attention(q: torch.Tensor, kv_chunks: Sequence[KvChunk], *, rank: int, world_size: int,
                          return_lse: bool = False):
    """Rank `rank`'s attention output for its zigzag query chunk; kv_chunks[r] = (k, v) of rank r, each
    [batch, kv_heads, local_seq, head_dim] in rank r's zigzag order.  Differentiable w.r.t. q and every chunk."""
    if len(kv_chunks) != world_size:
        raise ValueError(f"need one K/V chunk per rank ({world_size}), got {len(kv_chunks)}")
    flat: list[torch.Tensor] = []
    for k, v in kv_chunks:
        flat += [k, v]
    out, lse = _ZigzagRingFunction.apply(q, rank, world_size, *flat)
    return (out, lse) if return_lse else out


class HipRingAttentionCore(nn.Module):
    """`attn_core` drop-in (q, k, v, position_offset, position_ids, sequence_ids) -> out.

    With world_size == 1 it is plain local attention, as the reference's core is
    (runtime/layers/ring_attention.py:45-54).  With world_size > 1 the caller supplies
    `kv_source(rank, k_local, v_local) -> [(k, v) for every rank]`, the seam where a transport plugs in, and for
    packed documents `meta_source(rank, positions_local, sequence_ids_local) -> [(positions, sequence_ids) ...]`.
    """

    preserves_native_gqa = True

    def __init__(self, *, rank: int = 0, world_size: int = 1,
                 kv_source: Callable[[int, torch.Tensor, torch.Tensor], Sequence[KvChunk]] | None = None,
                 meta_source: Callable[[int, torch.Tensor, torch.Tensor], Sequence[KvChunk]] | None = None,
                 attention_backend: str = AttentionBackend.HIP) -> None:
        super().__init__()
        self.attention_backend = validate_attention_backend(attention_backend)
        if world_size > 1 and kv_source is None:
            raise ValueError("HipRingAttentionCore with world_size > 1 needs a kv_source")
        self.rank, self.world_size, self.kv_source, self.meta_source = rank, world_size, kv_source, meta_source

    def forward(self, q, k, v, position_offset: int, position_ids=None, sequence_ids=None) -> torch.Tensor:
        if self.world_size == 1:
            positions = canonical_position_ids(position_ids, batch_size=q.size(0), seq_len=q.size(-2),
                                               position_offset=position_offset, device=q.device)
            sequences = canonical_sequence_ids(sequence_ids, batch_size=q.size(0), seq_len=q.size(-2), device=q.device)
            return causal_attention(q, k, v, attention_backend=self.attention_backend, warning_prefix="HipRingAttentionCore",
                                    q_positions=positions, k_positions=positions, q_sequence_ids=sequences,
                                    k_sequence_ids=sequences)
        if sequence_ids is not None:
            if self.meta_source is None:
                raise ValueError("packed-document ring attention needs a meta_source for the chunks' positions and ids")
            positions = canonical_position_ids(position_ids, batch_size=q.size(0), seq_len=q.size(-2),
                                               position_offset=position_offset, device=q.device)
            sequences = canonical_sequence_ids(sequence_ids, batch_size=q.size(0), seq_len=q.size(-2), device=q.device)
            chunks = self.kv_source(self.rank, k, v)
            meta = self.meta_source(self.rank, positions, sequences)
            return packed_ring_attention(q, chunks, q_positions=positions, q_sequence_ids=sequences,
                                         kv_positions=[m[0] for m in meta], kv_sequence_ids=[m[1] for m in meta],
                                         rank=self.rank, world_size=self.world_size)
        chunks = self.kv_source(self.rank, k, v)
        return zigzag_ring_attention(q, chunks, rank=self.rank, world_size=self.world_size)
