"""Kernel-shaped attention functions backed by the HIP kernels.

The reference's ring / context-parallel code calls a small set of functions it expects from its
flash-attention provider (runtime/layers/flash_utils.py): dense forward with LSE, dense backward
with caller-supplied out/LSE, varlen forward, and `*_fallback_reason` probes.  This module offers
the same names and return conventions on top of libmaltos_hip, without the layout transposes the
reference wrapper performs (the kernels consume [B, H, S, D] views of [B, S, H, D] storage as is)
and without head-repeating K/V.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from . import ops
from .attention_backend import hip_fallback_reason
from .constants import PAD_SEQUENCE_ID


@dataclass(frozen=True)
class FlashAttnBlockOutput:
    out: torch.Tensor
    lse: torch.Tensor  # float32 [batch, heads, seq], natural log


@dataclass(frozen=True)
class VarlenQkvMetadata:
    """Document layout of one packed micro-batch (reference: flash_utils.py:38-46)."""

    source_version: int
    token_mask: torch.Tensor
    cu_seqlens: torch.Tensor
    max_seqlen: int


def flash_attn_is_available() -> bool:
    try:
        from . import _lib

        _lib.lib()
    except Exception:
        return False
    return torch.cuda.is_available()


def flash_attn_fallback_reason(q: torch.Tensor) -> str | None:
    return hip_fallback_reason(q)


flash_attn_block_fallback_reason = flash_attn_fallback_reason
flash_attn_dense_block_fallback_reason = flash_attn_fallback_reason


def flash_attn_dense(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """Differentiable causal attention (reference :266-276)."""
    return ops.attention(q, k, v, mask_mode=ops.MASK_CAUSAL)


def flash_attn_dense_with_lse(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *, causal: bool) -> FlashAttnBlockOutput:
    """Block forward without autograd, scale head_dim^-0.5 (reference :180-215)."""
    out, lse = ops.attention_forward(q, k, v, mask_mode=ops.MASK_CAUSAL if causal else ops.MASK_NONE)
    return FlashAttnBlockOutput(out=out, lse=lse)


def flash_attn_dense_backward(dout: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor,
                              softmax_lse: torch.Tensor, *, causal: bool) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dq, dk, dv) from caller-supplied out / LSE, which may be a ring's global ones (reference :218-263)."""
    return ops.attention_backward(dout, q, k, v, out, softmax_lse, mask_mode=ops.MASK_CAUSAL if causal else ops.MASK_NONE)


def varlen_qkv_metadata(sequence_ids: torch.Tensor) -> VarlenQkvMetadata:
    """cu_seqlens / max_seqlen / token mask of a [batch, seq] id tensor: a document is a maximal run of
    equal non-padding ids inside one row.  Cached on the tensor and invalidated by in-place edits
    through the tensor's version counter (reference :356-405).  The HIP kernels do not need it (they
    mask from the ids directly); it is what a varlen caller or a data pipeline would consume."""
    cache_attr = "_maltos_hip_varlen_metadata"
    version = sequence_ids._version
    cached = getattr(sequence_ids, cache_attr, None)
    if isinstance(cached, VarlenQkvMetadata) and cached.source_version == version:
        return cached
    ids = sequence_ids.detach()
    if ids.dim() != 2:
        raise ValueError(f"sequence_ids must have shape [batch, seq], got {tuple(ids.shape)}")
    valid = ids != PAD_SEQUENCE_ID
    # a run starts at a valid token whose left neighbour (in the same row) is absent, padding or another id
    left_ids = torch.roll(ids, 1, dims=1)
    left_valid = torch.roll(valid, 1, dims=1)
    left_valid[:, 0] = False
    starts = valid & (~left_valid | (ids != left_ids))
    flat_valid = valid.reshape(-1)
    start_idx = torch.nonzero(starts.reshape(-1)[flat_valid], as_tuple=False).flatten()
    total = int(flat_valid.sum().item())
    bounds = torch.cat([start_idx, start_idx.new_tensor([total])]) if total else start_idx.new_zeros(1)
    cu_seqlens = bounds.to(torch.int32)
    max_seqlen = int((bounds[1:] - bounds[:-1]).max().item()) if total else 0
    meta = VarlenQkvMetadata(source_version=version, token_mask=valid, cu_seqlens=cu_seqlens, max_seqlen=max_seqlen)
    setattr(sequence_ids, cache_attr, meta)
    return meta


def flash_attn_varlen(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, sequence_ids: torch.Tensor) -> torch.Tensor:
    """Packed-document causal attention (reference :493-520): causal inside each run of equal ids, nothing
    across runs, zeros at padding.  Runs directly on the padded [B, H, S, D] tensors: no gather/scatter."""
    if sequence_ids.dim() != 2 or sequence_ids.shape != (q.size(0), q.size(2)):
        raise ValueError(f"sequence_ids shape must match q/k/v batch+seq dimensions, got {tuple(sequence_ids.shape)}")
    ids = sequence_ids.to(q.device)
    valid = ids != PAD_SEQUENCE_ID
    left_valid = torch.roll(valid, 1, dims=1)
    left_valid[:, 0] = False
    starts = valid & (~left_valid | (ids != torch.roll(ids, 1, dims=1)))
    run_ids = torch.where(valid, starts.long().cumsum(dim=1) - 1, torch.full_like(ids, PAD_SEQUENCE_ID))
    index = torch.arange(ids.size(1), device=ids.device, dtype=torch.long).unsqueeze(0).expand_as(ids)
    return ops.attention(q, k, v, mask_mode=ops.MASK_DOC, q_pos=index, k_pos=index, q_seq=run_ids, k_seq=run_ids)
