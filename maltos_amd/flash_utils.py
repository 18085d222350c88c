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
    device = q.device

    def run_ids_and_index(sequence_ids):  # int32, what the kernels take; formed once per id tensor, not once per layer
        ids = sequence_ids.to(device)
        valid = ids != PAD_SEQUENCE_ID
        left_valid = torch.roll(valid, 1, dims=1)
        left_valid[:, 0] = False
        starts = valid & (~left_valid | (ids != torch.roll(ids, 1, dims=1)))
        run_ids = torch.where(valid, starts.long().cumsum(dim=1) - 1, torch.full_like(ids, PAD_SEQUENCE_ID, dtype=torch.long))
        index = torch.arange(ids.size(1), device=device, dtype=torch.int32).unsqueeze(0).expand_as(ids)
        return run_ids.to(torch.int32), index.contiguous()

    run_ids, index = ops.derived_from(sequence_ids, f"_maltos_hip_run_ids_{device}", run_ids_and_index)
    return ops.attention(q, k, v, mask_mode=ops.MASK_DOC, q_pos=index, k_pos=index, q_seq=run_ids, k_seq=run_ids)


# --------------------------------------------------------------------------------------------
# "prefix" function set: queries of one chunk against the keys of another (or a gathered) chunk
# --------------------------------------------------------------------------------------------
@dataclass(frozen=True)
class VarlenPrefixMetadata:
    """Index layout of one (query chunk, key chunk) pair (reference: flash_utils.py:49-57)."""

    q_indices: torch.Tensor
    k_indices: torch.Tensor
    cu_seqlens_q: torch.Tensor
    cu_seqlens_k: torch.Tensor
    max_seqlen_q: int
    max_seqlen_k: int


def _prefix_ids(q, k, v, q_positions, k_positions, q_sequence_ids, k_sequence_ids):
    """Shape checks of the reference's packer (flash_utils.py:577-621), same messages; missing ids mean one document."""
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("pack_varlen_prefix_qkv expects q, k, v to have shape [batch, heads, seq, dim]")
    if q_positions.dim() != 2 or k_positions.dim() != 2:
        raise ValueError("q_positions and k_positions must have shape [batch, seq]")
    batch_size, q_num_heads, q_seq_len, head_dim = q.shape
    k_batch_size, k_num_heads, k_seq_len, k_head_dim = k.shape
    if k_batch_size != batch_size or k_head_dim != head_dim or k.shape != v.shape:
        raise ValueError("q and k/v must agree on batch/head_dim and K/V shape, "
                         f"got q={tuple(q.shape)} k={tuple(k.shape)} v={tuple(v.shape)}")
    if q_num_heads % k_num_heads:
        raise ValueError("FlashAttention GQA requires query heads divisible by native KV heads, "
                         f"got {q_num_heads} and {k_num_heads}")
    if q_positions.shape != (batch_size, q_seq_len):
        raise ValueError("q_positions shape must match q batch+seq dimensions, "
                         f"got {tuple(q_positions.shape)} vs ({batch_size}, {q_seq_len})")
    if k_positions.shape != (batch_size, k_seq_len):
        raise ValueError("k_positions shape must match k/v batch+seq dimensions, "
                         f"got {tuple(k_positions.shape)} vs ({batch_size}, {k_seq_len})")
    if q_sequence_ids is None:
        q_sequence_ids = torch.zeros_like(q_positions)
    elif q_sequence_ids.shape != (batch_size, q_seq_len):
        raise ValueError("q_sequence_ids shape must match q batch+seq dimensions, "
                         f"got {tuple(q_sequence_ids.shape)} vs ({batch_size}, {q_seq_len})")
    if k_sequence_ids is None:
        k_sequence_ids = torch.zeros_like(k_positions)
    elif k_sequence_ids.shape != (batch_size, k_seq_len):
        raise ValueError("k_sequence_ids shape must match k/v batch+seq dimensions, "
                         f"got {tuple(k_sequence_ids.shape)} vs ({batch_size}, {k_seq_len})")
    return q_sequence_ids, k_sequence_ids


def varlen_prefix_metadata(*, q_positions: torch.Tensor, k_positions: torch.Tensor,
                           q_sequence_ids: torch.Tensor | None = None, k_sequence_ids: torch.Tensor | None = None,
                           allow_empty_kv: bool = False) -> VarlenPrefixMetadata:
    """The index layout the reference's `pack_varlen_prefix_qkv` builds (flash_utils.py:622-724), from tensor
    operations instead of its per-token host loop: a query run is a maximal stretch of valid tokens of one row with
    one sequence id and positions rising by one; its keys are the row's valid keys of that id at positions up to the
    run's last one, in storage order.  Runs without keys are dropped (`allow_empty_kv`) or raise.  The HIP kernels
    do not need this layout; it is what a varlen caller (or a cache keyed like the reference's) consumes."""
    if q_sequence_ids is None:
        q_sequence_ids = torch.zeros_like(q_positions)
    if k_sequence_ids is None:
        k_sequence_ids = torch.zeros_like(k_positions)
    device = q_positions.device
    batch, q_len = q_positions.shape
    k_len = k_positions.size(1)
    q_valid = q_sequence_ids != PAD_SEQUENCE_ID
    k_valid = k_sequence_ids != PAD_SEQUENCE_ID
    # valid query tokens in (row, index) order; a run starts where the row, the id or the +1 position chain breaks
    tok = torch.nonzero(q_valid.reshape(-1), as_tuple=False).flatten()
    if tok.numel() == 0:
        zero = torch.zeros(1, dtype=torch.int32, device=device)
        empty = torch.zeros(0, dtype=torch.long, device=device)
        return VarlenPrefixMetadata(empty, empty, zero, zero.clone(), 0, 0)
    row = tok // q_len
    seq = q_sequence_ids.reshape(-1)[tok]
    pos = q_positions.reshape(-1)[tok]
    brk = torch.ones_like(tok, dtype=torch.bool)
    brk[1:] = (row[1:] != row[:-1]) | (seq[1:] != seq[:-1]) | (pos[1:] != pos[:-1] + 1)
    run_of_tok = brk.long().cumsum(0) - 1
    first = torch.nonzero(brk, as_tuple=False).flatten()
    last = torch.cat([first[1:] - 1, first.new_tensor([tok.numel() - 1])])
    run_row, run_seq, run_end = row[first], seq[first], pos[last]
    # [runs, k_len] visibility of the run's row
    key_ok = (k_valid[run_row] & (k_sequence_ids[run_row] == run_seq.unsqueeze(1))
              & (k_positions[run_row] <= run_end.unsqueeze(1)))
    k_count = key_ok.sum(dim=1)
    keep = k_count > 0
    if not bool(keep.all()):
        if not allow_empty_kv:
            bad = int(torch.nonzero(~keep, as_tuple=False)[0])
            raise ValueError("pack_varlen_prefix_qkv found a query run without any matching key/value prefix; "
                             f"batch={int(run_row[bad])} sequence_id={int(run_seq[bad])} end_position={int(run_end[bad])}")
    q_indices = tok[keep[run_of_tok]]
    run_idx, key_idx = torch.nonzero(key_ok & keep.unsqueeze(1), as_tuple=True)
    k_indices = run_row[run_idx] * k_len + key_idx
    q_count = (last - first + 1)[keep]
    k_count = k_count[keep]
    cu_q = torch.zeros(q_count.numel() + 1, dtype=torch.int32, device=device)
    cu_k = torch.zeros(k_count.numel() + 1, dtype=torch.int32, device=device)
    if q_count.numel():
        cu_q[1:] = q_count.cumsum(0)
        cu_k[1:] = k_count.cumsum(0)
    return VarlenPrefixMetadata(q_indices=q_indices, k_indices=k_indices, cu_seqlens_q=cu_q, cu_seqlens_k=cu_k,
                                max_seqlen_q=int(q_count.max()) if q_count.numel() else 0,
                                max_seqlen_k=int(k_count.max()) if k_count.numel() else 0)


def _raise_on_empty_prefix(lse: torch.Tensor, q_sequence_ids: torch.Tensor) -> None:
    """`allow_empty_kv=False` of the reference (flash_utils.py:677-684) costs one device-to-host flag here: a valid
    query whose LSE is -inf saw no key.  The read stalls the stream, so it is left out while the stream is being
    captured into a HIP graph (a replay could not raise anyway): such callers pass `allow_empty_kv=True`."""
    if lse.is_cuda and torch.cuda.is_current_stream_capturing():
        return
    unseen = torch.isinf(lse).all(dim=1) & (q_sequence_ids != PAD_SEQUENCE_ID)
    if bool(unseen.any()):
        b, s = (int(x) for x in torch.nonzero(unseen, as_tuple=False)[0])
        raise ValueError("pack_varlen_prefix_qkv found a query run without any matching key/value prefix; "
                         f"batch={b} sequence_id={int(q_sequence_ids[b, s])} query_index={s}")


def flash_attn_varlen_prefix_with_lse(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *, q_positions: torch.Tensor,
                                      k_positions: torch.Tensor, q_sequence_ids: torch.Tensor | None = None,
                                      k_sequence_ids: torch.Tensor | None = None, allow_empty_kv: bool = False,
                                      metadata: VarlenPrefixMetadata | None = None, metadata_cache: dict | None = None,
                                      metadata_cache_key: object | None = None) -> FlashAttnBlockOutput:
    """One (query chunk, key chunk) block without autograd (reference :772-860): query i sees key j iff both are
    valid, carry the same sequence id and k_position <= q_position.  That is the rule the reference's own test pins
    for this function (tests/sequence_ids_attention_mask.py:223-246) and what its run / key-prefix packing computes
    whenever a run's keys end with the run's own positions.  Queries that see no key give zeros and LSE = -inf, as
    the reference's empty-prefix branch does (:810-819); with `allow_empty_kv=False` they raise instead.

    The masks are evaluated on the device from the id tensors: no packing, no gather/scatter, no host reads of the
    ids, which is why `metadata` and the cache arguments are accepted and left unused."""
    del metadata, metadata_cache, metadata_cache_key
    q_seq, k_seq = _prefix_ids(q, k, v, q_positions, k_positions, q_sequence_ids, k_sequence_ids)
    out, lse = ops.attention_forward(q, k, v, mask_mode=ops.MASK_DOC, q_pos=q_positions, k_pos=k_positions, q_seq=q_seq,
                                     k_seq=k_seq)
    if not allow_empty_kv:
        _raise_on_empty_prefix(lse, q_seq)
    return FlashAttnBlockOutput(out=out, lse=lse)


def flash_attn_varlen_prefix_backward(dout: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                                      out: torch.Tensor, softmax_lse: torch.Tensor, *, q_positions: torch.Tensor,
                                      k_positions: torch.Tensor, q_sequence_ids: torch.Tensor | None = None,
                                      k_sequence_ids: torch.Tensor | None = None, allow_empty_kv: bool = False,
                                      metadata: VarlenPrefixMetadata | None = None, metadata_cache: dict | None = None,
                                      metadata_cache_key: object | None = None
                                      ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dq, dk, dv) of one block from caller-supplied out / LSE, which may be a ring's merged ones (reference
    :863-962).  Tokens outside every visible pair receive zeros, as the reference's scatter leaves them.

    `allow_empty_kv=False` differs from the reference here: its packer raises from this block's metadata when a query
    run has no key in THIS chunk; this function only sees the LSE it is handed and raises when that says a valid query
    saw no key at all, which a merged LSE says only if no chunk held one.  The block's own forward
    (`flash_attn_varlen_prefix_with_lse`), which every schedule runs first, makes the per-block check."""
    del metadata, metadata_cache, metadata_cache_key
    q_seq, k_seq = _prefix_ids(q, k, v, q_positions, k_positions, q_sequence_ids, k_sequence_ids)
    if not allow_empty_kv:
        _raise_on_empty_prefix(softmax_lse, q_seq)
    return ops.attention_backward(dout, q, k, v, out, softmax_lse, mask_mode=ops.MASK_DOC, q_pos=q_positions,
                                  k_pos=k_positions, q_seq=q_seq, k_seq=k_seq)


def flash_attn_varlen_prefix(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *, q_positions: torch.Tensor,
                             k_positions: torch.Tensor, q_sequence_ids: torch.Tensor | None = None,
                             k_sequence_ids: torch.Tensor | None = None) -> torch.Tensor:
    """Differentiable form the backend router calls for `flash_varlen_mode="prefix"` (reference :727-769,
    utils/attention_backend.py:84-94); raises on a query run without keys like the reference's packer."""
    q_seq, k_seq = _prefix_ids(q, k, v, q_positions, k_positions, q_sequence_ids, k_sequence_ids)
    out, lse = ops.attention(q, k, v, mask_mode=ops.MASK_DOC, q_pos=q_positions, k_pos=k_positions, q_seq=q_seq,
                             k_seq=k_seq, return_lse=True)
    _raise_on_empty_prefix(lse.detach(), q_seq)
    return out
