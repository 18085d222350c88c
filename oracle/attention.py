"""Oracle: masks, eager/dense attention with LSE, explicit backward, LSE merge, zigzag ring schedule."""
from __future__ import annotations

import torch

PAD_SEQUENCE_ID = -1  # utils/constants.py:4


# ---- runtime/layers/attn_masking_utils.py:6-51 ------------------------------------------------
def canonical_ids(ids: torch.Tensor | None, *, batch_size: int, seq_len: int, position_offset: int | None,
                  device) -> torch.Tensor | None:
    """[B, S] int64 ids; `position_offset` not None means "positions" (arange default), None means sequence ids."""
    if ids is None:
        if position_offset is None:
            return None
        pos = torch.arange(position_offset, position_offset + seq_len, device=device, dtype=torch.long)
        return pos.unsqueeze(0).expand(batch_size, -1).contiguous()
    if ids.dim() == 1:
        if ids.numel() != seq_len:
            raise ValueError(f"ids length must match seq_len, got {ids.numel()} vs {seq_len}")
        return ids.to(device=device, dtype=torch.long).unsqueeze(0).expand(batch_size, -1).contiguous()
    if ids.dim() == 2:
        if ids.size(0) != batch_size or ids.size(1) != seq_len:
            raise ValueError(f"ids shape must match [batch, seq], got {tuple(ids.shape)}")
        return ids.to(device=device, dtype=torch.long).contiguous()
    raise ValueError(f"ids must have rank 1 or 2, got shape={tuple(ids.shape)}")


# ---- runtime/layers/attn_masking_utils.py:54-87 -----------------------------------------------
def example_causal_mask(q_pos, k_pos, q_seq=None, k_seq=None) -> torch.Tensor:
    """bool [B, Sq, Sk]: k_pos <= q_pos, and same sequence id when ids are given."""
    mask = k_pos.unsqueeze(1) <= q_pos.unsqueeze(2)
    if q_seq is None and k_seq is None:
        return mask
    if q_seq is None or k_seq is None:
        raise ValueError("q_sequence_ids and k_sequence_ids must both be provided or both be None")
    return mask & (q_seq.unsqueeze(2) == k_seq.unsqueeze(1))


# ---- models/llama.py:97-100 ------------------------------------------------------------------
def repeat_kv(x: torch.Tensor, repeats: int) -> torch.Tensor:
    return x if repeats == 1 else x.repeat_interleave(repeats, dim=1)


# ---- utils/attention_backend.py:121-135 (eager) with -inf masking and LSE ---------------------
def attention_with_lse(q, k, v, mask: torch.Tensor | None = None, *, scale: float | None = None):
    """softmax(scale q k^T + mask) v and natural-log LSE [B, H, Sq], all in the input dtype's fp32 upcast.

    `mask` is bool broadcastable to [B, H, Sq, Sk] (True = visible).  Fully masked rows give 0 and
    lse = -inf (the flash-attn convention the ring merge relies on, runtime/layers/flash_utils.py:810-819).
    GQA: k/v may have fewer heads (repeat_interleave, models/llama.py:97-100).
    """
    qf, kf, vf = q.float(), k.float(), v.float()
    rep = qf.size(1) // kf.size(1)
    kf, vf = repeat_kv(kf, rep), repeat_kv(vf, rep)
    scale = q.size(-1) ** -0.5 if scale is None else scale
    scores = torch.matmul(qf, kf.transpose(-2, -1)) * scale
    if mask is not None:
        scores = scores.masked_fill(~mask, float("-inf"))
    lse = torch.logsumexp(scores, dim=-1)
    safe = torch.where(torch.isfinite(lse), lse, torch.zeros_like(lse))
    probs = torch.exp(scores - safe.unsqueeze(-1))
    probs = torch.where(torch.isfinite(scores), probs, torch.zeros_like(probs))
    return torch.matmul(probs, vf), lse


def causal_mask(sq: int, sk: int, device) -> torch.Tensor:
    """Bottom-right aligned causal mask [1, 1, sq, sk]; square case is torch.tril (attention_backend.py:131-132)."""
    i = torch.arange(sq, device=device).unsqueeze(1)
    j = torch.arange(sk, device=device).unsqueeze(0)
    return (j <= i + (sk - sq)).view(1, 1, sq, sk)


def doc_mask(q_pos, k_pos, q_seq, k_seq) -> torch.Tensor:
    """[B, 1, Sq, Sk] document mask; padded queries (seq id -1) see nothing, the flash-varlen behaviour
    (runtime/layers/flash_utils.py:408-418) that the HIP backend keeps."""
    m = example_causal_mask(q_pos, k_pos, q_seq, k_seq)
    m = m & (q_seq.unsqueeze(2) != PAD_SEQUENCE_ID)
    return m.unsqueeze(1)


# ---- FlashAttention-2 recompute backward (what flash_attn_dense_backward computes,
#      runtime/layers/flash_utils.py:218-263); valid with a GLOBAL out/lse -------------------------
def attention_backward_explicit(dout, q, k, v, out, lse, mask=None, *, scale: float | None = None):
    """P = exp(S - LSE); dV = P^T dO; dP = dO V^T; delta = rowsum(dO * O); dS = P (dP - delta);
    dQ = scale dS K; dK = scale dS^T Q.  GQA grads are summed over each KV head's query group."""
    qf, kf, vf, do, of = q.float(), k.float(), v.float(), dout.float(), out.float()
    hq, hkv = qf.size(1), kf.size(1)
    rep = hq // hkv
    kr, vr = repeat_kv(kf, rep), repeat_kv(vf, rep)
    scale = q.size(-1) ** -0.5 if scale is None else scale
    s = torch.matmul(qf, kr.transpose(-2, -1)) * scale
    if mask is not None:
        s = s.masked_fill(~mask, float("-inf"))
    lse_f = lse.float()
    p = torch.exp(s - torch.where(torch.isfinite(lse_f), lse_f, torch.full_like(lse_f, float("inf"))).unsqueeze(-1))
    p = torch.where(torch.isfinite(s), p, torch.zeros_like(p))
    dv = torch.matmul(p.transpose(-2, -1), do)
    dp = torch.matmul(do, vr.transpose(-2, -1))
    delta = (do * of).sum(dim=-1, keepdim=True)
    ds = p * (dp - delta)
    dq = torch.matmul(ds, kr) * scale
    dk = torch.matmul(ds.transpose(-2, -1), qf) * scale
    if rep > 1:
        b, _, sk, d = dk.shape
        dk = dk.view(b, hkv, rep, sk, d).sum(dim=2)
        dv = dv.view(b, hkv, rep, sk, d).sum(dim=2)
    return dq, dk, dv


# ---- runtime/layers/functional.py:717-748 -----------------------------------------------------
def exp_delta_or_zero(source: torch.Tensor, target: torch.Tensor) -> torch.Tensor:
    out = torch.zeros_like(target)
    finite = torch.isfinite(source)
    if finite.any():
        out[finite] = torch.exp(source[finite] - target[finite])
    return out


def merge_attention_blocks(running_out, running_lse, block_out, block_lse, *, q_slice: slice | None = None):
    """Log-sum-exp merge; with q_slice only those rows of the running state are updated (in place)."""
    if q_slice is not None:
        cur_out, cur_lse = running_out[:, :, q_slice, :], running_lse[:, :, q_slice]
        new_lse = torch.logaddexp(cur_lse, block_lse)
        prev = exp_delta_or_zero(cur_lse, new_lse)
        blk = exp_delta_or_zero(block_lse, new_lse)
        running_out[:, :, q_slice, :] = cur_out * prev.unsqueeze(-1) + block_out.float() * blk.unsqueeze(-1)
        running_lse[:, :, q_slice] = new_lse
        return running_out, running_lse
    new_lse = torch.logaddexp(running_lse, block_lse)
    prev = exp_delta_or_zero(running_lse, new_lse)
    blk = exp_delta_or_zero(block_lse, new_lse)
    return running_out * prev.unsqueeze(-1) + block_out.float() * blk.unsqueeze(-1), new_lse


# ---- runtime/layers/ring_layout.py:6-23, parallel/context_token_planner.py:78-103 --------------
def zigzag_positions(local_seq_len: int, *, rank: int, world_size: int, device="cpu") -> torch.Tensor:
    if local_seq_len % 2 != 0:
        raise ValueError(f"zigzag ring attention requires an even local sequence length, got {local_seq_len}")
    half = local_seq_len // 2
    front = torch.arange(rank * half, rank * half + half, device=device, dtype=torch.long)
    back0 = (2 * world_size - rank - 1) * half
    back = torch.arange(back0, back0 + half, device=device, dtype=torch.long)
    return torch.cat([front, back], dim=0)


def zigzag_schedule(rank: int, world_size: int) -> list[tuple[int, str]]:
    """[(source_rank, kind)] per ring step; kind in {"causal", "front_kv", "tail_q"}
    (runtime/layers/functional.py:1031-1061; KV held at step s comes from rank (rank - s) mod W)."""
    steps = []
    for step in range(world_size):
        src = (rank - step) % world_size
        kind = "causal" if step == 0 else ("front_kv" if step <= rank else "tail_q")
        steps.append((src, kind))
    return steps


def dense_block(q, k, v, *, causal: bool):
    """The dense stand-in for flash_attn_dense_with_lse (tests/sequence_ids_attention_mask.py:196-206)."""
    mask = causal_mask(q.size(-2), k.size(-2), q.device) if causal else None
    return attention_with_lse(q, k, v, mask)


# ---- runtime/layers/functional.py:1012-1065 ---------------------------------------------------
def zigzag_ring_forward(q, kv_chunks, *, rank: int, world_size: int, block_fn=dense_block):
    """One rank's forward: q [B,H,S_loc,D]; kv_chunks[r] = (k, v) of rank r.  Returns (out fp32->v.dtype, lse)."""
    s_loc = q.size(-2)
    half = s_loc // 2
    running_out = torch.zeros(q.shape, dtype=torch.float32, device=q.device)
    running_lse = torch.full(q.shape[:-1], float("-inf"), dtype=torch.float32, device=q.device)
    calls = []
    for src, kind in zigzag_schedule(rank, world_size):
        k, v = kv_chunks[src]
        if kind == "causal":
            o, l = block_fn(q, k, v, causal=True)
            calls.append((s_loc, k.size(-2), True))
            running_out, running_lse = merge_attention_blocks(running_out, running_lse, o, l)
        elif kind == "front_kv":
            o, l = block_fn(q, k[:, :, :half], v[:, :, :half], causal=False)
            calls.append((s_loc, half, False))
            running_out, running_lse = merge_attention_blocks(running_out, running_lse, o, l)
        else:
            o, l = block_fn(q[:, :, half:], k, v, causal=False)
            calls.append((half, k.size(-2), False))
            running_out, running_lse = merge_attention_blocks(running_out, running_lse, o, l, q_slice=slice(half, None))
    return running_out.to(kv_chunks[rank][1].dtype), running_lse, calls


# ---- runtime/layers/functional.py:1068-1166 ---------------------------------------------------
def zigzag_ring_backward(dout, q, kv_chunks, out, lse, *, rank: int, world_size: int):
    """dq (fp32) for this rank's queries and this rank's contribution to every chunk's dk/dv (fp32),
    using the global out/lse in each block call."""
    s_loc = q.size(-2)
    half = s_loc // 2
    dq = torch.zeros(q.shape, dtype=torch.float32, device=q.device)
    dkv = {}
    for src, kind in zigzag_schedule(rank, world_size):
        k, v = kv_chunks[src]
        dk = torch.zeros(k.shape, dtype=torch.float32, device=q.device)
        dv = torch.zeros(v.shape, dtype=torch.float32, device=q.device)
        if kind == "causal":
            bdq, bdk, bdv = attention_backward_explicit(dout, q, k, v, out, lse, causal_mask(s_loc, s_loc, q.device))
            dq += bdq
            dk += bdk
            dv += bdv
        elif kind == "front_kv":
            bdq, bdk, bdv = attention_backward_explicit(dout, q, k[:, :, :half], v[:, :, :half], out, lse)
            dq += bdq
            dk[:, :, :half] += bdk
            dv[:, :, :half] += bdv
        else:
            bdq, bdk, bdv = attention_backward_explicit(dout[:, :, half:], q[:, :, half:], k, v, out[:, :, half:],
                                                        lse[:, :, half:])
            dq[:, :, half:] += bdq
            dk += bdk
            dv += bdv
        dkv[src] = (dk, dv)
    return dq, dkv


# ---- runtime/layers/functional.py:823-897 -------------------------------------------------------
def packed_ring_forward(q, kv_chunks, q_pos, q_seq, meta_chunks, *, rank: int, world_size: int):
    """One rank's forward for packed documents: at ring step s the K/V chunk of rank (rank - s) mod W arrives with
    its positions and sequence ids; a query sees the keys of its own document with k_pos <= q_pos (the varlen
    prefix blocks of flash_utils.py:566-962 select exactly those); blocks with no visible key merge as (0, -inf).
    kv_chunks[r] = (k, v), meta_chunks[r] = (positions, sequence_ids) of rank r."""
    running_out = torch.zeros(q.shape, dtype=torch.float32, device=q.device)
    running_lse = torch.full(q.shape[:-1], float("-inf"), dtype=torch.float32, device=q.device)
    for step in range(world_size):
        src = (rank - step) % world_size
        k, v = kv_chunks[src]
        k_pos, k_seq = meta_chunks[src]
        o, l = attention_with_lse(q, k, v, doc_mask(q_pos, k_pos, q_seq, k_seq))
        running_out, running_lse = merge_attention_blocks(running_out, running_lse, o, l)
    return running_out.to(kv_chunks[rank][1].dtype), running_lse


# ---- runtime/layers/functional.py:900-1009 ------------------------------------------------------
def packed_ring_backward(dout, q, kv_chunks, q_pos, q_seq, meta_chunks, out, lse, *, rank: int, world_size: int):
    """dq (fp32) and this rank's contribution to every chunk's dk/dv (fp32), global out/lse in each block."""
    dq = torch.zeros(q.shape, dtype=torch.float32, device=q.device)
    dkv = {}
    for step in range(world_size):
        src = (rank - step) % world_size
        k, v = kv_chunks[src]
        k_pos, k_seq = meta_chunks[src]
        bdq, bdk, bdv = attention_backward_explicit(dout, q, k, v, out, lse, doc_mask(q_pos, k_pos, q_seq, k_seq))
        dq += bdq
        dkv[src] = (bdk.float(), bdv.float())
    return dq, dkv


# ---- runtime/layers/ring_attention.py:221-258 (eager online softmax, single step form) ----------
def online_softmax_update(q, k, v, mask, running_max, running_sum, running_acc, *, scale: float | None = None):
    """(running_max, running_sum, running_acc) update in fp32; final output is acc / sum.clamp_min(1e-20)."""
    scale = q.size(-1) ** -0.5 if scale is None else scale
    scores = torch.matmul(q.float(), k.float().transpose(-2, -1)) * scale
    scores = scores.masked_fill(~mask, float("-inf"))
    block_max = scores.max(dim=-1).values
    new_max = torch.maximum(running_max, block_max)
    safe = torch.where(torch.isfinite(new_max), new_max, torch.zeros_like(new_max))
    prev = torch.where(torch.isfinite(running_max), torch.exp(running_max - safe), torch.zeros_like(running_max))
    p = torch.exp(scores - safe.unsqueeze(-1))
    p = torch.where(torch.isfinite(scores), p, torch.zeros_like(p))
    return new_max, running_sum * prev + p.sum(-1), running_acc * prev.unsqueeze(-1) + torch.matmul(p, v.float())


# ---- runtime/layers/flash_utils.py:356-405 ----------------------------------------------------
def varlen_metadata(sequence_ids: torch.Tensor):
    """(cu_seqlens int32, max_seqlen, token_mask): segments are maximal runs of equal non-pad ids per row."""
    valid = sequence_ids != PAD_SEQUENCE_ID
    lengths = []
    for row, vrow in zip(sequence_ids.tolist(), valid.tolist()):
        run, prev = 0, None
        for sid, ok in zip(row, vrow):
            if not ok:
                if run:
                    lengths.append(run)
                run, prev = 0, None
                continue
            if prev is not None and sid != prev:
                lengths.append(run)
                run = 0
            run += 1
            prev = sid
        if run:
            lengths.append(run)
    cu = torch.zeros(len(lengths) + 1, dtype=torch.int32)
    if lengths:
        cu[1:] = torch.tensor(lengths, dtype=torch.int32).cumsum(0)
    return cu, (max(lengths) if lengths else 0), valid
