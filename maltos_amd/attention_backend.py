"""Attention backend router with the MI355X-native backend added.

Counterpart of the reference's utils/attention_backend.py:20-142.  `causal_attention` keeps the
reference signature; `attention_backend="hip"` (and "flash_attn", whose kernel provider this package
replaces) dispatches to the HIP kernels:
  * no positions / sequence ids  -> causal kernel (reference: SDPA is_causal=True, :60-64)
  * positions and sequence ids   -> document-mask kernel, predicate of attn_masking_utils (:103-118)
K/V may arrive with fewer heads than Q (native GQA) or already head-repeated.
The HIP route never falls back silently: an unsupported dtype/shape raises, it does not warn and
degrade.  "eager", "sdpa_auto" and "sdpa_flash" remain the plain PyTorch evaluations they are in
the reference, for callers that select them explicitly.
"""
from __future__ import annotations

from enum import Enum
from typing import Literal

import torch
import torch.nn.functional as F

from . import ops
from .attn_masking_utils import build_example_causal_mask


class AttentionBackend(str, Enum):
    EAGER = "eager"
    SDPA_AUTO = "sdpa_auto"
    SDPA_FLASH = "sdpa_flash"
    FLASH_ATTN = "flash_attn"
    HIP = "hip"

    def __str__(self) -> str:  # StrEnum behaviour on Python 3.10
        return self.value


FlashVarlenMode = Literal["same_length", "prefix"]
ATTENTION_BACKEND_CHOICES: tuple[str, ...] = tuple(b.value for b in AttentionBackend)
_HIP_BACKENDS = (AttentionBackend.HIP, AttentionBackend.FLASH_ATTN)


def validate_attention_backend(attention_backend: "str | AttentionBackend") -> AttentionBackend:
    try:
        return AttentionBackend(attention_backend)
    except ValueError:
        raise ValueError(
            f"attention_backend must be one of {sorted(ATTENTION_BACKEND_CHOICES)}, got {attention_backend!r}"
        ) from None


def uses_hip_kernels(attention_backend: str) -> bool:
    """Whether this backend name routes to the hand-written kernels (the others evaluate attention with torch ops)."""
    return validate_attention_backend(attention_backend) in _HIP_BACKENDS


def hip_fallback_reason(q: torch.Tensor) -> str | None:
    """None when the HIP kernels can take `q`, else why not (reference: flash_attn_fallback_reason,
    runtime/layers/flash_utils.py:105-115).  The router raises with this string instead of degrading."""
    if not q.is_cuda:
        return "the HIP attention kernels require GPU tensors"
    if q.dtype not in (torch.bfloat16, torch.float32):
        return f"the HIP attention kernels take bfloat16 or float32 tensors, got {q.dtype}"
    if q.size(-1) > 192:
        return f"head_dim {q.size(-1)} > 192 is not supported"
    return None


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *, attention_backend: str, warning_prefix: str,
                     q_positions: torch.Tensor | None = None, k_positions: torch.Tensor | None = None,
                     q_sequence_ids: torch.Tensor | None = None, k_sequence_ids: torch.Tensor | None = None,
                     flash_varlen_mode: FlashVarlenMode | None = None) -> torch.Tensor:
    backend = validate_attention_backend(attention_backend)
    example_aware = not (q_positions is None and k_positions is None and q_sequence_ids is None and k_sequence_ids is None)
    if example_aware and (q_positions is None or k_positions is None):
        raise ValueError("q_positions and k_positions must both be provided when using example-aware attention")

    if backend in _HIP_BACKENDS:
        reason = hip_fallback_reason(q)
        if reason is not None:
            raise RuntimeError(f"{warning_prefix}: attention_backend={backend.value!r} cannot run: {reason}")
        if not example_aware:
            return ops.attention(q, k, v, mask_mode=ops.MASK_CAUSAL)
        if (q_sequence_ids is None) != (k_sequence_ids is None):
            raise ValueError("q_sequence_ids and k_sequence_ids must both be provided or both be None")
        if q_sequence_ids is None:  # positions only: one document per row (the zero ids are kept with the positions)
            zero_ids = lambda pos: torch.zeros(pos.shape, dtype=torch.int32, device=pos.device)
            q_sequence_ids = ops.derived_from(q_positions, "_maltos_hip_zero_ids", zero_ids)
            k_sequence_ids = q_sequence_ids if k_positions is q_positions else ops.derived_from(k_positions, "_maltos_hip_zero_ids", zero_ids)
        return ops.attention(q, k, v, mask_mode=ops.MASK_DOC, q_pos=q_positions, k_pos=k_positions,
                             q_seq=q_sequence_ids, k_seq=k_sequence_ids)

    rep = q.size(1) // k.size(1)
    if rep > 1:
        k, v = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
    if not example_aware:
        if backend in (AttentionBackend.SDPA_AUTO, AttentionBackend.SDPA_FLASH):
            return F.scaled_dot_product_attention(q, k, v, is_causal=True)
        return eager_causal_attention(q, k, v)
    mask = build_example_causal_mask(q_positions=q_positions, k_positions=k_positions, q_sequence_ids=q_sequence_ids,
                                     k_sequence_ids=k_sequence_ids).unsqueeze(1)
    if backend in (AttentionBackend.SDPA_AUTO, AttentionBackend.SDPA_FLASH):
        return F.scaled_dot_product_attention(q, k, v, attn_mask=mask, is_causal=False)
    return eager_causal_attention(q, k, v, mask=mask)


def eager_causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *, mask: torch.Tensor | None = None) -> torch.Tensor:
    """Materialised-score evaluation (reference :121-135): masked scores take finfo.min, not -inf."""
    scores = (q @ k.transpose(-2, -1)) * (q.size(-1) ** -0.5)
    if mask is None:
        n = q.size(-2)
        mask = torch.ones(n, n, device=q.device, dtype=torch.bool).tril()[None, None]
    return F.softmax(scores.masked_fill(~mask, torch.finfo(scores.dtype).min), dim=-1) @ v
