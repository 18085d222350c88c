"""Causal cross-entropy on the HIP kernel (reference: utils/losses.py:9-15).

Same contract: labels are already aligned with the logits, IGNORE_INDEX rows are not supervised,
the mean is over max(1, #supervised) so a micro-batch without targets yields exactly 0 with zero
gradients.  Difference, on purpose: the loss is returned as an fp32 scalar even for bf16 logits
(the reference's F.cross_entropy(reduction="sum") rounds the SUM to bf16, a relative error of up
to 2^-9); `.to(logits.dtype)` reproduces the reference's dtype.
"""
from __future__ import annotations

import torch

from . import ops
from .constants import IGNORE_INDEX


def causal_cross_entropy(logits: torch.Tensor, labels: torch.Tensor, *, overwrite_logits: bool = False) -> torch.Tensor:
    """overwrite_logits: the caller owns the logits and never reads them again; their gradient then replaces them in
    the same buffer (no second logits-sized tensor, and the kernel streams faster over one buffer than over two)."""
    return ops.cross_entropy(logits, labels, IGNORE_INDEX, overwrite_logits=overwrite_logits)
