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


def causal_cross_entropy(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    return ops.cross_entropy(logits, labels, IGNORE_INDEX)
