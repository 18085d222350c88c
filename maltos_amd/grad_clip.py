"""Global-norm gradient clipping on the HIP kernels.

Counterpart of the reference's GradClipPlugin.on_step_phase / _global_grad_norm
(runtime/plugins/grad_clip.py:30-77) and of ZeroPluginBase._maybe_clip_local_shards
(runtime/plugins/zero_common.py:307-351): norm = sqrt(sum g^2) accumulated in fp64,
coef = max_norm / (norm + 1e-6), grads scaled only when coef < 1, FloatingPointError on a
non-finite norm.  The norm is taken on the fp32 master grads when the optimizer keeps masters
(copy_master_params() is called first, as the reference does).
"""
from __future__ import annotations

import math

import torch

from . import ops


def _grad_tensors(optimizer: torch.optim.Optimizer) -> list[torch.Tensor]:
    return [p.grad for group in optimizer.param_groups for p in group["params"] if p is not None and p.grad is not None]


def global_grad_sq_norm(optimizer: torch.optim.Optimizer) -> torch.Tensor | None:
    """Device fp64 scalar with sum g^2 over the optimizer's (master) grads; one pass when they are flat."""
    copy_master = getattr(optimizer, "copy_master_params", None)
    flat = getattr(optimizer, "flat_master_grad", None)
    if callable(copy_master):
        if flat is not None:
            copy_master(fuse_norm=True)
            fused = getattr(optimizer, "grad_sq_norm", None)
            if fused is not None:
                return fused
        else:
            copy_master()
    if flat is not None and all(p.grad is not None for g in optimizer.param_groups for p in g["params"]):
        return ops.sq_norm(flat)
    grads = _grad_tensors(optimizer)
    if not grads:
        return None
    total = torch.zeros((), dtype=torch.float64, device=grads[0].device)
    for g in grads:
        g32 = g if g.dtype == torch.float32 and g.is_contiguous() else g.to(torch.float32).contiguous()
        total += ops.sq_norm(g32.view(-1))
    return total


def clip_grad_norm_(optimizer: torch.optim.Optimizer, max_norm: float) -> float | None:
    """Clip in place, return the pre-clip global norm as a Python float (one host read, as in the reference)."""
    sq = global_grad_sq_norm(optimizer)
    if sq is None:
        return None
    global_norm = float(sq.sqrt().item())
    if not math.isfinite(global_norm):
        raise FloatingPointError("non-finite gradient norm; refusing optimizer step to avoid inf * 0 -> NaN")
    clip_coef = float(max_norm) / (global_norm + 1e-6)
    if clip_coef < 1.0:
        flat = getattr(optimizer, "flat_master_grad", None)
        if flat is not None:
            ops.scale_(flat, clip_coef)
        else:
            for g in _grad_tensors(optimizer):
                if g.dtype == torch.float32 and g.is_contiguous():
                    ops.scale_(g.view(-1), clip_coef)
                else:
                    g.mul_(clip_coef)
    return global_norm


def clip_grad_norm_fused_(optimizer: torch.optim.Optimizer, max_norm: float) -> torch.Tensor:
    """No host round trip: the fp64 sum of squares stays on the device and the AdamW kernel applies
    max_norm / (sqrt(sq) + 1e-6) to the grads it reads when that is < 1.  Returns the device scalar sum g^2
    (take .sqrt() for the norm).  Needs an optimizer whose inner optimizer is FusedAdamW.  A non-finite norm
    is not detected here; callers that want the reference's fail-fast read the returned scalar."""
    inner = getattr(optimizer, "_optimizer", optimizer)
    set_clip = getattr(inner, "set_clip", None)
    if not callable(set_clip):
        raise TypeError("clip_grad_norm_fused_ needs FusedAdamW (directly or inside MasterWeightsOptimizer)")
    sq = global_grad_sq_norm(optimizer)
    if sq is None:
        raise ValueError("no gradients to clip")
    set_clip(sq, float(max_norm))
    return sq
