"""Oracle: AdamW closed form, global-norm clip, master-weights semantics, ZeRO flat-buffer layout."""
from __future__ import annotations

import math

import torch


# ---- torch.optim.AdamW as built by train/cli.py:432-441 (amsgrad=False, maximize=False) ---------
def adamw_reference_step(p, g, m, v, *, lr, beta1, beta2, eps, weight_decay, step: int):
    """Returns updated (p, m, v); textbook decoupled weight decay with bias correction."""
    p = p * (1.0 - lr * weight_decay)
    m = beta1 * m + (1.0 - beta1) * g
    v = beta2 * v + (1.0 - beta2) * g * g
    bc1 = 1.0 - beta1 ** step
    bc2 = 1.0 - beta2 ** step
    denom = v.sqrt() / math.sqrt(bc2) + eps
    return p - (lr / bc1) * m / denom, m, v


# ---- runtime/plugins/grad_clip.py:54-77, runtime/plugins/zero_common.py:324-350 -----------------
def global_grad_norm(grads) -> float:
    sq = torch.zeros((), dtype=torch.float64)
    for g in grads:
        sq = sq + g.detach().double().pow(2).sum().cpu()
    return float(sq.sqrt().item())


def clip_coefficient(global_norm: float, max_norm: float) -> float:
    """The reference scales grads by this only when it is < 1."""
    if not math.isfinite(global_norm):
        raise FloatingPointError("non-finite gradient norm")
    return float(max_norm) / (global_norm + 1e-6)


def clip_grads_(grads, max_norm: float) -> float:
    norm = global_grad_norm(grads)
    coef = clip_coefficient(norm, max_norm)
    if coef < 1.0:
        for g in grads:
            g.mul_(coef)
    return norm


# ---- runtime/optim.py:10-104 -----------------------------------------------------------------
def master_weights_step(model_params, master_params, inner_optimizer) -> None:
    """grad upcast -> inner step on fp32 masters -> low-precision write-back (optim.py:43-71)."""
    for mp, ms in zip(model_params, master_params):
        ms.grad = None if mp.grad is None else mp.grad.detach().to(dtype=ms.dtype).clone()
    inner_optimizer.step()
    with torch.no_grad():
        for mp, ms in zip(model_params, master_params):
            mp.copy_(ms.to(dtype=mp.dtype))


# ---- runtime/plugins/zero_common.py:176-193,293-302 ---------------------------------------------
def build_param_buckets(numels_bytes: list[int], bucket_byte_size: int = 25 * 1024 * 1024) -> list[list[int]]:
    """Greedy buckets over parameter indices (given in the order the plugin walks them, i.e. reversed
    model.parameters()): a bucket closes when adding the next parameter would exceed the byte budget;
    a parameter larger than the budget gets a bucket of its own."""
    buckets: list[list[int]] = []
    cur: list[int] = []
    cur_bytes = 0
    for idx, nbytes in enumerate(numels_bytes):
        if cur and cur_bytes + nbytes > bucket_byte_size:
            buckets.append(cur)
            cur, cur_bytes = [], 0
        cur.append(idx)
        cur_bytes += nbytes
    if cur:
        buckets.append(cur)
    return buckets


def padded_len(numel: int, world_size: int) -> int:
    return (numel + world_size - 1) // world_size * world_size
