"""Oracle: RMSNorm, interleaved RoPE, SwiGLU, causal cross-entropy -- forward as the reference's eager
ops evaluate them (including where they round in low precision) and textbook backward formulas."""
from __future__ import annotations

import torch
import torch.nn.functional as F

IGNORE_INDEX = -100  # utils/constants.py:3


# ---- models/llama.py:49-57 -------------------------------------------------------------------
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    variance = x.float().pow(2).mean(dim=-1, keepdim=True)
    return weight * (x * torch.rsqrt(variance + eps)).to(dtype=x.dtype)


def rms_norm_backward(dy, x, weight, eps):
    """dx = r (g - xhat mean(g xhat)), g = dy w, xhat = x r; dw = sum_rows dy xhat (fp32 math)."""
    xf, dyf, wf = x.float(), dy.float(), weight.float()
    r = torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)
    xhat = xf * r
    g = dyf * wf
    dx = r * (g - xhat * (g * xhat).mean(dim=-1, keepdim=True))
    dw = (dyf * xhat).reshape(-1, x.size(-1)).sum(0)
    return dx, dw


# ---- models/llama.py:60-94 -------------------------------------------------------------------
def rope_tables(head_dim: int, max_pos: int, base: float = 10000.0):
    inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    freqs = torch.outer(torch.arange(max_pos, dtype=torch.float32), inv_freq)
    return freqs.cos(), freqs.sin()


def rope_cos_sin(cos_tab, sin_tab, *, seq_len: int, position_offset: int = 0, position_ids=None):
    """[1 or B, 1, S, D/2] slices of the tables (models/llama.py:69-86)."""
    if position_ids is not None:
        if position_ids.dim() == 1:
            position_ids = position_ids.unsqueeze(0)
        flat = position_ids.to(device=cos_tab.device, dtype=torch.long).reshape(-1)
        cos = cos_tab.index_select(0, flat).view(*position_ids.shape, -1).unsqueeze(1)
        sin = sin_tab.index_select(0, flat).view(*position_ids.shape, -1).unsqueeze(1)
        return cos, sin
    return (cos_tab[position_offset:position_offset + seq_len].unsqueeze(0).unsqueeze(0),
            sin_tab[position_offset:position_offset + seq_len].unsqueeze(0).unsqueeze(0))


def apply_rotary(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Interleaved pairs; cos/sin already cast to x.dtype by the caller (models/llama.py:89-94,138-139)."""
    x_even, x_odd = x[..., 0::2], x[..., 1::2]
    out_even = x_even * cos - x_odd * sin
    out_odd = x_even * sin + x_odd * cos
    return torch.stack((out_even, out_odd), dim=-1).flatten(-2)


def apply_rotary_backward(dy: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Rotation by -theta: what autograd of apply_rotary produces, product by product."""
    d_even, d_odd = dy[..., 0::2], dy[..., 1::2]
    dx_even = d_even * cos + d_odd * sin
    dx_odd = d_odd * cos - d_even * sin
    return torch.stack((dx_even, dx_odd), dim=-1).flatten(-2)


# ---- models/llama.py:205-206 -----------------------------------------------------------------
def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return F.silu(gate) * up


def swiglu_backward(dh, gate, up):
    g, u, d = gate.float(), up.float(), dh.float()
    sg = torch.sigmoid(g)
    return d * u * (sg * (1.0 + g * (1.0 - sg))), d * (g * sg)


# ---- utils/losses.py:9-15 --------------------------------------------------------------------
def causal_cross_entropy(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    flat_logits = logits.contiguous().view(-1, logits.size(-1))
    flat_labels = labels.contiguous().view(-1)
    loss_sum = F.cross_entropy(flat_logits, flat_labels, ignore_index=IGNORE_INDEX, reduction="sum")
    target_count = flat_labels.ne(IGNORE_INDEX).sum().clamp_min(1)
    return loss_sum / target_count


def causal_cross_entropy_explicit(logits: torch.Tensor, labels: torch.Tensor):
    """Closed form in fp32: (loss, dlogits) with dlogits = (softmax - onehot) / max(1, count) on supervised rows."""
    z = logits.float().reshape(-1, logits.size(-1))
    y = labels.reshape(-1)
    sup = y != IGNORE_INDEX
    count = max(1, int(sup.sum()))
    lse = torch.logsumexp(z, dim=-1)
    safe_y = torch.where(sup, y, torch.zeros_like(y))
    picked = z.gather(1, safe_y.unsqueeze(1)).squeeze(1)
    loss = torch.where(sup, lse - picked, torch.zeros_like(lse)).sum() / count
    grad = torch.softmax(z, dim=-1)
    grad[torch.arange(z.size(0), device=z.device), safe_y] -= 1.0
    grad = torch.where(sup.unsqueeze(1), grad, torch.zeros_like(grad)) / count
    return loss, grad.view(logits.shape)
