"""LLaMA decoder path on the HIP kernels.

Counterpart of the reference's models/llama.py:30-330 with identical module and parameter names
(embed_tokens, layers.N.self_attn.{q,k,v,o}_proj, layers.N.mlp.{gate,up,down}_proj,
layers.N.{input,post_attention}_layernorm, norm, lm_head), so state dicts are interchangeable.
RMSNorm, RoPE, attention, SwiGLU and the loss are the `maltos::` custom ops; the projections and the
embedding stay on the vendor GEMM library through torch.  Attention consumes the [B, H, S, D] views
of the projection outputs in place and keeps K/V at their native head count.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .attention_backend import AttentionBackend, causal_attention, hip_fallback_reason, uses_hip_kernels, validate_attention_backend
from .attn_masking_utils import canonical_position_ids, canonical_sequence_ids
from .constants import (HIDDEN_STATES_KEY, INPUT_IDS_KEY, LABELS_KEY, LOSS_WEIGHT_KEY, POSITION_IDS_KEY,
                        POSITION_OFFSET_KEY, SEQUENCE_IDS_KEY)
from .losses import causal_cross_entropy
from .optim import notify_grad_written


@dataclass(frozen=True)
class LlamaConfig:
    vocab_size: int
    hidden_size: int = 512
    intermediate_size: int = 2048
    num_hidden_layers: int = 8
    num_attention_heads: int = 8
    num_key_value_heads: int | None = None
    max_position_embeddings: int = 2048
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    tie_word_embeddings: bool = False
    attention_backend: str = AttentionBackend.HIP
    # each residual add is done inside the RMSNorm kernel that follows it (same values; one pass less per sublayer,
    # forward and backward); False keeps the reference's op sequence
    fuse_residual_norm: bool = True
    # when the model computes the loss itself, the loss kernel writes the logits' gradient over the logits (no second
    # buffer of their size).  Nobody else may then read the lm_head output of that forward; the model falls back to a
    # separate gradient buffer by itself while lm_head carries forward hooks (which see that output).  False: always separate
    loss_overwrites_logits: bool = True
    # q/k/v (and gate/up) projections run as one product whenever their weights are adjacent in memory (flat optimizer
    # layouts); the sums inside that product are formed in another order than in three separate ones, so results differ
    # from the separate form in the last bit.  False (or `module.fuse_projections = False` on an attention / MLP module)
    # keeps one product per projection
    fuse_projections: bool = True

    def __post_init__(self) -> None:
        validate_attention_backend(self.attention_backend)


def _weight_grad_splits(rows: int, out_features: int, in_features: int) -> int:
    """Number of K-splits for dW = dY^T X.  The product has only out*in outputs but `rows` (= tokens) terms each:
    for the LLaMA-50M projections (512..1536 wide, 16384 tokens) a single GEMM fills a quarter of the 256 CUs and
    runs at ~85 TFLOP/s, the same work as a batch of 8-16 row slices reaches 300-600 TFLOP/s on MI355X."""
    tiles = -(-out_features // 256) * -(-in_features // 256)
    splits = 1
    while splits < 16 and tiles * splits < 128 and rows % (splits * 2) == 0 and rows // (splits * 2) >= 1024:
        splits *= 2
    return splits


def _weight_grad(x2: torch.Tensor, dy2: torch.Tensor, grad: torch.Tensor | None) -> torch.Tensor | None:
    """dW = dy2^T x2 for [rows, out] / [rows, in] operands, as a batch of row-slice products where that fills the chip
    better.  With `grad` (the gradient buffer the weight already owns, a view of a flat gradient buffer) dW is added
    into it in the pass that finishes it and None is returned; otherwise dW is returned."""
    splits = _weight_grad_splits(x2.shape[0], dy2.shape[1], x2.shape[1])
    if splits > 1 and x2.is_contiguous() and dy2.is_contiguous():
        rows = x2.shape[0] // splits
        part = torch.bmm(dy2.view(splits, rows, -1).transpose(1, 2), x2.view(splits, rows, -1))
        if grad is not None:
            ops.grad_sum_slices(part, grad, accumulate=True)    # fp32 sum of slices + old grad, rounded once
            return None
        return ops.grad_sum_slices(part)                        # slices added in fp32, rounded once
    if grad is not None:
        grad.addmm_(dy2.t(), x2)
        return None
    return dy2.t().matmul(x2)


class _SplitKLinearFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x: torch.Tensor, weight: torch.Tensor, into_grad: bool) -> torch.Tensor:
        ctx.save_for_backward(x, weight)
        ctx.into_grad = into_grad
        return F.linear(x, weight)

    @staticmethod
    def backward(ctx, dy: torch.Tensor):
        x, weight = ctx.saved_tensors
        dx = dw = None
        if ctx.needs_input_grad[0]:
            dx = dy.matmul(weight)
        if ctx.needs_input_grad[1]:
            grad = weight.grad if ctx.into_grad else None
            if grad is not None and not (grad.is_contiguous() and grad.dtype == weight.dtype and grad.shape == weight.shape):
                grad = None
            dw = _weight_grad(x.reshape(-1, x.shape[-1]), dy.reshape(-1, dy.shape[-1]), grad)
            if grad is not None:
                notify_grad_written(weight)   # autograd's hooks on the weight see no gradient for what was added here
        return dx, dw, None


# ---- projections that share their input, run as ONE GEMM over adjacent weights ------------------------------------
# q_proj / k_proj / v_proj (and gate_proj / up_proj) read the same activations.  When their weights are adjacent row
# blocks of one allocation (what the flat optimizer layouts make of them: MasterWeightsOptimizer(flat=True),
# Zero1FlatBuffers), they ARE one [sum of out_features, in_features] matrix, and the three (two) products are one: at
# LLaMA-50M sizes a 512-wide product has 128 output tiles for 256 compute units, the 1536-wide one fills the chip, and
# the backward's three input-gradient products and their two additions become one product.  Parameter names, shapes
# and values are untouched; without adjacency the projections run one by one as in the reference (models/llama.py:
# 134-142,196-206).
class _FusedRows:
    """Adjacent 2-D parameters seen as one matrix: `weight` [R, in] and, when their .grad views are adjacent in the same
    order, `grad` [R, in]; `cols[i]` = (first, last + 1) output column of parameter i (caller order)."""

    __slots__ = ("key", "weight", "grad", "cols")


def _fused_rows(holder: nn.Module, params: list[nn.Parameter]) -> _FusedRows | None:
    key = tuple((p.data_ptr(), 0 if p.grad is None else p.grad.data_ptr()) for p in params)
    cached = holder.__dict__.get("_maltos_hip_fused_rows")
    if cached is not None and cached.key == key:
        return cached if cached.weight is not None else None
    fused = _FusedRows()
    fused.key, fused.weight, fused.grad, fused.cols = key, None, None, []
    holder.__dict__["_maltos_hip_fused_rows"] = fused
    first = params[0]
    if not all(p.dim() == 2 and p.is_cuda and p.is_contiguous() and p.dtype == first.dtype and p.size(1) == first.size(1)
               and p.requires_grad for p in params):
        return None
    order = sorted(range(len(params)), key=lambda i: params[i].data_ptr())
    es = first.element_size()
    for a, b in zip(order, order[1:]):
        pa, pb = params[a], params[b]
        if pa.untyped_storage().data_ptr() != pb.untyped_storage().data_ptr() or pa.data_ptr() + pa.numel() * es != pb.data_ptr():
            return None
    rows = sum(p.size(0) for p in params)
    base = params[order[0]]
    fused.weight = base.data.as_strided((rows, base.size(1)), (base.size(1), 1))
    start, cols = 0, [None] * len(params)
    for i in order:
        cols[i] = (start, start + params[i].size(0))
        start += params[i].size(0)
    fused.cols = cols
    grads = [p.grad for p in params]
    if all(g is not None and g.is_contiguous() and g.dtype == first.dtype and g.shape == p.shape for g, p in zip(grads, params)):
        if all(grads[a].untyped_storage().data_ptr() == grads[b].untyped_storage().data_ptr()
               and grads[a].data_ptr() + grads[a].numel() * es == grads[b].data_ptr() for a, b in zip(order, order[1:])):
            g0 = grads[order[0]]
            fused.grad = g0.as_strided((rows, g0.size(1)), (g0.size(1), 1))
    return fused


def _adjacent_columns(parts: list[torch.Tensor]) -> torch.Tensor | None:
    """The [rows, sum of widths] matrix whose column ranges the given [..., width_i] tensors are, in this order, when
    they are such views of one dense buffer; None otherwise (then the caller copies them together)."""
    first = parts[0]
    lead = first.shape[:-1]
    total = sum(p.size(-1) for p in parts)
    want, step = [], total
    for n in reversed(lead):   # strides of a dense [*lead, total] buffer
        want.append(step)
        step *= n
    want = tuple(reversed(want)) + (1,)
    storage, offset = first.untyped_storage().data_ptr(), first.storage_offset()
    for p in parts:
        if (p.shape[:-1] != lead or p.dtype != first.dtype or p.untyped_storage().data_ptr() != storage
                or p.storage_offset() != offset or any(n > 1 and a != b for n, a, b in zip(p.shape, p.stride(), want))):
            return None
        offset += p.size(-1)
    rows = 1
    for n in lead:
        rows *= n
    return first.as_strided((rows, total), (total, 1), first.storage_offset())


def _fusable(modules: list[nn.Module]) -> bool:
    return all(isinstance(m, HipLinear) and m.bias is None for m in modules)


class _FusedLinearsFn(torch.autograd.Function):
    """(x W_0^T, x W_1^T, ...) from one product with the parameters' common matrix; the outputs are column slices of it."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, fused: _FusedRows, into_grad: bool, *weights: torch.Tensor):
        ctx.save_for_backward(x)
        ctx.fused, ctx.into_grad, ctx.weights = fused, into_grad and fused.grad is not None, weights
        y = F.linear(x, fused.weight)
        return tuple(y[..., a:b] for a, b in fused.cols)

    @staticmethod
    def backward(ctx, *dys):
        (x,) = ctx.saved_tensors
        fused = ctx.fused
        rows_total = fused.weight.size(0)
        x2 = x.reshape(-1, x.shape[-1])
        # the slices' gradients side by side, in the order of the rows of the common matrix
        order = sorted(range(len(dys)), key=lambda i: fused.cols[i][0])
        if all(dy is not None for dy in dys):
            dy2 = _adjacent_columns([dys[i] for i in order])   # already side by side (attention's joint gradient buffer)?
            if dy2 is None:
                dy2 = torch.cat([dys[i].reshape(-1, fused.cols[i][1] - fused.cols[i][0]) for i in order], dim=1)  # one launch
        else:
            dy2 = torch.empty((x2.shape[0], rows_total), dtype=x.dtype, device=x.device)
            for (a, b), dy in zip(fused.cols, dys):
                if dy is None:
                    dy2[:, a:b].zero_()
                else:
                    dy2[:, a:b].copy_(dy.reshape(-1, b - a))
        dx = dy2.matmul(fused.weight).view(x.shape) if ctx.needs_input_grad[0] else None
        dw = _weight_grad(x2, dy2, fused.grad if ctx.into_grad else None)
        if dw is None:
            for w in ctx.weights:
                notify_grad_written(w)
            return (dx, None, None, *([None] * len(ctx.weights)))
        return (dx, None, None, *(dw[a:b] for a, b in fused.cols))


class _FusedGateUpFn(torch.autograd.Function):
    """round(silu(x W_gate^T)) * (x W_up^T) (models/llama.py:205-206) with the two projections as one product; the
    backward writes d gate and d up side by side, so that the input gradient is one product as well."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, fused: _FusedRows, into_grad: bool, w_gate: torch.Tensor, w_up: torch.Tensor):
        gu = F.linear(x, fused.weight)
        ctx.save_for_backward(x, gu)
        ctx.fused, ctx.into_grad, ctx.weights = fused, into_grad and fused.grad is not None, (w_gate, w_up)
        return ops.swiglu_rows(gu, fused.cols[0][0], fused.cols[1][0], w_gate.size(0))

    @staticmethod
    def backward(ctx, dh: torch.Tensor):
        x, gu = ctx.saved_tensors
        fused = ctx.fused
        dgu = ops.swiglu_rows_backward(dh, gu, fused.cols[0][0], fused.cols[1][0], ctx.weights[0].size(0))
        dgu2 = dgu.view(-1, dgu.shape[-1])
        dx = dgu2.matmul(fused.weight).view(x.shape) if ctx.needs_input_grad[0] else None
        dw = _weight_grad(x.reshape(-1, x.shape[-1]), dgu2, fused.grad if ctx.into_grad else None)
        if dw is None:
            for w in ctx.weights:
                notify_grad_written(w)
            return dx, None, None, None, None
        return (dx, None, None, *(dw[a:b] for a, b in fused.cols))


class HipLinear(nn.Linear):
    """nn.Linear (same parameter name and init) whose weight gradient is computed as a batch of row slices when the
    output is too small to fill the chip (reference: plain nn.Linear, models/llama.py:69-75,196-198).

    `accumulate_into_grad = True` (off by default; set it on the class or on an instance) makes the backward add dW
    straight into an existing `weight.grad` and return no gradient for the weight: one pass instead of two when the
    gradients live in a flat buffer that is cleared, not dropped, between steps.  Autograd hooks on the weight see no
    gradient in that mode (they run with None), so it is for callers that read the gradients from the buffer after
    backward; whoever needs to know that the buffer was written is told through `optim.notify_grad_written`."""

    accumulate_into_grad = False

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.bias is not None or not x.is_cuda:
            return F.linear(x, self.weight, self.bias)
        return _SplitKLinearFn.apply(x, self.weight, bool(self.accumulate_into_grad))


def set_grad_accumulation_into_buffers(model: nn.Module, enabled: bool = True) -> int:
    """Switches `HipLinear.accumulate_into_grad` on every HipLinear of `model`; returns how many were switched."""
    count = 0
    for module in model.modules():
        if isinstance(module, HipLinear):
            module.accumulate_into_grad = bool(enabled)
            count += 1
    return count


class LlamaRMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.eps = eps

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.rms_norm(x, self.weight, self.eps)


class LlamaRotaryEmbedding(nn.Module):
    """cos/sin tables [max_position_embeddings, head_dim / 2], built in fp32 and cast with the module."""

    def __init__(self, head_dim: int, max_position_embeddings: int, base: float) -> None:
        super().__init__()
        exponents = torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim
        angles = torch.arange(max_position_embeddings, dtype=torch.float32)[:, None] * (base ** -exponents)[None, :]
        self.register_buffer("cos", torch.cos(angles), persistent=False)
        self.register_buffer("sin", torch.sin(angles), persistent=False)

    def tables(self, dtype: torch.dtype, device: torch.device) -> tuple[torch.Tensor, torch.Tensor]:
        if self.cos.dtype != dtype or self.cos.device != device:
            # fp32 -> dtype is the single rounding the reference applies (cos.to(x.dtype))
            return self.cos.to(device=device, dtype=dtype), self.sin.to(device=device, dtype=dtype)
        return self.cos, self.sin


class HipAttentionCore(nn.Module):
    """`attn_core` of LlamaAttention: (q, k, v, position_offset, position_ids, sequence_ids) -> out."""

    preserves_native_gqa = True

    def __init__(self, attention_backend: str = AttentionBackend.HIP) -> None:
        super().__init__()
        self.attention_backend = validate_attention_backend(attention_backend)

    def row_ids(self, q, position_offset: int, position_ids=None, sequence_ids=None):
        """(positions, sequence ids) of the rows as the attention kernels take them, or (None, None) for plain causal rows."""
        if position_ids is None and sequence_ids is None:
            return None, None
        positions = canonical_position_ids(position_ids, batch_size=q.size(0), seq_len=q.size(-2),
                                           position_offset=position_offset, device=q.device)
        return positions, canonical_sequence_ids(sequence_ids, batch_size=q.size(0), seq_len=q.size(-2), device=q.device)

    def forward(self, q, k, v, position_offset: int, position_ids=None, sequence_ids=None) -> torch.Tensor:
        positions, sequences = self.row_ids(q, position_offset, position_ids, sequence_ids)
        return causal_attention(q, k, v, attention_backend=self.attention_backend, warning_prefix="LlamaAttention",
                                q_positions=positions, k_positions=positions, q_sequence_ids=sequences,
                                k_sequence_ids=sequences, flash_varlen_mode="same_length")


class _RopeAttentionFn(torch.autograd.Function):
    """attention(rotary(q), rotary(k), v) (models/llama.py:143-150) as one autograd node over the same kernels as the
    separate ops, hence the same values.  What the node adds is the layout of its backward: dQ, dK and dV are head ranges
    of one [B, S, Hq + 2 Hkv, D] buffer and the rotation of dQ / dK back is done in place there (the buffer is the node's
    own until it returns), so the gradient of q/k/v projections that run as one product arrives as one matrix."""

    @staticmethod
    def forward(ctx, q, k, v, cos, sin, rope_positions, position_offset: int, positions, sequences):
        q, k = torch.ops.maltos.rope_pair(q, k, cos, sin, rope_positions, position_offset, False)
        mask_mode = ops.MASK_CAUSAL
        if positions is not None:
            mask_mode = ops.MASK_DOC
            if sequences is None:   # positions only: one document per row (the zero ids are kept with the positions)
                sequences = ops.derived_from(positions, "_maltos_hip_zero_ids",
                                             lambda pos: torch.zeros(pos.shape, dtype=torch.int32, device=pos.device))
        out, lse = ops.attention_forward(q, k, v, mask_mode=mask_mode, q_pos=positions, k_pos=positions, q_seq=sequences,
                                         k_seq=sequences)
        ctx.save_for_backward(q, k, v, out, lse, cos, sin, rope_positions, positions, sequences)
        ctx.position_offset, ctx.mask_mode = position_offset, mask_mode
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse, cos, sin, rope_positions, positions, sequences = ctx.saved_tensors
        dq, dk, dv = ops.attention_backward(dout, q, k, v, out, lse, mask_mode=ctx.mask_mode, q_pos=positions,
                                            k_pos=positions, q_seq=sequences, k_seq=sequences)
        ops.rope_pair_(dq, dk, cos, sin, positions=rope_positions, position_offset=ctx.position_offset, inverse=True)
        return dq, dk, dv, None, None, None, None, None, None


class LlamaAttention(nn.Module):
    # rotary embedding and attention as one autograd node whenever `attn_core` is the stock HipAttentionCore on the HIP
    # kernels (same values; see _RopeAttentionFn).  False keeps the two ops apart
    fuse_rope_attention = True

    def __init__(self, config: LlamaConfig) -> None:
        super().__init__()
        if config.hidden_size % config.num_attention_heads != 0:
            raise ValueError("hidden_size must be divisible by num_attention_heads")
        self.num_heads = config.num_attention_heads
        self.num_kv_heads = config.num_key_value_heads or config.num_attention_heads
        if self.num_heads % self.num_kv_heads != 0:
            raise ValueError("num_attention_heads must be divisible by num_key_value_heads")
        self.head_dim = config.hidden_size // config.num_attention_heads
        self.rotary_emb = LlamaRotaryEmbedding(self.head_dim, config.max_position_embeddings, config.rope_theta)
        self.q_proj = HipLinear(config.hidden_size, self.num_heads * self.head_dim, bias=False)
        self.k_proj = HipLinear(config.hidden_size, self.num_kv_heads * self.head_dim, bias=False)
        self.v_proj = HipLinear(config.hidden_size, self.num_kv_heads * self.head_dim, bias=False)
        self.o_proj = HipLinear(config.hidden_size, config.hidden_size, bias=False)
        self.attn_core = HipAttentionCore(config.attention_backend)
        self.fuse_projections = config.fuse_projections

    def forward(self, x: torch.Tensor, *, position_offset: int = 0, position_ids: torch.Tensor | None = None,
                sequence_ids: torch.Tensor | None = None) -> torch.Tensor:
        batch, seq_len, _ = x.shape
        cos, sin = self.rotary_emb.tables(x.dtype, x.device)
        rope_pos = None
        if position_ids is not None:
            rope_pos = canonical_position_ids(position_ids, batch_size=batch, seq_len=seq_len, position_offset=0,
                                              device=x.device)
        # [B, S, H*D] -> [B, H, S, D] views; no copies until the kernels read them
        projections = [self.q_proj, self.k_proj, self.v_proj]
        fused = None
        if self.fuse_projections and x.is_cuda and _fusable(projections):
            fused = _fused_rows(self, [m.weight for m in projections])
        if fused is not None:   # one product over the three adjacent weights
            q, k, v = _FusedLinearsFn.apply(x, fused, all(m.accumulate_into_grad for m in projections),
                                            *(m.weight for m in projections))
        else:
            q, k, v = self.q_proj(x), self.k_proj(x), self.v_proj(x)
        q = q.view(batch, seq_len, self.num_heads, self.head_dim).transpose(1, 2)
        k = k.view(batch, seq_len, self.num_kv_heads, self.head_dim).transpose(1, 2)
        v = v.view(batch, seq_len, self.num_kv_heads, self.head_dim).transpose(1, 2)
        core = self.attn_core
        if (self.fuse_rope_attention and type(core) is HipAttentionCore and uses_hip_kernels(core.attention_backend)
                and hip_fallback_reason(q) is None):
            positions, sequences = core.row_ids(q, position_offset, position_ids, sequence_ids)
            vo = _RopeAttentionFn.apply(q, k, v, cos, sin, rope_pos, int(position_offset), positions, sequences)
            return self.o_proj(vo.transpose(1, 2).reshape(batch, seq_len, self.num_heads * self.head_dim))
        q, k = ops.rope_pair(q, k, cos, sin, positions=rope_pos, position_offset=position_offset)
        if not getattr(self.attn_core, "preserves_native_gqa", False) and self.num_heads != self.num_kv_heads:
            rep = self.num_heads // self.num_kv_heads
            k, v = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
        vo = self.attn_core(q, k, v, position_offset, position_ids, sequence_ids)
        return self.o_proj(vo.transpose(1, 2).reshape(batch, seq_len, self.num_heads * self.head_dim))


class LlamaMLP(nn.Module):
    def __init__(self, config: LlamaConfig) -> None:
        super().__init__()
        self.gate_proj = HipLinear(config.hidden_size, config.intermediate_size, bias=False)
        self.up_proj = HipLinear(config.hidden_size, config.intermediate_size, bias=False)
        self.down_proj = HipLinear(config.intermediate_size, config.hidden_size, bias=False)
        self.fuse_projections = config.fuse_projections

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        pair = [self.gate_proj, self.up_proj]
        fused = None
        if self.fuse_projections and x.is_cuda and _fusable(pair) and self.gate_proj.out_features % (16 // x.element_size()) == 0:
            fused = _fused_rows(self, [m.weight for m in pair])
        if fused is not None:
            h = _FusedGateUpFn.apply(x, fused, all(m.accumulate_into_grad for m in pair), self.gate_proj.weight, self.up_proj.weight)
            return self.down_proj(h)
        return self.down_proj(ops.swiglu(self.gate_proj(x), self.up_proj(x)))


class LlamaDecoderLayer(nn.Module):
    def __init__(self, config: LlamaConfig) -> None:
        super().__init__()
        self.self_attn = LlamaAttention(config)
        self.mlp = LlamaMLP(config)
        self.input_layernorm = LlamaRMSNorm(config.hidden_size, config.rms_norm_eps)
        self.post_attention_layernorm = LlamaRMSNorm(config.hidden_size, config.rms_norm_eps)

    def forward(self, x: torch.Tensor, position_offset: int = 0, position_ids: torch.Tensor | None = None,
                sequence_ids: torch.Tensor | None = None, pending: torch.Tensor | None = None,
                defer_residual: bool = False):
        """Reference form (:217-231): x -> x.  With `defer_residual` the layer returns (x, mlp_out) and leaves the last
        residual add to whoever normalises next, and takes such a not-yet-added `pending` from the layer before."""
        if not defer_residual:
            if pending is not None:
                x = x + pending
            x = x + self.self_attn(self.input_layernorm(x), position_offset=position_offset, position_ids=position_ids,
                                   sequence_ids=sequence_ids)
            return x + self.mlp(self.post_attention_layernorm(x))
        ln1, ln2 = self.input_layernorm, self.post_attention_layernorm
        if pending is None:
            normed = ln1(x)
        else:
            x, normed = ops.add_rms_norm(x, pending, ln1.weight, ln1.eps)
        attn_out = self.self_attn(normed, position_offset=position_offset, position_ids=position_ids, sequence_ids=sequence_ids)
        x, normed = ops.add_rms_norm(x, attn_out, ln2.weight, ln2.eps)
        return x, self.mlp(normed)


class LlamaForCausalLM(nn.Module):
    def __init__(self, config: LlamaConfig) -> None:
        super().__init__()
        self.config = config
        self.embed_tokens = nn.Embedding(config.vocab_size, config.hidden_size)
        self.layers = nn.ModuleList([LlamaDecoderLayer(config) for _ in range(config.num_hidden_layers)])
        self.norm = LlamaRMSNorm(config.hidden_size, config.rms_norm_eps)
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)
        if config.tie_word_embeddings:
            self.lm_head.weight = self.embed_tokens.weight

    def forward(self, batch):
        """Accepts the reference's batch forms: dict with the constants' keys, (input_ids, labels), or input_ids.
        Returns the scalar loss when labels are given (already aligned, no shift), else the logits."""
        hidden_states = position_ids = sequence_ids = loss_weight = labels = None
        position_offset = 0
        if isinstance(batch, dict):
            input_ids = batch.get(INPUT_IDS_KEY)
            hidden_states = batch.get(HIDDEN_STATES_KEY)
            labels = batch.get(LABELS_KEY)
            position_offset = int(batch.get(POSITION_OFFSET_KEY, 0))
            position_ids = batch.get(POSITION_IDS_KEY)
            sequence_ids = batch.get(SEQUENCE_IDS_KEY)
            loss_weight = batch.get(LOSS_WEIGHT_KEY)
        elif isinstance(batch, (tuple, list)):
            input_ids, labels = batch
        else:
            input_ids = batch
        if hidden_states is not None:
            x = hidden_states
        elif input_ids is None:
            raise ValueError("LlamaForCausalLM requires input_ids or hidden_states")
        else:
            x = self.embed_tokens(input_ids)
        if position_ids is not None or sequence_ids is not None:
            # canonical [batch, seq] ids once per forward: every layer's attention is then handed the SAME tensors and
            # shares what is derived from them (int32 forms, the document-mask plan), where per-layer canonicalisation
            # (models/llama.py:163-175 of the reference) makes fresh ones whenever the batch's ids are rank 1, not int64,
            # on the host, or absent.  Positions made here carry position_offset, which the rotary kernel then ignores.
            position_ids = canonical_position_ids(position_ids, batch_size=x.size(0), seq_len=x.size(1),
                                                  position_offset=position_offset, device=x.device)
            sequence_ids = canonical_sequence_ids(sequence_ids, batch_size=x.size(0), seq_len=x.size(1), device=x.device)
        if self.config.fuse_residual_norm and x.is_cuda and len(self.layers) > 0:
            pending = None
            for layer in self.layers:
                x, pending = layer(x, position_offset=position_offset, position_ids=position_ids, sequence_ids=sequence_ids,
                                   pending=pending, defer_residual=True)
            _, normed = ops.add_rms_norm(x, pending, self.norm.weight, self.norm.eps)
        else:
            for layer in self.layers:
                x = layer(x, position_offset=position_offset, position_ids=position_ids, sequence_ids=sequence_ids)
            normed = self.norm(x)
        logits = self.lm_head(normed)
        if labels is None:
            return logits
        if input_ids is not None and labels.shape != input_ids.shape:
            raise ValueError(f"labels shape must match input_ids shape, got {labels.shape} vs {input_ids.shape}")
        # the logits are this function's own and are not returned with the loss: their gradient may take their place
        own = self.config.loss_overwrites_logits and not self.lm_head._forward_hooks
        loss = causal_cross_entropy(logits, labels, overwrite_logits=own and logits.is_cuda and logits.is_contiguous())
        return loss if loss_weight is None else loss * float(loss_weight)

    def context_parallel_spec(self) -> list[str]:
        """Module paths whose `attn_core` a context-parallel plugin swaps (reference :311-314)."""
        return [f"layers.{i}.self_attn" for i in range(len(self.layers))]

    def flops_per_token(self) -> float:
        """The reference's estimator (:319-330): 3 x forward, attention counted non-causal."""
        c = self.config
        h, i, s, v = c.hidden_size, c.intermediate_size, c.max_position_embeddings, c.vocab_size
        per_layer = 6 * h * h + 2 * h * h + 6 * h * i + 4 * s * h
        return float(3 * (c.num_hidden_layers * per_layer + 2 * h * v))
