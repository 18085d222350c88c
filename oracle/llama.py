"""Oracle: the LLaMA decoder path of the reference as a plain-PyTorch functional model.

Follows models/llama.py:30-302 op for op (RMSNorm -> q/k/v proj -> view/transpose -> interleaved RoPE
with tables cast to the activation dtype -> repeat_kv -> masked / causal attention -> o_proj ->
residual -> RMSNorm -> SwiGLU MLP -> residual; final norm, lm_head, causal cross-entropy on labels
that are already aligned).  Parameters live in an ordered dict whose names and order are those of
LlamaForCausalLM.named_parameters(): embed_tokens.weight, layers.N.self_attn.{q,k,v,o}_proj.weight,
layers.N.mlp.{gate,up,down}_proj.weight, layers.N.input_layernorm.weight,
layers.N.post_attention_layernorm.weight, norm.weight, lm_head.weight.
"""
from __future__ import annotations

from collections import OrderedDict
from dataclasses import dataclass

import torch
import torch.nn.functional as F

from . import attention as oa
from . import layers as ol


@dataclass(frozen=True)
class OracleLlamaConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int | None = None
    max_position_embeddings: int = 2048
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    @property
    def kv_heads(self) -> int:
        return self.num_key_value_heads or self.num_attention_heads


def param_shapes(cfg: OracleLlamaConfig) -> "OrderedDict[str, tuple[int, ...]]":
    h, i, d = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim
    shapes: "OrderedDict[str, tuple[int, ...]]" = OrderedDict()
    shapes["embed_tokens.weight"] = (cfg.vocab_size, h)
    for n in range(cfg.num_hidden_layers):
        pre = f"layers.{n}."
        shapes[pre + "self_attn.q_proj.weight"] = (cfg.num_attention_heads * d, h)
        shapes[pre + "self_attn.k_proj.weight"] = (cfg.kv_heads * d, h)
        shapes[pre + "self_attn.v_proj.weight"] = (cfg.kv_heads * d, h)
        shapes[pre + "self_attn.o_proj.weight"] = (h, h)
        shapes[pre + "mlp.gate_proj.weight"] = (i, h)
        shapes[pre + "mlp.up_proj.weight"] = (i, h)
        shapes[pre + "mlp.down_proj.weight"] = (h, i)
        shapes[pre + "input_layernorm.weight"] = (h,)
        shapes[pre + "post_attention_layernorm.weight"] = (h,)
    shapes["norm.weight"] = (h,)
    shapes["lm_head.weight"] = (cfg.vocab_size, h)
    return shapes


def init_params(cfg: OracleLlamaConfig, seed: int, std: float = 0.02) -> "OrderedDict[str, torch.Tensor]":
    """Every >=2-D parameter <- randn * std from one CPU generator, in named_parameters() order; norm
    weights stay 1.0 (the benchmark configurations' init rule)."""
    gen = torch.Generator().manual_seed(seed)
    params: "OrderedDict[str, torch.Tensor]" = OrderedDict()
    for name, shape in param_shapes(cfg).items():
        if len(shape) >= 2:
            params[name] = torch.randn(shape, generator=gen, dtype=torch.float32) * std
        else:
            params[name] = torch.ones(shape, dtype=torch.float32)
    return params


def attention_core(q, k, v, *, position_ids=None, sequence_ids=None, position_offset: int = 0):
    """_LlamaAttentionCore + causal_attention (models/llama.py:154-195, utils/attention_backend.py:42-118):
    plain causal when no ids are given, else the example-aware mask; computed in the activation dtype's
    fp32 upcast and returned in the activation dtype."""
    b, _, s, _ = q.shape
    if position_ids is None and sequence_ids is None:
        mask = oa.causal_mask(s, s, q.device)
    else:
        pos = oa.canonical_ids(position_ids, batch_size=b, seq_len=s, position_offset=position_offset, device=q.device)
        seq = oa.canonical_ids(sequence_ids, batch_size=b, seq_len=s, position_offset=None, device=q.device)
        mask = oa.example_causal_mask(pos, pos, seq, seq).unsqueeze(1)
    out, _ = oa.attention_with_lse(q, k, v, mask)
    return out.to(q.dtype)


def forward(params, cfg: OracleLlamaConfig, input_ids, labels=None, *, position_ids=None, sequence_ids=None,
            position_offset: int = 0):
    """Loss (labels given) or logits; models/llama.py:245-302."""
    dtype = params["embed_tokens.weight"].dtype
    b, s = input_ids.shape
    d = cfg.head_dim
    cos_tab, sin_tab = ol.rope_tables(d, cfg.max_position_embeddings, cfg.rope_theta)
    cos_tab, sin_tab = cos_tab.to(input_ids.device), sin_tab.to(input_ids.device)
    cos, sin = ol.rope_cos_sin(cos_tab, sin_tab, seq_len=s, position_offset=position_offset, position_ids=position_ids)
    cos, sin = cos.to(dtype), sin.to(dtype)
    x = F.embedding(input_ids, params["embed_tokens.weight"])
    for n in range(cfg.num_hidden_layers):
        pre = f"layers.{n}."
        hn = ol.rms_norm(x, params[pre + "input_layernorm.weight"], cfg.rms_norm_eps)
        q = F.linear(hn, params[pre + "self_attn.q_proj.weight"]).view(b, s, -1, d).transpose(1, 2)
        k = F.linear(hn, params[pre + "self_attn.k_proj.weight"]).view(b, s, -1, d).transpose(1, 2)
        v = F.linear(hn, params[pre + "self_attn.v_proj.weight"]).view(b, s, -1, d).transpose(1, 2)
        q, k = ol.apply_rotary(q, cos, sin), ol.apply_rotary(k, cos, sin)
        vo = attention_core(q, k, v, position_ids=position_ids, sequence_ids=sequence_ids, position_offset=position_offset)
        x = x + F.linear(vo.transpose(1, 2).contiguous().view(b, s, -1), params[pre + "self_attn.o_proj.weight"])
        hn = ol.rms_norm(x, params[pre + "post_attention_layernorm.weight"], cfg.rms_norm_eps)
        act = ol.swiglu(F.linear(hn, params[pre + "mlp.gate_proj.weight"]), F.linear(hn, params[pre + "mlp.up_proj.weight"]))
        x = x + F.linear(act, params[pre + "mlp.down_proj.weight"])
    logits = F.linear(ol.rms_norm(x, params["norm.weight"], cfg.rms_norm_eps), params["lm_head.weight"])
    if labels is None:
        return logits
    return ol.causal_cross_entropy(logits, labels)


def flops_per_token(cfg: OracleLlamaConfig) -> float:
    """models/llama.py:319-330 (attention counted non-causal)."""
    h, i, s, v = cfg.hidden_size, cfg.intermediate_size, cfg.max_position_embeddings, cfg.vocab_size
    fwd = cfg.num_hidden_layers * (6 * h * h + 2 * h * h + 6 * h * i + 4 * s * h) + 2 * h * v
    return float(3 * fwd)


def train_step(params, cfg: OracleLlamaConfig, input_ids, labels, *, lr=3e-4, betas=(0.9, 0.95), eps=1e-8,
               weight_decay=0.1, max_norm: float | None = None, **fwd_kwargs):
    """One full step with stock torch.optim.AdamW on fp32 masters (runtime/optim.py:65-71 semantics when the
    model dtype is low precision).  Returns (loss, grad_norm, new_params fp32 masters)."""
    leaves = OrderedDict((n, p.detach().clone().requires_grad_(True)) for n, p in params.items())
    loss = forward(leaves, cfg, input_ids, labels, **fwd_kwargs)
    loss.backward()
    masters = [torch.nn.Parameter(p.detach().float().clone()) for p in leaves.values()]
    grads = [p.grad.detach().float().clone() for p in leaves.values()]
    from .optim import clip_grads_, global_grad_norm

    grad_norm = clip_grads_(grads, max_norm) if max_norm is not None else global_grad_norm(grads)
    for mp, g in zip(masters, grads):
        mp.grad = g
    opt = torch.optim.AdamW(masters, lr=lr, betas=betas, eps=eps, weight_decay=weight_decay)
    opt.step()
    new_params = OrderedDict((n, mp.detach()) for n, mp in zip(leaves.keys(), masters))
    return float(loss.detach().float()), grad_norm, new_params
