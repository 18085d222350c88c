"""Pins oracle/llama.py.

  * parameter inventory and estimator : the derived sizes 7,358,720 / 58,073,600 params and
    350,748,672 flops/token (reference formulas models/llama.py:233-243,319-330).
  * forward                           : the same network evaluated with library routines only
    (F.rms_norm, F.scaled_dot_product_attention(is_causal), F.silu, F.cross_entropy(mean)) agrees to 1e-5
    on logits, the tolerance of the reference's sdpa-vs-eager check (tests/smoke_runtime_core.py:920-942);
    packed documents agree with running each document separately.
  * train_step                        : the committed cfg1 fixture is reproduced (determinism across runs).
"""
import json
from collections import OrderedDict

import torch
import torch.nn.functional as F

from oracle import layers as ol_layers
from oracle import llama as ol
from tests.golden.make_cfg1_fixture import CFG1, cfg1_inputs
from tests.conftest import GOLDEN_DIR

CFG5 = dict(vocab_size=32000, hidden_size=512, intermediate_size=1376, num_hidden_layers=8, num_attention_heads=8,
            max_position_embeddings=2048, rms_norm_eps=1e-5)


def test_derived_sizes(known_answers):
    ds = known_answers["derived_sizes"]
    c1, c5 = ol.OracleLlamaConfig(**CFG1), ol.OracleLlamaConfig(**CFG5)
    count = lambda c: sum(torch.Size(s).numel() for s in ol.param_shapes(c).values())
    assert count(c1) == ds["cfg1_params"] and count(c5) == ds["cfg5_params"]
    assert ol.flops_per_token(c5) == ds["cfg5_flops_per_token"]


def _library_forward(params, cfg, input_ids):
    b, s = input_ids.shape
    d = cfg.head_dim
    cos_t, sin_t = ol_layers.rope_tables(d, cfg.max_position_embeddings, cfg.rope_theta)
    ang = torch.arange(s, dtype=torch.float32)[:, None] * (cfg.rope_theta ** (-torch.arange(0, d, 2).float() / d))[None]
    x = params["embed_tokens.weight"][input_ids]

    def rot(t):  # complex multiplication form of the interleaved rotation
        tc = torch.view_as_complex(t.float().reshape(*t.shape[:-1], -1, 2).contiguous())
        return torch.view_as_real(tc * torch.polar(torch.ones_like(ang), ang)).flatten(-2)

    for n in range(cfg.num_hidden_layers):
        pre = f"layers.{n}."
        hn = F.rms_norm(x, (cfg.hidden_size,), params[pre + "input_layernorm.weight"], cfg.rms_norm_eps)
        q = (hn @ params[pre + "self_attn.q_proj.weight"].T).view(b, s, -1, d).transpose(1, 2)
        k = (hn @ params[pre + "self_attn.k_proj.weight"].T).view(b, s, -1, d).transpose(1, 2)
        v = (hn @ params[pre + "self_attn.v_proj.weight"].T).view(b, s, -1, d).transpose(1, 2)
        a = F.scaled_dot_product_attention(rot(q), rot(k), v, is_causal=True)
        x = x + a.transpose(1, 2).reshape(b, s, -1) @ params[pre + "self_attn.o_proj.weight"].T
        hn = F.rms_norm(x, (cfg.hidden_size,), params[pre + "post_attention_layernorm.weight"], cfg.rms_norm_eps)
        x = x + (F.silu(hn @ params[pre + "mlp.gate_proj.weight"].T) * (hn @ params[pre + "mlp.up_proj.weight"].T)) @ params[pre + "mlp.down_proj.weight"].T
    return F.rms_norm(x, (cfg.hidden_size,), params["norm.weight"], cfg.rms_norm_eps) @ params["lm_head.weight"].T


def test_forward_matches_library_composition(known_answers):
    cfg = ol.OracleLlamaConfig(vocab_size=97, hidden_size=64, intermediate_size=112, num_hidden_layers=2,
                               num_attention_heads=4, max_position_embeddings=32)
    params = ol.init_params(cfg, 3, std=0.2)
    ids = torch.randint(0, 97, (2, 17), generator=torch.Generator().manual_seed(4))
    logits = ol.forward(params, cfg, ids)
    ref = _library_forward(params, cfg, ids)
    assert torch.allclose(logits, ref, atol=known_answers["tolerances"]["sdpa_vs_eager_logits_atol"])
    labels = torch.randint(0, 97, (2, 17), generator=torch.Generator().manual_seed(5))
    loss = ol.forward(params, cfg, ids, labels)
    assert torch.allclose(loss, F.cross_entropy(ref.view(-1, 97), labels.view(-1)), atol=1e-5)


def test_packed_documents_equal_separate_documents():
    cfg = ol.OracleLlamaConfig(vocab_size=50, hidden_size=32, intermediate_size=48, num_hidden_layers=2,
                               num_attention_heads=2, max_position_embeddings=16)
    params = ol.init_params(cfg, 8, std=0.3)
    ids = torch.randint(0, 50, (1, 9), generator=torch.Generator().manual_seed(9))
    pos = torch.tensor([[0, 1, 2, 3, 0, 1, 2, 3, 4]])
    seq = torch.tensor([[0, 0, 0, 0, 1, 1, 1, 1, 1]])
    packed = ol.forward(params, cfg, ids, position_ids=pos, sequence_ids=seq)
    a = ol.forward(params, cfg, ids[:, :4])
    b = ol.forward(params, cfg, ids[:, 4:])
    assert torch.allclose(packed, torch.cat([a, b], dim=1), atol=1e-5)


def test_cfg1_fixture_is_reproduced():
    fixture = json.loads((GOLDEN_DIR / "cfg1_tiny_llama_step.json").read_text())
    cfg, params, input_ids, labels = cfg1_inputs()
    assert list(params.keys()) == list(fixture["params"].keys())
    loss, grad_norm, new_params = ol.train_step(params, cfg, input_ids, labels)
    assert abs(loss - fixture["loss"]) <= 1e-4 * abs(fixture["loss"])
    assert abs(grad_norm - fixture["grad_norm"]) <= 1e-4 * fixture["grad_norm"]
    for name, rec in fixture["params"].items():
        p = new_params[name]
        assert abs(float(p.double().abs().sum()) - rec["abs_sum"]) <= 1e-4 * rec["abs_sum"], name
        assert torch.allclose(p.flatten()[:4], torch.tensor(rec["head"]), rtol=1e-4, atol=1e-7), name
