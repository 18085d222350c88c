"""Pins oracle/layers.py and oracle/optim.py.

  * rms_norm                 : F.rms_norm (library routine) in fp32; in bf16 the double rounding is checked
                               against a literal evaluation; backward formula vs autograd.
  * rope                     : closed-form rotation on a hand-checked pair; invariants (norm preserving,
                               q.k depends only on the position difference, inverse rotation undoes it);
                               backward vs autograd.  The interleaved (LLaMA) convention is told apart from
                               rotate-half by a vector on which the two differ.
  * swiglu                   : F.silu * up (library); backward vs autograd.
  * causal_cross_entropy     : the reference's own test vectors (seed 123 logits, labels with one ignored)
                               against F.cross_entropy(mean); all-ignored gives exactly 0 and zero grads;
                               the explicit closed form vs autograd.
  * adamw_reference_step     : three steps of torch.optim.AdamW (library) on random data.
  * clip                     : torch.nn.utils.clip_grad_norm_ (library) to 1e-5, eps 1e-6 branch both ways,
                               FloatingPointError on inf.
  * master_weights_step      : the reference's resync scenario (bf16 zeros -> 3.0 survives a zero-grad step).
  * build_param_buckets      : greedy rule on hand-sized inputs, incl. an oversize parameter.
"""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import layers as ol
from oracle import optim as oo


def test_rmsnorm_matches_library_and_rounds_twice_in_bf16():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(7, 64, generator=g)
    w = 1 + 0.1 * torch.randn(64, generator=g)
    assert torch.allclose(ol.rms_norm(x, w, 1e-5), F.rms_norm(x, (64,), w, 1e-5), atol=1e-6)
    xb, wb = x.bfloat16(), w.bfloat16()
    r = torch.rsqrt(xb.float().pow(2).mean(-1, keepdim=True) + 1e-5)
    literal = (wb.float() * (xb.float() * r).bfloat16().float()).bfloat16()
    assert torch.equal(ol.rms_norm(xb, wb, 1e-5), literal)


def test_rmsnorm_backward_matches_autograd():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(5, 32, generator=g, requires_grad=True)
    w = (1 + 0.1 * torch.randn(32, generator=g)).requires_grad_(True)
    dy = torch.randn(5, 32, generator=g)
    ol.rms_norm(x, w, 1e-5).backward(dy)
    dx, dw = ol.rms_norm_backward(dy, x.detach(), w.detach(), 1e-5)
    assert torch.allclose(dx, x.grad, atol=1e-5) and torch.allclose(dw, w.grad, atol=1e-5)


def test_rope_closed_form_and_invariants():
    cos_t, sin_t = ol.rope_tables(4, 16, 10000.0)
    # theta_0 = 1, theta_1 = 10000^(-1/2) = 0.01
    assert math.isclose(cos_t[3, 0].item(), math.cos(3.0), rel_tol=1e-6)
    assert math.isclose(sin_t[3, 1].item(), math.sin(0.03), rel_tol=1e-5)
    x = torch.tensor([1.0, 0.0, 0.0, 2.0]).view(1, 1, 1, 4)
    cos, sin = ol.rope_cos_sin(cos_t, sin_t, seq_len=1, position_offset=3)
    y = ol.apply_rotary(x, cos, sin).flatten()
    # interleaved pairs (x0,x1) and (x2,x3); rotate-half would pair (x0,x2),(x1,x3) and give a different vector
    want = torch.tensor([math.cos(3.0), math.sin(3.0), -2 * math.sin(0.03), 2 * math.cos(0.03)])
    assert torch.allclose(y, want, atol=1e-6)
    g = torch.Generator().manual_seed(2)
    q = torch.randn(1, 2, 6, 8, generator=g)
    k = torch.randn(1, 2, 6, 8, generator=g)
    ct, st = ol.rope_tables(8, 64)
    c0, s0 = ol.rope_cos_sin(ct, st, seq_len=6, position_offset=0)
    c9, s9 = ol.rope_cos_sin(ct, st, seq_len=6, position_offset=9)
    q0, k0, q9, k9 = ol.apply_rotary(q, c0, s0), ol.apply_rotary(k, c0, s0), ol.apply_rotary(q, c9, s9), ol.apply_rotary(k, c9, s9)
    assert torch.allclose(q0.norm(dim=-1), q.norm(dim=-1), atol=1e-5)
    assert torch.allclose(q0 @ k0.transpose(-1, -2), q9 @ k9.transpose(-1, -2), atol=1e-4)
    assert torch.allclose(ol.apply_rotary_backward(q0, c0, s0), q, atol=1e-5)
    # position_ids gather == slice
    cp, sp = ol.rope_cos_sin(ct, st, seq_len=6, position_ids=torch.arange(9, 15))
    assert torch.equal(cp, c9) and torch.equal(sp, s9)


def test_rope_backward_matches_autograd():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 2, 5, 8, generator=g, requires_grad=True)
    dy = torch.randn(2, 2, 5, 8, generator=g)
    ct, st = ol.rope_tables(8, 32)
    c, s = ol.rope_cos_sin(ct, st, seq_len=5, position_ids=torch.tensor([[0, 1, 2, 0, 1], [3, 4, 5, 6, 7]]))
    ol.apply_rotary(x, c, s).backward(dy)
    assert torch.allclose(ol.apply_rotary_backward(dy, c, s), x.grad, atol=1e-6)


def test_swiglu_forward_and_backward():
    g = torch.Generator().manual_seed(4)
    a = torch.randn(6, 10, generator=g, requires_grad=True)
    b = torch.randn(6, 10, generator=g, requires_grad=True)
    d = torch.randn(6, 10, generator=g)
    out = ol.swiglu(a, b)
    assert torch.equal(out, F.silu(a) * b)
    out.backward(d)
    dg, du = ol.swiglu_backward(d, a.detach(), b.detach())
    assert torch.allclose(dg, a.grad, atol=1e-6) and torch.allclose(du, b.grad, atol=1e-6)


def test_causal_cross_entropy_reference_vectors(known_answers):
    ka = known_answers["causal_loss"]
    torch.manual_seed(ka["seed"])
    logits = torch.randn(*ka["logits_shape"], requires_grad=True)
    labels = torch.tensor(ka["labels"])
    actual = ol.causal_cross_entropy(logits, labels)
    expected = F.cross_entropy(logits.view(-1, 5), labels.view(-1), ignore_index=-100)
    torch.testing.assert_close(actual, expected)
    actual.backward()
    loss2, grad2 = ol.causal_cross_entropy_explicit(logits.detach(), labels)
    assert torch.allclose(loss2, actual.detach(), atol=1e-6) and torch.allclose(grad2, logits.grad, atol=1e-6)
    # no targets: finite, exactly zero, zero grads
    lg = torch.randn(2, 3, 5, requires_grad=True)
    none = torch.full((2, 3), -100)
    loss = ol.causal_cross_entropy(lg, none)
    assert torch.isfinite(loss) and loss.item() == 0.0
    loss.backward()
    torch.testing.assert_close(lg.grad, torch.zeros_like(lg))
    l0, g0 = ol.causal_cross_entropy_explicit(lg.detach(), none)
    assert l0.item() == 0.0 and not g0.any()


def test_adamw_closed_form_matches_library():
    g = torch.Generator().manual_seed(5)
    p0 = torch.randn(257, generator=g)
    hp = dict(lr=3e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
    ref = torch.nn.Parameter(p0.clone())
    opt = torch.optim.AdamW([ref], lr=hp["lr"], betas=(hp["beta1"], hp["beta2"]), eps=hp["eps"], weight_decay=hp["weight_decay"])
    p, m, v = p0.clone(), torch.zeros(257), torch.zeros(257)
    for step in (1, 2, 3):
        grad = torch.randn(257, generator=g)
        ref.grad = grad.clone()
        opt.step()
        p, m, v = oo.adamw_reference_step(p, grad, m, v, step=step, **hp)
        assert torch.allclose(p, ref.detach(), rtol=1e-6, atol=1e-7)
    st = opt.state[ref]
    assert torch.allclose(m, st["exp_avg"], atol=1e-7) and torch.allclose(v, st["exp_avg_sq"], atol=1e-8)


@pytest.mark.parametrize("scale", [10.0, 1e-3])
def test_clip_matches_library(known_answers, scale):
    g = torch.Generator().manual_seed(6)
    grads = [torch.randn(33, generator=g) * scale, torch.randn(4, 9, generator=g) * scale]
    params = [torch.nn.Parameter(torch.zeros_like(t)) for t in grads]
    for p, t in zip(params, grads):
        p.grad = t.clone()
    ref_norm = torch.nn.utils.clip_grad_norm_(params, 1.0)
    mine = [t.clone() for t in grads]
    norm = oo.clip_grads_(mine, 1.0)
    atol = known_answers["tolerances"]["clip_atol"]
    assert abs(norm - ref_norm.item()) < atol * max(1.0, norm)
    for a, p in zip(mine, params):
        assert torch.allclose(a, p.grad, atol=atol)
    assert (oo.clip_coefficient(norm, 1.0) < 1.0) == (scale > 1.0)
    with pytest.raises(FloatingPointError):
        oo.clip_coefficient(float("inf"), 1.0)


def test_master_weights_resync_scenario():
    model_param = torch.nn.Parameter(torch.zeros(4, dtype=torch.bfloat16))
    master = torch.nn.Parameter(model_param.detach().float())
    inner = torch.optim.SGD([master], lr=1.0)
    with torch.no_grad():
        model_param.fill_(3.0)
        master.copy_(model_param.float())  # sync_master_params_from_model
    model_param.grad = torch.zeros_like(model_param)
    oo.master_weights_step([model_param], [master], inner)
    torch.testing.assert_close(model_param, torch.full_like(model_param, 3.0))


def test_bucket_builder_greedy_rule():
    mib = 1024 * 1024
    assert oo.build_param_buckets([10 * mib, 10 * mib, 10 * mib, 1 * mib], 25 * mib) == [[0, 1], [2, 3]]
    assert oo.build_param_buckets([30 * mib, 1 * mib], 25 * mib) == [[0], [1]]  # oversize parameter stands alone
    assert oo.build_param_buckets([], 25 * mib) == []
    assert oo.padded_len(10, 4) == 12 and oo.padded_len(8, 4) == 8
