"""GPU tests of the optimizer side: FusedAdamW as an optimizer_factory product, the flat
MasterWeightsOptimizer layout, global-norm clipping (host-read and fully fused forms), state_dict
round trips.  Checked against torch.optim.AdamW / clip_grad_norm_ (library) and the oracle's closed forms."""
import copy

import pytest
import torch
import torch.nn as nn

from maltos_amd.grad_clip import clip_grad_norm_, clip_grad_norm_fused_
from maltos_amd.optim import FusedAdamW, MasterWeightsOptimizer
from oracle import optim as oo

pytestmark = pytest.mark.gpu

HP = dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)


def _model(dev, dtype):
    torch.manual_seed(0)
    m = nn.Sequential(nn.Linear(24, 40, bias=True), nn.Linear(40, 8, bias=False), nn.LayerNorm(8)).to(dev)
    return m.to(dtype)


def _loss(model, x):
    return model(x).float().pow(2).mean()


def test_fused_adamw_matches_library_fp32(dev):
    ref_model, my_model = _model(dev, torch.float32), _model(dev, torch.float32)
    ref = torch.optim.AdamW(ref_model.parameters(), **HP)
    mine = FusedAdamW(my_model.parameters(), **HP)
    sched = torch.optim.lr_scheduler.LambdaLR(mine, lambda s: 1.0 / (1 + s))  # lr must be re-read every step
    ref_sched = torch.optim.lr_scheduler.LambdaLR(ref, lambda s: 1.0 / (1 + s))
    for step in range(4):
        x = torch.randn(16, 24, device=dev, generator=torch.Generator(device=dev).manual_seed(step))
        for model, opt, sc in ((ref_model, ref, ref_sched), (my_model, mine, sched)):
            _loss(model, x).backward()
            opt.step()
            sc.step()
            opt.zero_grad(set_to_none=True)
        for a, b in zip(ref_model.parameters(), my_model.parameters()):
            torch.testing.assert_close(a, b, rtol=1e-4, atol=1e-7)
    sd = mine.state_dict()
    assert set(sd["state"][0]) == {"step", "exp_avg", "exp_avg_sq"} and float(sd["state"][0]["step"]) == 4.0
    # a stock AdamW accepts the state and continues identically
    clone_model = copy.deepcopy(my_model)
    stock = torch.optim.AdamW(clone_model.parameters(), **HP)
    stock.load_state_dict(copy.deepcopy(sd))
    fresh = FusedAdamW(my_model.parameters(), **HP)
    fresh.load_state_dict(copy.deepcopy(sd))
    x = torch.randn(16, 24, device=dev)
    for model, opt in ((clone_model, stock), (my_model, fresh)):
        _loss(model, x).backward()
        opt.step()
    for a, b in zip(clone_model.parameters(), my_model.parameters()):
        torch.testing.assert_close(a, b, rtol=1e-4, atol=1e-7)


@pytest.mark.parametrize("inner", ["fused", "stock"])
@pytest.mark.parametrize("flat", [True, False])
def test_master_weights_optimizer_bf16(dev, inner, flat):
    """bf16 model, fp32 masters: equals the reference recipe (upcast grads, stock AdamW on masters, round back)."""
    model = _model(dev, torch.bfloat16)
    shadow = [p.detach().float().clone().requires_grad_(True) for p in model.parameters()]
    lib = torch.optim.AdamW(shadow, **HP)
    factory = (lambda ps: FusedAdamW(ps, **HP)) if inner == "fused" else (lambda ps: torch.optim.AdamW(ps, **HP))
    opt = MasterWeightsOptimizer(model.parameters(), optimizer_factory=factory, flat=flat)
    assert opt.model_param_for(opt.master_params[1]) is list(model.parameters())[1]
    assert all(mp.dtype == torch.float32 for mp in opt.master_params)
    for step in range(3):
        x = torch.randn(16, 24, device=dev, dtype=torch.bfloat16, generator=torch.Generator(device=dev).manual_seed(step))
        _loss(model, x).backward()
        for s, p in zip(shadow, model.parameters()):
            s.grad = p.grad.detach().float().clone()
        opt.step()
        lib.step()
        opt.zero_grad(set_to_none=True)
        for s, mp, p in zip(shadow, opt.master_params, model.parameters()):
            torch.testing.assert_close(mp.detach(), s.detach(), rtol=1e-4, atol=1e-7)
            assert torch.equal(p.detach(), mp.detach().to(torch.bfloat16))
    sd = opt.state_dict()
    assert set(sd) == {"inner_optimizer", "master_params", "master_dtype"}
    assert sd["master_dtype"] == "torch.float32" and all(not t.is_cuda for t in sd["master_params"])
    with torch.no_grad():
        for p in model.parameters():
            p.add_(1.0)
    opt.load_state_dict(sd)
    for s, p in zip(shadow, model.parameters()):
        assert torch.equal(p.detach(), s.detach().to(torch.bfloat16))


def test_resync_scenario_on_gpu(dev):
    p = nn.Parameter(torch.zeros(4, dtype=torch.bfloat16, device=dev))
    opt = MasterWeightsOptimizer([p], optimizer_factory=lambda ps: FusedAdamW(ps, lr=1.0, weight_decay=0.0))
    with torch.no_grad():
        p.fill_(3.0)
    opt.sync_master_params_from_model()
    opt.zero_grad()
    opt.step()  # zero gradient: the update is 0 / (0 + eps) = 0
    torch.testing.assert_close(p.detach(), torch.full_like(p, 3.0))


@pytest.mark.parametrize("scale", [50.0, 1e-3])
def test_clip_matches_library(dev, scale, known_answers):
    model = _model(dev, torch.bfloat16)
    opt = MasterWeightsOptimizer(model.parameters(), optimizer_factory=lambda ps: FusedAdamW(ps, **HP))
    x = torch.randn(16, 24, device=dev, dtype=torch.bfloat16)
    (scale * _loss(model, x)).backward()
    ref_grads = [p.grad.detach().float().clone() for p in model.parameters()]
    ref_params = [nn.Parameter(torch.zeros_like(g)) for g in ref_grads]
    for rp, g in zip(ref_params, ref_grads):
        rp.grad = g.clone()
    want_norm = torch.nn.utils.clip_grad_norm_(ref_params, 1.0).item()
    norm = clip_grad_norm_(opt, 1.0)
    atol = known_answers["tolerances"]["clip_atol"]
    assert abs(norm - want_norm) <= atol * max(1.0, want_norm)
    assert (norm > 1.0) == (scale > 1.0)
    assert abs(norm - oo.global_grad_norm(ref_grads)) <= 1e-9 * max(1.0, norm)
    for mp, rp in zip(opt.master_params, ref_params):
        torch.testing.assert_close(mp.grad, rp.grad, rtol=1e-5, atol=atol)


def test_fused_clip_equals_clip_then_step(dev):
    m1, m2 = _model(dev, torch.bfloat16), _model(dev, torch.bfloat16)
    o1 = MasterWeightsOptimizer(m1.parameters(), optimizer_factory=lambda ps: FusedAdamW(ps, **HP))
    o2 = MasterWeightsOptimizer(m2.parameters(), optimizer_factory=lambda ps: FusedAdamW(ps, **HP))
    x = torch.randn(16, 24, device=dev, dtype=torch.bfloat16)
    (50 * _loss(m1, x)).backward()
    (50 * _loss(m2, x)).backward()
    n1 = clip_grad_norm_(o1, 1.0)
    sq = clip_grad_norm_fused_(o2, 1.0)
    assert n1 > 1.0 and abs(float(sq.sqrt()) - n1) <= 1e-9 * n1
    o1.step()
    o2.step()
    for a, b in zip(o1.master_params, o2.master_params):
        assert torch.equal(a.detach(), b.detach())
    for a, b in zip(m1.parameters(), m2.parameters()):
        assert torch.equal(a.detach(), b.detach())


def test_non_finite_norm_raises(dev):
    model = _model(dev, torch.float32)
    opt = FusedAdamW(model.parameters(), **HP)
    _loss(model, torch.randn(4, 24, device=dev)).backward()
    next(model.parameters()).grad[0, 0] = float("inf")
    with pytest.raises(FloatingPointError):
        clip_grad_norm_(opt, 1.0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_zero1_flat_buffers_step_equals_plain_optimizer(dev, dtype):
    """The fused optimizer inside the ZeRO-1 layout (reverse-order buckets, flat data/grad buffers, per-bucket local
    shards; world_size 1) takes the same steps as the same optimizer on the model's own parameters: AdamW is
    elementwise, so only the clip coefficient (an fp64 sum in another order) can differ, in its last bits."""
    from maltos_amd.zero1 import Zero1FlatBuffers

    plain_model = _model(dev, dtype)
    zero_model = copy.deepcopy(plain_model)
    inner = lambda ps: FusedAdamW(ps, **HP)
    factory = (lambda ps: MasterWeightsOptimizer(ps, optimizer_factory=inner)) if dtype == torch.bfloat16 else inner
    plain = factory(list(plain_model.parameters()))
    z = Zero1FlatBuffers(zero_model, optimizer_factory=factory, bucket_mb_size=25)
    assert sum(len(b.params) for b in z.buckets) == len(list(zero_model.parameters()))
    max_norm = 0.5
    for step in range(3):
        x = torch.randn(16, 24, device=dev, dtype=dtype, generator=torch.Generator(device=dev).manual_seed(step))
        _loss(plain_model, x).backward()
        want_norm = clip_grad_norm_(plain, max_norm)
        plain.step()
        plain.zero_grad(set_to_none=True)
        z.reset_grads()
        _loss(zero_model, x).backward()
        got_norm = z.step(max_norm)
        assert got_norm == pytest.approx(want_norm, rel=1e-6)
        for p, q in zip(zero_model.parameters(), plain_model.parameters()):
            assert p.data_ptr() >= z.data_buffer.data_ptr()  # still a view of the flat buffer
            torch.testing.assert_close(p.detach().float(), q.detach().float(), rtol=1e-5 if dtype == torch.float32 else 2 ** -7, atol=1e-7)
