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


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("slices,shape", [(1, (7,)), (4, (33, 65)), (16, (512, 512)), (8, (3, 1376))])
def test_grad_sum_slices(dev, dtype, slices, shape):
    """Sum of the row-slice partial products in fp32 with one rounding, plain and added onto an existing gradient
    (vector path, odd sizes and the one-slice case)."""
    from maltos_amd import ops

    g = torch.Generator().manual_seed(slices * 131 + len(shape))
    parts = torch.randn(slices, *shape, generator=g).to(dtype)
    old = torch.randn(*shape, generator=g).to(dtype)
    got = ops.grad_sum_slices(parts.to(dev))
    want = parts.double().sum(0)
    # one final rounding to dtype plus, in fp32, one rounding per term of the running sum
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else (slices + 1) * 2.0 ** -24
    assert got.dtype == dtype and got.shape == tuple(shape)
    mag = parts.double().abs().sum(0)      # rounding of the running fp32 sum scales with the terms, not with the result
    assert ((got.double().cpu() - want).abs() <= ulp * mag + 1e-9).all()
    acc = old.to(dev).clone()
    assert ops.grad_sum_slices(parts.to(dev), acc, accumulate=True) is acc
    want_acc = want + old.double()
    assert ((acc.double().cpu() - want_acc).abs() <= ulp * (mag + old.double().abs()) + 1e-9).all()
    with pytest.raises(ValueError):
        ops.grad_sum_slices(parts.to(dev), accumulate=True)
    with pytest.raises(ValueError):
        ops.grad_sum_slices(parts.to(dev), torch.empty(3, device=dev, dtype=dtype))


@pytest.mark.parametrize("rows,out_f,in_f", [(4096, 256, 256), (512, 64, 96)])
def test_linear_accumulates_weight_grad_into_bound_buffer(dev, rows, out_f, in_f):
    """HipLinear with accumulate_into_grad adds dW into the existing gradient buffer (sliced and single-product
    forms) and leaves the same numbers as autograd's own accumulation, to one bf16 rounding."""
    from maltos_amd.llama import HipLinear, _weight_grad_splits

    assert (_weight_grad_splits(rows, out_f, in_f) > 1) == (rows == 4096)
    torch.manual_seed(3)
    plain = HipLinear(in_f, out_f, bias=False).to(dev).to(torch.bfloat16)
    fused = HipLinear(in_f, out_f, bias=False).to(dev).to(torch.bfloat16)
    fused.load_state_dict(plain.state_dict())
    fused.accumulate_into_grad = True
    start = (torch.randn(out_f, in_f, device=dev) * 0.5).to(torch.bfloat16)
    plain.weight.grad = start.clone()
    fused.weight.grad = start.clone()
    buffer_ptr = fused.weight.grad.data_ptr()
    x = torch.randn(rows, in_f, device=dev).to(torch.bfloat16)
    dy = (torch.randn(rows, out_f, device=dev) * 0.1).to(torch.bfloat16)
    grads = []
    for lin in (plain, fused):
        xi = x.clone().requires_grad_(True)
        lin(xi).backward(dy)
        grads.append(xi.grad)
    assert fused.weight.grad.data_ptr() == buffer_ptr
    assert torch.equal(grads[0], grads[1])
    exact = start.double() + dy.double().t() @ x.double()
    # both forms carry the bf16 rounding of the GEMM outputs; the fused one saves the rounding of `grad += dW`
    err_plain = (plain.weight.grad.double() - exact).abs()
    err_fused = (fused.weight.grad.double() - exact).abs()
    bound = 2.0 ** -7 * exact.abs().max()      # the partial products are of the size of the largest results
    assert err_plain.max() <= bound and err_fused.max() <= bound
    assert err_fused.mean() <= err_plain.mean() * 1.02
    # without a bound gradient the module falls back to returning dW
    fused.weight.grad = None
    xi = x.clone().requires_grad_(True)
    fused(xi).backward(dy)
    assert fused.weight.grad is not None and (fused.weight.grad.double() - (exact - start.double())).abs().max() < 0.5


def test_unused_parameter_is_skipped(dev):
    """A parameter that received no gradient: the reference leaves its master gradient at None and the inner optimizer
    skips it (runtime/optim.py:46-50).  MasterWeightsOptimizer does the same in both layouts: per parameter
    (flat=False) through `.grad is None`, flat (the default, every gradient bound to a buffer) through the record of
    whose gradient was written this step."""
    used = nn.Parameter(torch.randn(8, 16, device=dev).bfloat16())
    unused = nn.Parameter(torch.randn(4, 16, device=dev).bfloat16())
    shadow = [used.detach().float().clone().requires_grad_(True), unused.detach().float().clone().requires_grad_(True)]
    lib = torch.optim.AdamW(shadow, **HP)
    opt = MasterWeightsOptimizer([used, unused], optimizer_factory=lambda ps: FusedAdamW(ps, **HP), flat=False)
    before = unused.detach().clone()
    for _ in range(2):
        (used.float() ** 2).sum().backward()
        shadow[0].grad = used.grad.detach().float().clone()
        assert unused.grad is None
        opt.step()
        lib.step()
        opt.zero_grad(set_to_none=True)
        lib.zero_grad(set_to_none=True)
    assert torch.equal(unused.detach(), before)                      # never touched, like the library's
    torch.testing.assert_close(opt.master_params[0].detach(), shadow[0].detach(), rtol=1e-4, atol=1e-7)
    torch.testing.assert_close(opt.master_params[1].detach(), shadow[1].detach(), rtol=0, atol=0)
    # the flat layout (the default): the same against the library, over steps in which the second parameter is unused,
    # then used, then unused again (its step count and moments must follow the library's)
    torch.manual_seed(4)
    a = nn.Parameter(torch.randn(8, 16, device=dev).bfloat16())
    b = nn.Parameter(torch.randn(4, 16, device=dev).bfloat16())
    shadow = [a.detach().float().clone().requires_grad_(True), b.detach().float().clone().requires_grad_(True)]
    lib = torch.optim.AdamW(shadow, **HP)
    flat = MasterWeightsOptimizer([a, b], optimizer_factory=lambda ps: FusedAdamW(ps, **HP), flat=True)
    assert flat.flat_model_grad is not None
    for step, use_b in enumerate((False, True, False, False, True)):
        loss = (a.float() ** 2).sum() + ((b.float() * 3).sin().sum() if use_b else 0.0)
        loss.backward()
        shadow[0].grad = a.grad.detach().float().clone()
        shadow[1].grad = b.grad.detach().float().clone() if use_b else None
        b_before = flat.master_params[1].detach().clone()
        flat.step()
        lib.step()
        flat.zero_grad(set_to_none=True)
        lib.zero_grad(set_to_none=True)
        if not use_b:
            assert torch.equal(flat.master_params[1].detach(), b_before), f"step {step}: the unused parameter moved"
        for mp, sp, p_ in zip(flat.master_params, shadow, (a, b)):
            torch.testing.assert_close(mp.detach(), sp.detach(), rtol=1e-4, atol=1e-7)
            assert torch.equal(p_.detach(), mp.detach().to(torch.bfloat16))
    assert float(flat.state[flat.master_params[1]]["step"]) == 2.0 and float(flat.state[flat.master_params[0]]["step"]) == 5.0
    # gradients written by hand into the bound views are reported by hand
    b.grad.fill_(0.5)
    flat.mark_grads_written([b])
    b_before = flat.master_params[1].detach().clone()
    flat.step()
    assert not torch.equal(flat.master_params[1].detach(), b_before)
