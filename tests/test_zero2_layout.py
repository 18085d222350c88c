"""ZeRO-2 per-bucket gradient buffers and step phases (maltos_amd/zero2.py) on the CPU.

What runtime/plugins/zero2.py:107-395 of the reference must do is pinned by behaviour: the parameters' gradients
are views of the bucket's exec-state buffer from the first gradient of a backward on; a bucket's reduction fires inside
the backward pass, when its last gradient has been accumulated, the buckets in the order their gradients complete (last
layers first); buckets whose parameters took no part are reduced at the wait; micro-steps of an accumulation window add
up in the shards' gradients; and the whole step equals torch.optim.AdamW + clip_grad_norm_ on an unsharded copy of the
model, for one rank and for two emulated ranks, with one and with two exec states per bucket.
"""
import copy

import pytest
import torch
import torch.nn as nn

from maltos_amd.zero1 import Zero1FlatBuffers
from maltos_amd.zero2 import Zero2FlatBuffers


def _toy(seed=0):
    torch.manual_seed(seed)
    return nn.Sequential(nn.Linear(7, 13), nn.Tanh(), nn.Linear(13, 11), nn.Tanh(), nn.Linear(11, 3))


def _tiny_buckets(model, **kw):
    # 600-byte buckets, parameters in reverse registration order: [4.bias, 4.weight, 2.bias], [2.weight], [0.bias, 0.weight]
    return Zero2FlatBuffers(model, optimizer_factory=lambda ps: torch.optim.SGD(ps, lr=0.1), bucket_mb_size=600 / 2 ** 20, **kw)


def test_layout_is_the_zero1_layout_without_a_whole_model_gradient_buffer():
    a, b = _toy(), _toy()
    z1 = Zero1FlatBuffers(a, optimizer_factory=lambda ps: torch.optim.SGD(ps, lr=0.1), bucket_mb_size=600 / 2 ** 20, world_size=2, rank=1,
                          reduce_scatter_avg=lambda *_: None, all_gather=lambda *_: None, all_reduce_sum=lambda *_: None)
    z2 = _tiny_buckets(b, world_size=2, rank=1, microbatches=3, reduce_scatter_avg=lambda *_: None, all_gather=lambda *_: None,
                       all_reduce_sum=lambda *_: None)
    assert z2.grad_buffer is None and torch.equal(z1.data_buffer, z2.data_buffer)
    assert len(z2.buckets) == len(z1.buckets) == 3
    for b1, b2 in zip(z1.buckets, z2.buckets):
        assert (b1.start, b1.end, b1.shard_start, b1.shard_end, b1.logical_names) == (b2.start, b2.end, b2.shard_start, b2.shard_end, b2.logical_names)
        assert len(b2.exec_states) == 3
        for state in b2.exec_states:
            assert state.grad_buffer.numel() == b2.end - b2.start and state.shard_buffer.numel() == b2.local_param.numel()
    assert all(p.grad is None for p in b.parameters())


def test_gradients_land_in_the_bucket_buffers_and_buckets_fire_inside_backward():
    model = _toy(1)
    z = _tiny_buckets(model)
    plain = copy.deepcopy(model)
    for p in plain.parameters():
        p.grad = None
    x = torch.randn(5, 7, generator=torch.Generator().manual_seed(2))
    fired_when = []
    # a probe on the first layer's output: its gradient is computed after the two later layers' parameters are complete
    hidden = model[1](model[0](x))
    hidden.register_hook(lambda g: fired_when.append(list(z.fired_order)))
    model[4](model[3](model[2](hidden))).pow(2).sum().backward()
    plain(x).pow(2).sum().backward()
    assert fired_when == [[0, 1]]            # the last two layers' buckets were reduced before the first layer's backward ran
    assert z.fired_order == [0, 1, 2]
    for bucket in z.buckets:
        state = bucket.exec_states[0]
        offset = 0
        for p in bucket.params:
            assert p.grad.data_ptr() == state.grad_buffer[offset:].data_ptr()
            offset += p.numel()
        assert bucket.pending_exec_reductions == 0 and state.pending == 0
        assert torch.equal(state.shard_buffer, state.grad_buffer[:bucket.local_param.numel()])
    for p, q in zip(model.parameters(), plain.parameters()):
        assert torch.equal(p.grad, q.grad)
    z.wait_grad_sync()
    for bucket in z.buckets:
        assert torch.equal(bucket.local_param.grad, bucket.exec_states[0].grad_buffer)


def test_bucket_with_an_unused_parameter_is_reduced_at_the_wait():
    model = _toy(3)
    z = _tiny_buckets(model)
    x = torch.randn(4, 7, generator=torch.Generator().manual_seed(4))
    model[2](model[1](model[0](x))).sum().backward()   # the last layer takes no part
    assert z.fired_order == [1, 2] and z.buckets[0].exec_states[0].pending == 2
    z.wait_grad_sync()
    assert z.fired_order == [1, 2, 0]
    g0 = z.buckets[0].local_param.grad
    assert g0[:36].abs().max() == 0 and torch.equal(g0[36:], torch.full((11,), 4.0))   # layer 4 untouched, 2.bias = batch size
    assert z.buckets[1].local_param.grad.abs().max() > 0


@pytest.mark.parametrize("world_size,microbatches", [(1, 1), (2, 1), (2, 2)])
def test_step_phases_equal_unsharded_adamw_with_clipping_and_accumulation(world_size, microbatches):
    """Ranks are emulated in one process: the transport callables read the other ranks' buffers directly.  Two micro-steps
    per optimizer step; with two exec states the micro-steps fill different states (as two micro-batches of a pipeline
    schedule do) and both are taken in at the wait."""
    hp = dict(lr=1e-2, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    max_norm, micro_steps = 0.05, 2
    base = _toy(3)
    ranks, models, bus = [], [], {}
    for rank in range(world_size):
        model = copy.deepcopy(base)
        models.append(model)

        def reduce_scatter_avg(out, full_grad, rank=rank):
            z = ranks[rank]
            i, s = next((i, s) for i, b in enumerate(z.buckets) for s, st in enumerate(b.exec_states) if st.shard_buffer is out)
            b = z.buckets[i]
            mean = sum(r.buckets[i].exec_states[s].grad_buffer for r in ranks) / world_size
            out.copy_(mean[b.shard_start - b.start:b.shard_end - b.start])

        def all_gather(out_full, local, rank=rank):
            z = ranks[rank]
            i = next(i for i, b in enumerate(z.buckets) if z.data_buffer[b.start:].data_ptr() == out_full.data_ptr())
            out_full.copy_(torch.cat([r.buckets[i].local_param.detach() for r in ranks]))

        def all_reduce_sum(t, rank=rank):
            t.copy_(bus["sq"])

        ranks.append(Zero2FlatBuffers(model, optimizer_factory=lambda ps: torch.optim.AdamW(ps, **hp), world_size=world_size,
                                      rank=rank, bucket_mb_size=600 / 2 ** 20, microbatches=microbatches,
                                      reduce_scatter_avg=reduce_scatter_avg if world_size > 1 else None,
                                      all_gather=all_gather if world_size > 1 else None,
                                      all_reduce_sum=all_reduce_sum if world_size > 1 else None))
    plain = copy.deepcopy(base)
    plain_opt = torch.optim.AdamW(plain.parameters(), **hp)
    gen = torch.Generator().manual_seed(9)
    for step in range(3):
        plain_opt.zero_grad()
        for micro in range(micro_steps):
            xs = [torch.randn(6, 7, generator=gen) for _ in range(world_size)]
            (sum(plain(x).pow(2).sum() for x in xs) / world_size).backward()
            # emulated ranks run one after the other, so a bucket's reduction must not fire before every rank has its
            # gradients: run all backward passes with the reductions held back, then let the wait fire them
            for z, model, x in zip(ranks, models, xs):
                z.microbatch_index = micro % microbatches
                z.reset_buckets(grad_accum_start=micro == 0)
            if world_size > 1:
                for z in ranks:
                    for b in z.buckets:
                        z._exec_state(b).pending += 10 ** 6   # hold the in-backward reductions back (see above)
            for z, model, x in zip(ranks, models, xs):
                model(x).pow(2).sum().backward()
            # one rank: the reductions fired inside the backward pass, and a micro-step that is not the last leaves them to
            # the next reset, which takes them in before it clears the state (the reference waits only at a step boundary)
            if micro == micro_steps - 1 or (world_size > 1 and microbatches == 1):
                for z in ranks:
                    z.wait_grad_sync()
        want_norm = float(torch.nn.utils.clip_grad_norm_(plain.parameters(), max_norm))
        plain_opt.step()
        bus["sq"] = sum(z.local_sq_norm() for z in ranks)
        norms = [z.clip_local_shards(max_norm) for z in ranks]
        for z in ranks:
            z.optimizer.step()
        for z in ranks:
            z.gather_updated_params()
        assert all(n == pytest.approx(want_norm, rel=1e-6) for n in norms)
        for model in models:
            for p, q in zip(model.parameters(), plain.parameters()):
                assert torch.allclose(p, q, rtol=1e-5, atol=1e-7), step


class _LinearIntoGrad(torch.autograd.Function):
    """x W^T whose backward adds dW into W.grad itself and hands autograd None for W (what HipLinear.accumulate_into_grad does)."""

    @staticmethod
    def forward(ctx, x, w, b):
        ctx.save_for_backward(x, w)
        return torch.nn.functional.linear(x, w, b)

    @staticmethod
    def backward(ctx, dy):
        x, w = ctx.saved_tensors
        if w.grad is None:
            return dy @ w, dy.t() @ x, dy.sum(0)
        w.grad.add_(dy.t() @ x)
        return dy @ w, None, dy.sum(0)


def test_gradients_added_into_the_buffers_by_the_backward_function_still_complete_their_bucket():
    model = _toy(6)
    z = _tiny_buckets(model)
    x = torch.randn(4, 7, generator=torch.Generator().manual_seed(4))

    def forward(m):
        h = x
        for layer in m:
            h = _LinearIntoGrad.apply(h, layer.weight, layer.bias) if isinstance(layer, nn.Linear) else layer(h)
        return h.pow(2).sum()

    plain = copy.deepcopy(model)
    for p in plain.parameters():
        p.grad = None
    forward(plain).backward()
    for step in range(2):   # first pass: the gradients are unbound and go through autograd; second pass: added in place
        z.reset_buckets(grad_accum_start=True)
        forward(model).backward()
        assert sorted(z.fired_order[:2]) == [0, 1] and z.fired_order[2:] == [2], step   # all inside the backward pass
        z.wait_grad_sync()
        for bucket in z.buckets:
            offset = 0
            for name, p in zip(bucket.logical_names, bucket.params):
                assert torch.equal(bucket.local_param.grad[offset:offset + p.numel()].view_as(p), dict(plain.named_parameters())[name].grad), (step, name)
                offset += p.numel()
    z.remove_hooks()
    z.reset_buckets(grad_accum_start=True)
    forward(model).backward()
    assert z.fired_order == []
