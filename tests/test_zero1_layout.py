"""ZeRO-1 flat-buffer layout and step phases (maltos_amd/zero1.py) on the CPU.

The layout rules come from runtime/plugins/zero1.py:98-164 and zero_common.py:176-193, 293-302 of the reference.  They are
pinned here by what they must satisfy rather than by a second copy of the same loops: every trainable parameter
appears exactly once, in reverse registration order; a bucket only exceeds the byte limit when it holds a single
parameter and closing it earlier would not have helped; bucket lengths are multiples of the world size; the ranks'
shards tile every bucket; the parameters are views of the flat buffers.  One known answer comes from the reference's
own LLaMA-50M recipe: the two 32.8 MB vocabulary matrices are larger than the 25 MiB limit and get buckets of their
own.  The step phases are checked against torch.optim.AdamW + clip_grad_norm_ on unsharded copies of the model.
"""
import copy

import pytest
import torch
import torch.nn as nn

from maltos_amd.zero1 import Zero1FlatBuffers, build_param_buckets, padded_len, role_params


def _toy(seed=0, dtype=torch.float32):
    torch.manual_seed(seed)
    model = nn.Sequential(nn.Linear(7, 13), nn.Tanh(), nn.Linear(13, 5, bias=False), nn.Linear(5, 3))
    model[2].weight.requires_grad_(False)  # frozen parameters stay out of the buffers
    return model.to(dtype)


def test_padded_len():
    assert [padded_len(n, 4) for n in (0, 1, 4, 5, 8)] == [0, 4, 4, 8, 8]
    assert padded_len(10, 1) == 10


@pytest.mark.parametrize("limit", [1, 64, 400, 10 ** 9])
def test_buckets_are_greedy_and_cover_everything_in_order(limit):
    gen = torch.Generator().manual_seed(limit)
    params = [nn.Parameter(torch.zeros(int(n))) for n in torch.randint(1, 60, (40,), generator=gen)]
    buckets = build_param_buckets(params, limit)
    flat = [p for b in buckets for p in b]
    assert len(flat) == len(params) and all(a is b for a, b in zip(flat, params))
    size = lambda b: sum(p.numel() * p.element_size() for p in b)
    for i, b in enumerate(buckets):
        assert b and (size(b) <= limit or len(b) == 1)
        if i + 1 < len(buckets):  # greedy: the next parameter did not fit any more
            nxt = buckets[i + 1][0]
            assert size(b) + nxt.numel() * nxt.element_size() > limit


@pytest.mark.parametrize("world_size", [1, 2, 4])
def test_flat_buffers_alias_the_model_and_shards_tile_the_buckets(world_size):
    reference = _toy()
    for rank in range(world_size):
        model = copy.deepcopy(reference)
        noop = lambda *a: None
        z = Zero1FlatBuffers(model, optimizer_factory=lambda ps: torch.optim.SGD(ps, lr=0.1), world_size=world_size, rank=rank,
                             bucket_mb_size=25, reduce_scatter_avg=noop, all_gather=noop, all_reduce_sum=noop)
        trainable = [p for p in model.parameters() if p.requires_grad]
        assert [p for b in z.buckets for p in b.params] == trainable[::-1] == role_params(model)
        names = dict(model.named_parameters())
        assert all(names[n] is p for b in z.buckets for n, p in zip(b.logical_names, b.params))
        cursor = 0
        for b in z.buckets:
            assert b.start == cursor and (b.end - b.start) % world_size == 0
            assert b.end - b.start == padded_len(sum(p.numel() for p in b.params), world_size)
            per_rank = (b.end - b.start) // world_size
            assert (b.shard_start, b.shard_end) == (b.start + rank * per_rank, b.start + (rank + 1) * per_rank)
            off = b.start
            for p in b.params:  # views of the flat buffers, values preserved
                assert p.data_ptr() == z.data_buffer[off:].data_ptr() and p.grad.data_ptr() == z.grad_buffer[off:].data_ptr()
                off += p.numel()
            assert torch.equal(z.data_buffer[off:b.end], torch.zeros(b.end - off))  # padding
            assert torch.equal(b.local_param.detach(), z.data_buffer[b.shard_start:b.shard_end])
            assert b.local_param.data_ptr() != z.data_buffer[b.shard_start:].data_ptr()  # a clone, not a view
            cursor = b.end
        assert cursor == z.data_buffer.numel() == z.grad_buffer.numel()
        for p, q in zip(model.parameters(), reference.parameters()):
            assert torch.equal(p, q)
        assert not any(model[2].weight is p for b in z.buckets for p in b.params)


def test_llama50m_vocabulary_matrices_get_buckets_of_their_own():
    from maltos_amd.llama import LlamaConfig, LlamaForCausalLM

    cfg = LlamaConfig(vocab_size=32000, hidden_size=512, intermediate_size=1376, num_hidden_layers=8, num_attention_heads=8,
                      max_position_embeddings=2048, rms_norm_eps=1e-5, attention_backend="eager")
    with torch.device("meta"):
        model = LlamaForCausalLM(cfg).to(torch.bfloat16)
    buckets = build_param_buckets(role_params(model), 25 * 1024 * 1024)
    names = {id(p): n for n, p in model.named_parameters()}
    big = [b for b in buckets if any(p.numel() == 32000 * 512 for p in b)]
    assert len(big) == 2 and all(len(b) == 1 for b in big)
    assert 4 <= len(buckets) <= 5
    assert names[id(buckets[0][0])] == "lm_head.weight"          # reverse order: the head first ...
    assert names[id(buckets[-1][0])] == "embed_tokens.weight"  # ... the embedding last
    assert sum(p.numel() for b in buckets for p in b) * 2 == pytest.approx(116e6, rel=0.01)


@pytest.mark.parametrize("world_size", [1, 2])
def test_step_phases_equal_unsharded_adamw_with_clipping(world_size):
    """Ranks are emulated in one process: the transport callables read the other rank's buffers directly."""
    hp = dict(lr=1e-2, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    max_norm = 0.05
    base = _toy(3)
    ranks, models, bus = [], [], {}
    for rank in range(world_size):
        model = copy.deepcopy(base)
        models.append(model)

        def reduce_scatter_avg(out, full_grad, rank=rank):
            z = ranks[rank]
            b = next(b for b in z.buckets if b.local_param.grad is out)
            mean = sum(r.grad_buffer[b.start:b.end] for r in ranks) / world_size
            out.copy_(mean[b.shard_start - b.start:b.shard_end - b.start])

        def all_gather(out_full, local, rank=rank):
            z = ranks[rank]
            b = next(b for b in z.buckets if z.data_buffer[b.start:].data_ptr() == out_full.data_ptr())
            i = z.buckets.index(b)
            out_full.copy_(torch.cat([r.buckets[i].local_param.detach() for r in ranks]))

        def all_reduce_sum(t, rank=rank):
            t.copy_(bus["sq"])  # summed before any rank scales its shard: the emulated ranks run one after the other

        ranks.append(Zero1FlatBuffers(model, optimizer_factory=lambda ps: torch.optim.AdamW(ps, **hp), world_size=world_size,
                                      rank=rank, bucket_mb_size=25, reduce_scatter_avg=reduce_scatter_avg, all_gather=all_gather,
                                      all_reduce_sum=all_reduce_sum))
    plain = copy.deepcopy(base)
    plain_opt = torch.optim.AdamW([p for p in plain.parameters() if p.requires_grad], **hp)
    gen = torch.Generator().manual_seed(9)
    for step in range(3):
        xs = [torch.randn(6, 7, generator=gen) for _ in range(world_size)]
        # sharded: every rank its own micro-batch; unsharded: the mean loss over all of them
        for z, model, x in zip(ranks, models, xs):
            z.reset_grads()
            model(x).pow(2).sum().backward()
        plain_opt.zero_grad()
        (sum(plain(x).pow(2).sum() for x in xs) / world_size).backward()
        want_norm = float(torch.nn.utils.clip_grad_norm_([p for p in plain.parameters() if p.requires_grad], max_norm))
        plain_opt.step()
        for z in ranks:
            z.reduce_grads()
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
            assert all(p.grad.abs().max() == 0 for p in model.parameters() if p.requires_grad)  # grads zeroed, views kept


def test_sync_local_params_after_load_and_non_finite_norm():
    model = _toy(5)
    z = Zero1FlatBuffers(model, optimizer_factory=lambda ps: torch.optim.SGD(ps, lr=0.1))
    with torch.no_grad():
        for p in model.parameters():
            p.add_(1.0)  # a checkpoint load writes through the views into the data buffer
    z.sync_local_params_from_data_buffer()
    for b in z.buckets:
        assert torch.equal(b.local_param.detach(), z.data_buffer[b.shard_start:b.shard_end])
    model(torch.randn(2, 7)).sum().backward()
    z.grad_buffer[0] = float("inf")
    z.reduce_grads()
    with pytest.raises(FloatingPointError, match="non-finite ZeRO gradient norm"):
        z.clip_local_shards(1.0)
    with pytest.raises(ValueError):
        Zero1FlatBuffers(_toy(), optimizer_factory=lambda ps: torch.optim.SGD(ps, lr=0.1), world_size=2, rank=0)
