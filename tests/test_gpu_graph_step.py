"""Forward + backward replayed from a HIP graph against the same steps run eagerly.

Every replay is checked (not only the first), with unrelated eager GPU work and a device synchronisation between the
replays, on different batches, through the real clip + fused AdamW step, so stale or wrongly re-used graph memory
would show up as a loss or parameter difference.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _make(dev, dtype, seed=11):
    from maltos_amd.llama import LlamaConfig, LlamaForCausalLM
    from maltos_amd.optim import FusedAdamW, MasterWeightsOptimizer

    cfg = LlamaConfig(vocab_size=1024, hidden_size=256, intermediate_size=688, num_hidden_layers=2, num_attention_heads=4,
                      max_position_embeddings=1024, rms_norm_eps=1e-5)
    torch.manual_seed(seed)
    model = LlamaForCausalLM(cfg)
    with torch.no_grad():
        for p in model.parameters():
            if p.dim() >= 2:
                p.normal_(0.0, 0.02)
    model = model.to(dev).to(dtype)
    opt = MasterWeightsOptimizer(model.parameters(), optimizer_factory=lambda ps: FusedAdamW(
        ps, lr=1e-2, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1))
    return cfg, model, opt


def _batches(cfg, dev, n, B=2, S=1024):
    gen = torch.Generator().manual_seed(99)
    out = []
    for _ in range(n):
        ids = torch.randint(0, cfg.vocab_size, (B, S + 1), generator=gen).to(dev)
        out.append({"input_ids": ids[:, :-1].contiguous(), "labels": ids[:, 1:].contiguous()})
    return out


def test_captured_forward_backward_matches_eager(dev):
    from maltos_amd.grad_clip import clip_grad_norm_fused_
    from maltos_amd.graph_step import CapturedForwardBackward

    cfg, eager_model, eager_opt = _make(dev, torch.bfloat16)
    _, graph_model, graph_opt = _make(dev, torch.bfloat16)
    batches = _batches(cfg, dev, 5)

    def finish(opt):
        sq = clip_grad_norm_fused_(opt, 1.0)
        opt.step()
        opt.zero_grad(set_to_none=True)
        return sq.sqrt().item()

    want = []
    for b in batches:
        loss = eager_model(b)
        loss.backward()
        want.append((loss.item(), finish(eager_opt)))

    # 2048 tokens per batch: the linears' weight gradients take the sliced (bmm + sum) form inside the graph
    step = CapturedForwardBackward(graph_model, batches[0], embed=graph_model.embed_tokens,
                                   clear_grads=lambda: graph_opt.zero_grad(set_to_none=True))
    noise = torch.randn(1 << 20, device=dev)
    for b, (want_loss, want_norm) in zip(batches, want):
        loss = step(b).item()
        norm = finish(graph_opt)
        assert abs(loss - want_loss) <= 1e-6 * abs(want_loss), (loss, want_loss)
        assert abs(norm - want_norm) <= 1e-5 * abs(want_norm), (norm, want_norm)
        noise = (noise * 1.0001).sin()          # eager work of the program's own between the replays
        torch.cuda.synchronize()
    for (name, p), q in zip(eager_model.named_parameters(), graph_model.parameters()):
        assert torch.equal(p, q), name
    for p, q in zip(eager_opt.master_params, graph_opt.master_params):
        assert torch.allclose(p, q, rtol=1e-6, atol=1e-9)


def test_capture_refuses_unbound_gradients_and_changed_shapes(dev):
    from maltos_amd.graph_step import CapturedForwardBackward
    from maltos_amd.llama import LlamaConfig, LlamaForCausalLM

    cfg = LlamaConfig(vocab_size=256, hidden_size=128, intermediate_size=256, num_hidden_layers=1, num_attention_heads=2,
                      max_position_embeddings=128, rms_norm_eps=1e-5)
    model = LlamaForCausalLM(cfg).to(dev)
    batch = _batches(cfg, dev, 1, B=1, S=64)[0]
    with pytest.raises(RuntimeError, match="bound .grad"):
        CapturedForwardBackward(model, batch)
    for p in model.parameters():
        p.grad = torch.zeros_like(p)
    with pytest.raises(RuntimeError, match="pass embed="):
        CapturedForwardBackward(model, batch)
    step = CapturedForwardBackward(model, batch, embed=model.embed_tokens)
    want = model(batch)
    want.backward()
    want_grads = [p.grad.clone() for p in model.parameters()]
    for p in model.parameters():
        p.grad.zero_()
    assert abs(step(batch).item() - want.item()) <= 1e-6 * abs(want.item())
    for (name, p), g in zip(model.named_parameters(), want_grads):
        assert torch.allclose(p.grad, g, rtol=1e-5, atol=1e-7), name
    short = {k: v[:, :32].contiguous() for k, v in batch.items()}
    with pytest.raises(ValueError, match="recorded"):
        step(short)


def test_fused_residual_norm_and_in_buffer_gradients_equal_the_plain_model(dev):
    """The model with residual adds fused into the norms (the default) and with weight gradients accumulated straight
    into bound buffers gives bit for bit the loss and the gradients of the reference op sequence."""
    from dataclasses import replace

    from maltos_amd.llama import LlamaForCausalLM, set_grad_accumulation_into_buffers

    cfg, fused_model, _ = _make(dev, torch.bfloat16)
    plain_model = LlamaForCausalLM(replace(cfg, fuse_residual_norm=False)).to(dev).to(torch.bfloat16)
    plain_model.load_state_dict(fused_model.state_dict())
    assert fused_model.config.fuse_residual_norm
    for module in fused_model.modules():   # one product per projection, as in the plain model: the comparison is bit for bit
        if hasattr(module, "fuse_projections"):
            module.fuse_projections = False
    assert set_grad_accumulation_into_buffers(fused_model) == 2 * 7
    batch = _batches(cfg, dev, 1)[0]
    for p in plain_model.parameters():
        p.grad = None
    for p in fused_model.parameters():
        p.grad = torch.zeros_like(p)
    want = plain_model(batch)
    want.backward()
    got = fused_model(batch)
    got.backward()
    assert torch.equal(got, want)
    for (name, p), q in zip(plain_model.named_parameters(), fused_model.parameters()):
        assert torch.equal(p.grad, q.grad), name
    # packed documents take the same path
    packed = dict(batch)
    S = batch["input_ids"].size(1)
    packed["position_ids"] = (torch.arange(S, device=dev) % 300).expand_as(batch["input_ids"]).contiguous()
    packed["sequence_ids"] = (torch.arange(S, device=dev) // 300).expand_as(batch["input_ids"]).contiguous()
    assert torch.equal(fused_model(packed), plain_model(packed))
