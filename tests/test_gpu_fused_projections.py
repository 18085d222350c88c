"""q/k/v and gate/up projections as one product over adjacent weights (what the flat optimizer layouts make of them)
against the same model with every projection on its own."""
import pytest
import torch

from maltos_amd.llama import LlamaConfig, LlamaForCausalLM, set_grad_accumulation_into_buffers
from maltos_amd.optim import FusedAdamW, MasterWeightsOptimizer

pytestmark = pytest.mark.gpu


def _close(got, want, what):
    got, want = got.float(), want.float()
    # the two forms run different GEMM shapes: sums of the same products in another order, rounded to bf16 at the end
    # of every product; the differences travel down the layers to the gradients nearest the input
    bound = 2.0 ** -5 * want.abs() + 1e-2 * want.abs().max()
    err = (got - want).abs()
    assert (err <= bound).all(), f"{what}: worst excess {(err - bound).max().item():.3e}"


@pytest.mark.parametrize("into_grad", [False, True], ids=["autograd-accumulates", "into-grad-buffers"])
def test_fused_projections_match_separate_ones(dev, into_grad):
    cfg = LlamaConfig(vocab_size=512, hidden_size=256, intermediate_size=688, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, max_position_embeddings=128, rms_norm_eps=1e-5)
    torch.manual_seed(9)
    plain = LlamaForCausalLM(cfg).to(dev).to(torch.bfloat16)
    fused = LlamaForCausalLM(cfg).to(dev).to(torch.bfloat16)
    fused.load_state_dict(plain.state_dict())
    adam = lambda ps: FusedAdamW(ps, lr=1e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    opt_plain = MasterWeightsOptimizer(plain.parameters(), optimizer_factory=adam, flat=False)
    opt_fused = MasterWeightsOptimizer(fused.parameters(), optimizer_factory=adam, flat=True)   # adjacent weights and grads
    if into_grad:
        set_grad_accumulation_into_buffers(fused)
    gen = torch.Generator().manual_seed(1)
    ids = torch.randint(0, 512, (2, 129), generator=gen).to(dev)
    batch = {"input_ids": ids[:, :-1].contiguous(), "labels": ids[:, 1:].contiguous()}
    for step in range(2):
        losses = []
        for model in (plain, fused):
            loss = model(batch)
            loss.backward()
            losses.append(loss.item())
        for layer in fused.layers:   # the one-product forms were taken
            assert layer.self_attn.__dict__["_maltos_hip_fused_rows"].weight.shape == (256 + 128 + 128, 256)
            assert layer.mlp.__dict__["_maltos_hip_fused_rows"].weight.shape == (2 * 688, 256)
            assert (layer.mlp.__dict__["_maltos_hip_fused_rows"].grad is not None)
        for layer in plain.layers:
            assert "_maltos_hip_fused_rows" not in layer.self_attn.__dict__ or layer.self_attn.__dict__["_maltos_hip_fused_rows"].weight is None
        assert abs(losses[0] - losses[1]) <= 1e-3 * abs(losses[0])
        for (name, p), q in zip(plain.named_parameters(), fused.parameters()):
            _close(q.grad, p.grad, f"step {step} grad of {name}")
        opt_plain.step(), opt_fused.step()
        opt_plain.zero_grad(set_to_none=True), opt_fused.zero_grad(set_to_none=True)
        # fp32 masters: a step moves an element by at most lr (1 + wd |p|), in either direction where its gradient is ~ 0
        for (name, _), p, q in zip(plain.named_parameters(), opt_plain.master_params, opt_fused.master_params):
            assert (p.detach() - q.detach()).abs().max() <= (step + 1) * 2.2e-3, name


def test_strided_swiglu_equals_the_flat_kernels(dev):
    """The row-strided SwiGLU kernels (gate and up as column blocks of one buffer) give the flat kernels' bits."""
    from maltos_amd import ops

    gen = torch.Generator().manual_seed(3)
    rows, cols = 300, 688
    for order in ((0, cols), (cols, 0)):
        gu = torch.randn(rows, 2 * cols, generator=gen).bfloat16().to(dev)
        dh = torch.randn(rows, cols, generator=gen).bfloat16().to(dev)
        gate, up = gu[:, order[0]:order[0] + cols].contiguous(), gu[:, order[1]:order[1] + cols].contiguous()
        assert torch.equal(ops.swiglu_rows(gu, order[0], order[1], cols), torch.ops.maltos.swiglu_fwd(gate, up))
        dgu = ops.swiglu_rows_backward(dh, gu, order[0], order[1], cols)
        dg, du = torch.ops.maltos.swiglu_bwd(dh, gate, up)
        assert torch.equal(dgu[:, order[0]:order[0] + cols], dg) and torch.equal(dgu[:, order[1]:order[1] + cols], du)


@pytest.mark.parametrize("documents", [False, True], ids=["causal", "documents"])
def test_rope_attention_node_equals_the_separate_ops_and_hands_over_one_gradient_matrix(dev, documents, monkeypatch):
    """Rotary embedding + attention as one autograd node: the bits of the two separate ops, forward and backward; with
    the flat layout's one-product q/k/v projection its three gradients arrive side by side and nothing is copied together
    (no torch.cat in the backward pass)."""
    from maltos_amd.llama import LlamaAttention

    cfg = LlamaConfig(vocab_size=512, hidden_size=256, intermediate_size=688, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, max_position_embeddings=128, rms_norm_eps=1e-5)
    torch.manual_seed(11)
    model = LlamaForCausalLM(cfg).to(dev).to(torch.bfloat16)
    adam = lambda ps: FusedAdamW(ps, lr=1e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    MasterWeightsOptimizer(model.parameters(), optimizer_factory=adam, flat=True)   # adjacent weights: one-product projections
    gen = torch.Generator().manual_seed(2)
    ids = torch.randint(0, 512, (2, 129), generator=gen).to(dev)
    batch = {"input_ids": ids[:, :-1].contiguous(), "labels": ids[:, 1:].contiguous()}
    if documents:
        cuts = [0, 1, 40, 64, 65, 128]
        batch["position_ids"] = torch.cat([torch.arange(b - a) for a, b in zip(cuts, cuts[1:])]).expand(2, -1).contiguous().to(dev)
        batch["sequence_ids"] = torch.cat([torch.full((b - a,), i) for i, (a, b) in enumerate(zip(cuts, cuts[1:]))]).expand(2, -1).contiguous().to(dev)
    results = []
    for fused_node in (False, True):
        monkeypatch.setattr(LlamaAttention, "fuse_rope_attention", fused_node)
        cats = []
        real_cat = torch.cat
        monkeypatch.setattr(torch, "cat", lambda *a, **kw: (cats.append(1), real_cat(*a, **kw))[1])
        loss = model(batch)
        before = len(cats)
        loss.backward()
        monkeypatch.setattr(torch, "cat", real_cat)
        results.append((loss.detach().clone(), [p.grad.clone() for p in model.parameters()], len(cats) - before))
        for p in model.parameters():
            p.grad.zero_()
    (loss_a, grads_a, cats_a), (loss_b, grads_b, cats_b) = results
    assert torch.equal(loss_a, loss_b)
    for (name, _), a, b in zip(model.named_parameters(), grads_a, grads_b):
        assert torch.equal(a, b), name
    assert cats_a == cfg.num_hidden_layers and cats_b == 0, (cats_a, cats_b)


def test_rope_pair_in_place_equals_the_copying_form(dev):
    from maltos_amd import ops

    gen = torch.Generator().manual_seed(5)
    B, S, D = 2, 70, 64
    joint = torch.randn(B, S, 4 + 2 + 2, D, generator=gen).bfloat16().to(dev).transpose(1, 2)
    q, k = joint[:, :4], joint[:, 4:6]
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2).float() / D))
    ang = torch.arange(128).float()[:, None] * inv[None]
    cos, sin = ang.cos().bfloat16().to(dev), ang.sin().bfloat16().to(dev)
    pos = torch.randint(0, 128, (B, S), generator=gen).int().to(dev)
    for inverse in (False, True):
        for positions in (None, pos):
            want = torch.ops.maltos.rope_pair(q, k, cos, sin, positions, 3, inverse)
            untouched = joint[:, 6:].clone()
            mine = joint.clone()
            ops.rope_pair_(mine[:, :4], mine[:, 4:6], cos, sin, positions=positions, position_offset=3, inverse=inverse)
            assert torch.equal(mine[:, :4], want[0]) and torch.equal(mine[:, 4:6], want[1])
            assert torch.equal(mine[:, 6:], untouched)
