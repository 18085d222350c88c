"""GPU parity of the HBM-bound kernels (through the torch.library ops, i.e. through the C ABI) against
the CPU oracle on identical seeded inputs.

Tolerances:
  * fp32                : 1e-4 relative (the stated fp32 bar); most agree to ~1e-6.
  * bf16 forward        : RMSNorm / RoPE / SwiGLU reproduce the reference's eager roundings, so they are
                          compared to the oracle's bf16 evaluation and may differ by at most one bf16 ulp
                          (rsqrt/exp differ in the last fp32 bit between CPU and GPU) on < 0.1 % of entries.
  * bf16 backward, loss : fp32 math inside the kernel and ONE rounding of the result, so against the oracle's
                          fp32 formulas on the bf16-rounded inputs |err| <= 2^-8 |want| + 1e-3 (half a bf16 ulp);
                          loss 1e-4 relative (it is returned in fp32).
"""
import pytest
import torch

from maltos_amd import ops
from oracle import layers as ol
from oracle import optim as oo

pytestmark = pytest.mark.gpu


def _one_rounding(got: torch.Tensor, want: torch.Tensor) -> None:
    """fp32 math + a single bf16 rounding of the result: |err| <= 2^-8 |want| (half an ulp) + 1e-3."""
    got, want = got.float().cpu(), want.float().cpu()
    err = (got - want).abs()
    bound = 2.0 ** -8 * want.abs() + 1e-3
    assert (err <= bound).all(), f"worst excess {(err - bound).max().item()}"


def _ulp_close(got: torch.Tensor, want: torch.Tensor, max_frac: float = 1e-3) -> None:
    got, want = got.float().cpu(), want.float().cpu()
    diff = (got - want).abs()
    ulp = torch.maximum(want.abs(), torch.tensor(1e-30)) * 2.0 ** -7  # one bf16 ulp is <= 2^-7 relative
    assert (diff <= ulp).all(), f"max diff {diff.max().item()} exceeds one bf16 ulp"
    assert (diff > 0).float().mean().item() <= max_frac, "too many entries differ from the oracle's rounding"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,hidden", [(1, 256), (37, 512), (300, 1024)])
def test_rmsnorm_forward_backward(dev, dtype, rows, hidden):
    g = torch.Generator().manual_seed(rows + hidden)
    x = torch.randn(rows, hidden, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(dtype)
    dy = torch.randn(rows, hidden, generator=g).to(dtype)
    xg, wg = x.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
    y = ops.rms_norm(xg, wg, 1e-5)
    y.backward(dy.to(dev))
    want = ol.rms_norm(x, w, 1e-5)
    dx, dw = ol.rms_norm_backward(dy, x, w, 1e-5)
    if dtype == torch.float32:
        torch.testing.assert_close(y.cpu(), want, rtol=1e-4, atol=1e-6)
        torch.testing.assert_close(xg.grad.cpu(), dx, rtol=1e-4, atol=1e-5)
        torch.testing.assert_close(wg.grad.cpu(), dw, rtol=1e-4, atol=1e-4)
    else:
        _ulp_close(y, want)
        _one_rounding(xg.grad, dx)
        assert ((wg.grad.float().cpu() - dw).abs() <= 2e-2 + 2.0 ** -8 * dw.abs()).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,hidden", [(4099, 512), (4101, 256), (5003, 1024)])
def test_rmsnorm_many_narrow_rows(dev, dtype, rows, hidden):
    """Millions of elements: every row is what the same row gives in a call of few rows (rows are independent), and the
    oracle's values up to the rare second rounding flip that a different summation order of the mean allows."""
    g = torch.Generator().manual_seed(rows + hidden)
    x = torch.randn(rows, hidden, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(dtype)
    xd, wd = x.to(dev), w.to(dev)
    y = ops.rms_norm(xd, wd, 1e-5)
    for lo, hi in ((0, 700), (rows - 301, rows), (2048, 2049)):
        assert torch.equal(y[lo:hi], ops.rms_norm(xd[lo:hi].contiguous(), wd, 1e-5)), (lo, hi)
    want = ol.rms_norm(x, w, 1e-5).float()
    diff = (y.float().cpu() - want).abs()
    tol = want.abs() * (1e-4 if dtype == torch.float32 else 2.0 ** -7) + 1e-6
    assert (diff <= 2 * tol).all()
    assert (diff > tol).float().mean().item() < 1e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,hidden", [(1, 256), (37, 512), (300, 1024), (4099, 2048), (4099, 512), (4102, 256),
                                         (5001, 1024)])
def test_add_rmsnorm_equals_add_then_rmsnorm(dev, dtype, rows, hidden):
    """The fused residual add + RMSNorm gives bit for bit what the two separate ops give, forward and backward, with
    the summed row used again downstream (the residual path) and without."""
    g = torch.Generator().manual_seed(rows * 7 + hidden)
    x, res, dy, dh = ((torch.randn(rows, hidden, generator=g)).to(dtype).to(dev) for _ in range(4))
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(dtype).to(dev)
    for use_residual_path in (True, False):
        leaves_a = [t.clone().requires_grad_(True) for t in (x, res, w)]
        h = leaves_a[0] + leaves_a[1]
        y = ops.rms_norm(h, leaves_a[2], 1e-5)
        leaves_b = [t.clone().requires_grad_(True) for t in (x, res, w)]
        h2, y2 = ops.add_rms_norm(leaves_b[0], leaves_b[1], leaves_b[2], 1e-5)
        assert torch.equal(h, h2) and torch.equal(y, y2)
        if use_residual_path:
            torch.autograd.backward([y, h], [dy, dh])
            torch.autograd.backward([y2, h2], [dy, dh])
        else:
            y.backward(dy)
            y2.backward(dy)
        for a, b, name in zip(leaves_a, leaves_b, ("x", "res", "w")):
            assert torch.equal(a.grad, b.grad), (name, use_residual_path)
    # only the summed row is used: the gradient passes through to both addends
    xa, ra = x.clone().requires_grad_(True), res.clone().requires_grad_(True)
    h3, _ = ops.add_rms_norm(xa, ra, w, 1e-5)
    h3.backward(dh)
    assert torch.equal(xa.grad, dh) and torch.equal(ra.grad, dh)
    with pytest.raises(ValueError):
        ops.add_rms_norm(x, res[:, : hidden // 2], w, 1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("use_ids", [False, True])
def test_rope_forward_backward(dev, dtype, use_ids):
    B, H, S, D = 2, 3, 17, 64
    g = torch.Generator().manual_seed(42)
    x = torch.randn(B, S, H, D, generator=g).to(dtype).transpose(1, 2)  # the [B,H,S,D] view LlamaAttention makes
    dy = torch.randn(B, S, H, D, generator=g).to(dtype).transpose(1, 2)
    cos_t, sin_t = ol.rope_tables(D, 64)
    cos_t, sin_t = cos_t.to(dtype), sin_t.to(dtype)
    pos = torch.stack([torch.arange(S) % 5, torch.arange(S) + 3]) if use_ids else None
    cos, sin = ol.rope_cos_sin(cos_t, sin_t, seq_len=S, position_offset=4, position_ids=pos)
    want = ol.apply_rotary(x, cos, sin)
    want_dx = ol.apply_rotary_backward(dy, cos, sin)
    xg = x.to(dev).requires_grad_(True)
    y = ops.rope(xg, cos_t.to(dev), sin_t.to(dev), positions=None if pos is None else pos.to(dev), position_offset=4)
    assert y.stride() == xg.stride()
    y.backward(dy.to(dev))
    if dtype == torch.float32:
        torch.testing.assert_close(y.cpu(), want, rtol=1e-4, atol=1e-6)
        torch.testing.assert_close(xg.grad.cpu(), want_dx, rtol=1e-4, atol=1e-6)
    else:  # every product and sum rounded where the reference's eager ops round: bit exact
        assert torch.equal(y.cpu(), want)
        assert torch.equal(xg.grad.cpu(), want_dx)
    with pytest.raises(ValueError):
        ops.rope(xg, cos_t.to(dev)[:8], sin_t.to(dev)[:8], position_offset=4)  # table too short


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("use_ids", [False, True])
def test_rope_pair_equals_two_rotations(dev, dtype, use_ids):
    """q and k of a GQA layer (models/llama.py:143-144) rotated by one launch: the oracle's values for each operand, bit
    for bit what two single launches give, forward and backward, on the strided views the model hands over."""
    B, Hq, Hk, S, D = 2, 6, 2, 19, 64
    g = torch.Generator().manual_seed(7)
    mk = lambda h: torch.randn(B, S, h, D, generator=g).to(dtype).transpose(1, 2)
    xq, xk, dq, dk = mk(Hq), mk(Hk), mk(Hq), mk(Hk)
    cos_t, sin_t = ol.rope_tables(D, 64)
    cos_t, sin_t = cos_t.to(dtype), sin_t.to(dtype)
    pos = torch.stack([torch.arange(S) % 5, torch.arange(S) + 3]) if use_ids else None
    cos, sin = ol.rope_cos_sin(cos_t, sin_t, seq_len=S, position_offset=2, position_ids=pos)
    kw = dict(positions=None if pos is None else pos.to(dev), position_offset=2)
    qg, kg = xq.to(dev).requires_grad_(True), xk.to(dev).requires_grad_(True)
    yq, yk = ops.rope_pair(qg, kg, cos_t.to(dev), sin_t.to(dev), **kw)
    assert yq.stride() == qg.stride() and yk.stride() == kg.stride()
    (yq * dq.to(dev)).sum().backward(retain_graph=True)
    (yk * dk.to(dev)).sum().backward()
    q1, k1 = xq.to(dev).requires_grad_(True), xk.to(dev).requires_grad_(True)
    sq, sk = ops.rope(q1, cos_t.to(dev), sin_t.to(dev), **kw), ops.rope(k1, cos_t.to(dev), sin_t.to(dev), **kw)
    sq.backward(dq.to(dev))
    sk.backward(dk.to(dev))
    for got, single in ((yq, sq), (yk, sk), (qg.grad, q1.grad), (kg.grad, k1.grad)):
        assert torch.equal(got, single)
    for got, x, d in ((yq, xq, None), (yk, xk, None), (qg.grad, None, dq), (kg.grad, None, dk)):
        want = ol.apply_rotary(x, cos, sin) if d is None else ol.apply_rotary_backward(d, cos, sin)
        if dtype == torch.float32:
            torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=1e-6)
        else:
            assert torch.equal(got.cpu(), want)
    with pytest.raises(ValueError):
        ops.rope_pair(qg, kg[:, :, :5], cos_t.to(dev), sin_t.to(dev))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [(5, 7), (64, 1376)])
def test_swiglu_forward_backward(dev, dtype, n):
    g = torch.Generator().manual_seed(sum(n))
    gate = (2 * torch.randn(*n, generator=g)).to(dtype)
    up = torch.randn(*n, generator=g).to(dtype)
    dh = torch.randn(*n, generator=g).to(dtype)
    gg, ug = gate.to(dev).requires_grad_(True), up.to(dev).requires_grad_(True)
    h = ops.swiglu(gg, ug)
    h.backward(dh.to(dev))
    want = ol.swiglu(gate, up)
    dg, du = ol.swiglu_backward(dh, gate, up)
    if dtype == torch.float32:
        torch.testing.assert_close(h.cpu(), want, rtol=1e-4, atol=1e-6)
        torch.testing.assert_close(gg.grad.cpu(), dg, rtol=1e-4, atol=1e-6)
        torch.testing.assert_close(ug.grad.cpu(), du, rtol=1e-4, atol=1e-6)
    else:
        _ulp_close(h, want)
        _one_rounding(gg.grad, dg)
        _one_rounding(ug.grad, du)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,vocab", [(6, 5), (64, 8192), (33, 32000), (5, 50257)])
def test_cross_entropy(dev, dtype, rows, vocab):
    g = torch.Generator().manual_seed(rows * vocab % 9973)
    logits = (3 * torch.randn(rows, vocab, generator=g)).to(dtype)
    labels = torch.randint(0, vocab, (rows,), generator=g)
    labels[::3] = -100
    lg = logits.to(dev).requires_grad_(True)
    loss = ops.cross_entropy(lg, labels.to(dev))
    assert loss.dtype == torch.float32
    (loss * 1.0).backward()
    want_loss, want_grad = ol.causal_cross_entropy_explicit(logits, labels)
    assert abs(loss.item() - want_loss.item()) <= 1e-4 * abs(want_loss.item()) + 1e-6
    tol = 1e-6 if dtype == torch.float32 else 2.0 ** -8
    assert ((lg.grad.float().cpu() - want_grad).abs() <= tol * want_grad.abs() + 1e-7).all()
    # upstream gradient other than one, and the reference's library form
    lg2 = logits.to(dev).requires_grad_(True)
    (ops.cross_entropy(lg2, labels.to(dev)) * 0.25).backward()
    assert ((lg2.grad.float().cpu() - 0.25 * want_grad).abs() <= 2 * tol * want_grad.abs() + 1e-7).all()
    lib = ol.causal_cross_entropy(logits.float(), labels)
    assert abs(loss.item() - lib.item()) <= 1e-4 * abs(lib.item()) + 1e-6


def test_cross_entropy_backward_consumes_its_buffer_once(dev):
    """The logits gradient written by the forward kernel is scaled in place and handed on without a copy: the result
    is right for a scaled loss, nothing of the logits' size is allocated in backward, and a second walk is refused."""
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(16, 1000, generator=g)
    labels = torch.randint(0, 1000, (16,), generator=g)
    lg = logits.to(dev).requires_grad_(True)
    loss = ops.cross_entropy(lg, labels.to(dev))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    (loss * 0.5).backward(retain_graph=True)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() - before < 2 * lg.numel() * 4     # lg.grad itself, no second buffer
    _, want_grad = ol.causal_cross_entropy_explicit(logits, labels)
    assert torch.allclose(lg.grad.cpu(), 0.5 * want_grad, rtol=1e-5, atol=1e-8)
    with pytest.raises(RuntimeError, match="backward ran twice"):
        loss.backward()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,vocab", [(7, 1000), (48, 32000), (3, 70001)])
def test_cross_entropy_over_its_logits(dev, dtype, rows, vocab):
    """overwrite_logits=True: the same loss and the same gradient, bit for bit, as the form with its own gradient
    buffer, and the gradient stands where the logits stood (every row-kernel form: registers, LDS, re-read)."""
    g = torch.Generator().manual_seed(rows + vocab)
    logits = (3 * torch.randn(rows, vocab, generator=g)).to(dtype)
    labels = torch.randint(0, vocab, (rows,), generator=g)
    labels[1::4] = -100
    a = logits.to(dev).requires_grad_(True)
    (ops.cross_entropy(a, labels.to(dev)) * 0.5).backward()
    base = logits.to(dev)
    b = base.clone().requires_grad_(True)
    owned = b * 1                      # a non-leaf the loss may consume, as the model's logits are
    store = owned.data_ptr()
    loss_b = ops.cross_entropy(owned, labels.to(dev), overwrite_logits=True)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    (loss_b * 0.5).backward(retain_graph=True)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() - before <= b.numel() * b.element_size() + 4096   # b.grad only
    assert loss_b.item() == ops.cross_entropy(logits.to(dev), labels.to(dev)).item()
    assert torch.equal(b.grad, a.grad)
    assert owned.data_ptr() == store and torch.equal(owned.detach(), a.grad)
    with pytest.raises(RuntimeError, match="backward ran twice"):
        loss_b.backward()
    with pytest.raises(ValueError, match="contiguous"):
        ops.cross_entropy(base.t().contiguous().t(), labels.to(dev), overwrite_logits=True)
    # another consumer that saved the logits for its own backward is told that they are gone
    c = base.clone().requires_grad_(True)
    shared = c * 1
    other = shared.sin().sum()
    ops.cross_entropy(shared, labels.to(dev), overwrite_logits=True)
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        other.backward()


def test_cross_entropy_without_targets_is_zero(dev):
    lg = torch.randn(2, 3, 5, device=dev, requires_grad=True)
    loss = ops.cross_entropy(lg, torch.full((2, 3), -100, device=dev))
    assert loss.item() == 0.0
    loss.backward()
    assert not lg.grad.any()


@pytest.mark.parametrize("n", [1, 5, 1000, 4099, 1 << 20])
def test_adamw_steps_match_library_and_closed_form(dev, n):
    g = torch.Generator().manual_seed(n)
    p0 = torch.randn(n, generator=g)
    hp = dict(lr=3e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
    ref = torch.nn.Parameter(p0.clone())
    lib = torch.optim.AdamW([ref], lr=hp["lr"], betas=(hp["beta1"], hp["beta2"]), eps=hp["eps"], weight_decay=hp["weight_decay"])
    p, m, v = p0.to(dev), torch.zeros(n, device=dev), torch.zeros(n, device=dev)
    lowp = torch.empty(n, dtype=torch.bfloat16, device=dev)
    cp, cm, cv = p0.clone(), torch.zeros(n), torch.zeros(n)
    for step in (1, 2, 3):
        grad = 0.01 * torch.randn(n, generator=g)
        ref.grad = grad.clone()
        lib.step()
        ops.adamw_step_(p, grad.to(dev), m, v, step=step, p_lowp=lowp, **hp)
        cp, cm, cv = oo.adamw_reference_step(cp, grad, cm, cv, step=step, **hp)
        torch.testing.assert_close(p.cpu(), ref.detach(), rtol=1e-4, atol=1e-7)
        torch.testing.assert_close(p.cpu(), cp, rtol=1e-4, atol=1e-7)
        assert torch.equal(lowp.cpu(), p.cpu().bfloat16())
    torch.testing.assert_close(m.cpu(), lib.state[ref]["exp_avg"], rtol=1e-4, atol=1e-9)
    torch.testing.assert_close(v.cpu(), lib.state[ref]["exp_avg_sq"], rtol=1e-4, atol=1e-12)


def test_adamw_on_unaligned_views_and_fused_clip(dev):
    n = 1003
    g = torch.Generator().manual_seed(3)
    base = torch.randn(4 * n + 8, generator=g).to(dev)
    p, grad, m, v = (base[1 + i * n: 1 + (i + 1) * n] for i in range(4))  # 4-byte aligned only
    m.zero_(), v.zero_()
    p0, g0 = p.cpu().clone(), grad.cpu().clone()
    hp = dict(lr=1e-2, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.0)
    sq = ops.sq_norm(grad.contiguous())
    norm = float(sq.sqrt().item())
    assert abs(norm - oo.global_grad_norm([g0])) <= 1e-6 * norm
    ops.adamw_step_(p, grad, m, v, step=1, sq_norm=sq, max_norm=1.0, **hp)
    coef = oo.clip_coefficient(norm, 1.0)
    assert coef < 1.0
    want, _, _ = oo.adamw_reference_step(p0, g0 * coef, torch.zeros(n), torch.zeros(n), step=1, **hp)
    torch.testing.assert_close(p.cpu(), want, rtol=1e-4, atol=1e-7)


@pytest.mark.parametrize("n", [3, 4096, 1234567])
@pytest.mark.parametrize("src_dtype", [torch.bfloat16, torch.float32])
def test_grad_to_f32_and_norm(dev, n, src_dtype):
    g = torch.Generator().manual_seed(n)
    src = torch.randn(n, generator=g).to(src_dtype)
    dst = torch.full((n,), 7.0, device=dev)
    sq = torch.zeros((), dtype=torch.float64, device=dev)
    ops.grad_to_f32_(dst, src.to(dev), sq_out=sq)
    assert torch.equal(dst.cpu(), src.float())
    want = src.double().pow(2).sum().item()
    assert abs(sq.item() - want) <= 1e-12 * want
    ops.grad_to_f32_(dst, src.to(dev), accumulate=True)
    assert torch.equal(dst.cpu(), src.float() * 2)
    assert abs(ops.sq_norm(dst).item() - 4 * want) <= 1e-12 * 4 * want
    ops.scale_(dst, 0.5)
    assert torch.equal(dst.cpu(), src.float())


def test_model_keeps_hooked_logits(dev):
    """LlamaForCausalLM lets its loss write the gradient over the logits it owns; while lm_head carries a forward hook
    (somebody sees that output), or with LlamaConfig.loss_overwrites_logits=False, the logits are left as they were.  The
    loss and the gradients are the same in every form."""
    from maltos_amd.llama import LlamaConfig, LlamaForCausalLM

    gen = torch.Generator().manual_seed(11)
    ids = torch.randint(0, 300, (2, 65), generator=gen).to(dev)
    batch = (ids[:, :-1].contiguous(), ids[:, 1:].contiguous())
    results = {}
    for form in ("own", "hooked", "config-off"):
        cfg = LlamaConfig(vocab_size=300, hidden_size=128, intermediate_size=256, num_hidden_layers=1, num_attention_heads=2,
                          max_position_embeddings=64, loss_overwrites_logits=form != "config-off")
        torch.manual_seed(3)
        model = LlamaForCausalLM(cfg).to(dev).to(torch.bfloat16)
        seen = []
        if form != "own":
            model.lm_head.register_forward_hook(lambda mod, args, out: seen.append((out, out.detach().clone())))
        loss = model(batch)
        loss.backward()
        for out, copy in seen:
            assert torch.equal(out.detach(), copy), f"{form}: the hooked logits were overwritten"
        results[form] = (loss.detach().clone(), model.lm_head.weight.grad.clone())
    for form in ("hooked", "config-off"):
        assert torch.equal(results[form][0], results["own"][0]) and torch.equal(results[form][1], results["own"][1])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_empty_inputs_are_served(dev, dtype):
    """Zero rows, zero batch, zero length: every op returns outputs of the right shape (and gradients of the right shape
    through its backward) without launching into nothing; a loss over no rows is 0."""
    h, I, V, H, D = 256, 384, 512, 2, 64
    w = torch.ones(h, dtype=dtype, device=dev, requires_grad=True)
    x = torch.zeros(0, h, dtype=dtype, device=dev, requires_grad=True)
    y = ops.rms_norm(x, w, 1e-5)
    y.sum().backward()
    assert y.shape == (0, h) and x.grad.shape == (0, h) and w.grad.shape == (h,) and w.grad.abs().max() == 0
    s, y2 = ops.add_rms_norm(x, x, w, 1e-5)
    assert s.shape == (0, h) and y2.shape == (0, h)
    (s.sum() + y2.sum()).backward()

    cos = torch.ones(16, D // 2, dtype=dtype, device=dev)
    sin = torch.zeros(16, D // 2, dtype=dtype, device=dev)
    for shape in ((0, H, 8, D), (2, H, 0, D)):
        q = torch.zeros(shape, dtype=dtype, device=dev, requires_grad=True)
        k = torch.zeros(shape, dtype=dtype, device=dev, requires_grad=True)
        r = ops.rope(q, cos, sin)
        rq, rk = ops.rope_pair(q, k, cos, sin)
        (r.sum() + rq.sum() + rk.sum()).backward()
        assert r.shape == shape and rq.shape == shape and q.grad.shape == shape
        for mode in (ops.MASK_CAUSAL, ops.MASK_NONE):
            o, lse = ops.attention(q, k, k, mask_mode=mode, return_lse=True)
            o.sum().backward()
            assert o.shape == shape and lse.shape == shape[:3] and k.grad.shape == shape

    # queries without any key: zeros and LSE = -inf; keys without any query: zero gradients
    q = torch.randn(1, H, 5, D, device=dev).to(dtype).requires_grad_(True)
    k0 = torch.zeros(1, H, 0, D, dtype=dtype, device=dev, requires_grad=True)
    o, lse = ops.attention(q, k0, k0, mask_mode=ops.MASK_NONE, return_lse=True)
    o.sum().backward()
    assert o.abs().max() == 0 and torch.isinf(lse).all() and (lse < 0).all() and q.grad.abs().max() == 0 and k0.grad.shape == k0.shape

    g = torch.zeros(0, I, dtype=dtype, device=dev, requires_grad=True)
    u = torch.zeros(0, I, dtype=dtype, device=dev, requires_grad=True)
    hh = ops.swiglu(g, u)
    hh.sum().backward()
    assert hh.shape == (0, I) and g.grad.shape == (0, I)

    logits = torch.zeros(0, V, dtype=dtype, device=dev, requires_grad=True)
    loss = ops.cross_entropy(logits, torch.zeros(0, dtype=torch.long, device=dev))
    loss.backward()
    assert float(loss.detach()) == 0.0 and logits.grad.shape == (0, V)

    if dtype == torch.float32:
        p = torch.zeros(0, device=dev)
        ops.adamw_step_(p, p.clone(), p.clone(), p.clone(), lr=1e-3, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1, step=1)
        assert float(ops.sq_norm(p)) == 0.0
        ops.scale_(p, 0.5)
        ops.grad_to_f32_(p, torch.zeros(0, dtype=torch.bfloat16, device=dev))
    out_acc = torch.zeros(1, H, 0, D, device=dev)
    ops.attention_merge_(out_acc, torch.zeros(1, H, 0, device=dev), torch.zeros(1, H, 0, D, dtype=dtype, device=dev), torch.zeros(1, H, 0, device=dev))


def test_more_than_two_to_the_31_elements(dev):
    """Tensors of more than 2^31 elements (flat indices past 32 bits): the head, the middle that straddles the 2^31st
    element and the tail of every result equal what the same kernel gives for those rows alone."""
    torch.manual_seed(5)
    # cross-entropy: 70,000 x 32,000 = 2.24e9 logits
    rows, V = 70_000, 32_000
    logits = torch.randn(rows, V, device=dev, dtype=torch.bfloat16)
    labels = torch.randint(0, V, (rows,), device=dev)
    labels[::7] = -100
    loss, dlogits, count = torch.ops.maltos.ce_fwd_bwd(logits, labels, -100)   # mean over the rows that have a target
    parts = 0.0
    cut = (2 ** 31) // V
    for a, b in ((0, 300), (cut - 150, cut + 150), (rows - 300, rows)):
        s, d, c = torch.ops.maltos.ce_fwd_bwd(logits[a:b].contiguous(), labels[a:b].contiguous(), -100)
        # the gradient carries 1 / count of its own call
        assert torch.allclose(dlogits[a:b].float() * float(count), d.float() * float(c), rtol=2 ** -7, atol=1e-6), (a, b)
    for a in range(0, rows, 10_000):
        s, _, c = torch.ops.maltos.ce_fwd_bwd(logits[a:a + 10_000].contiguous(), labels[a:a + 10_000].contiguous(), -100)
        parts += float(s) * float(c)
    assert int(count) == int((labels != -100).sum()) and abs(float(loss) * float(count) - parts) <= 1e-5 * parts
    del logits, dlogits

    # SwiGLU and RMSNorm: 4,400,000 rows of 512
    n_rows, h = 4_400_000, 512
    cut = (2 ** 31) // h
    g = torch.randn(n_rows, h, device=dev, dtype=torch.bfloat16)
    u = torch.randn(n_rows, h, device=dev, dtype=torch.bfloat16)
    w = torch.randn(h, device=dev, dtype=torch.bfloat16)
    out = torch.ops.maltos.swiglu_fwd(g, u)
    y, rstd = torch.ops.maltos.rmsnorm_fwd(g, w, 1e-5)
    dg, du = torch.ops.maltos.swiglu_bwd(out, g, u)
    dx, dw = torch.ops.maltos.rmsnorm_bwd(u, g, w, rstd)
    for a, b in ((0, 200), (cut - 100, cut + 100), (n_rows - 200, n_rows)):
        ga, ua = g[a:b].contiguous(), u[a:b].contiguous()
        assert torch.equal(out[a:b], torch.ops.maltos.swiglu_fwd(ga, ua))
        ya, ra = torch.ops.maltos.rmsnorm_fwd(ga, w, 1e-5)
        assert torch.equal(y[a:b], ya) and torch.equal(rstd[a:b], ra)
        dga, dua = torch.ops.maltos.swiglu_bwd(out[a:b].contiguous(), ga, ua)
        assert torch.equal(dg[a:b], dga) and torch.equal(du[a:b], dua)
        assert torch.equal(dx[a:b], torch.ops.maltos.rmsnorm_bwd(ua, ga, w, ra)[0])
    assert torch.isfinite(dw.float()).all()
    del g, u, out, y, dg, du, dx

    # AdamW, the norm and the gradient conversion over 2.2e9 parameters
    n = 2 ** 31 + 4096 * 13 + 5
    p = torch.randn(n, device=dev)
    grad16 = torch.randn(n, device=dev, dtype=torch.bfloat16)
    grad = torch.empty(n, device=dev)
    sq = torch.zeros((), dtype=torch.float64, device=dev)
    ops.grad_to_f32_(grad, grad16, sq_out=sq)
    want_sq = sum(float(grad16[a:a + 2 ** 28].double().pow(2).sum()) for a in range(0, n, 2 ** 28))
    assert abs(float(sq) - want_sq) <= 1e-9 * want_sq and abs(float(ops.sq_norm(grad)) - want_sq) <= 1e-9 * want_sq
    m, v = torch.zeros(n, device=dev), torch.zeros(n, device=dev)
    hp = dict(lr=1e-2, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1, step=1)
    for a, b in ((0, 4096), (2 ** 31 - 2048, 2 ** 31 + 2048), (n - 4101, n)):
        a -= a % 4   # 16-byte aligned views, like the whole buffer
        pa, ga = p[a:b].clone(), grad[a:b].clone()
        ma, va = torch.zeros_like(pa), torch.zeros_like(pa)
        ops.adamw_step_(pa, ga, ma, va, **hp)
        if a == 0:
            first = (pa, ma, va)
        elif b == n:
            last = (a, pa, ma, va)
        else:
            mid = (a, b, pa, ma, va)
    ops.adamw_step_(p, grad, m, v, **hp)
    assert all(torch.equal(x[:4096], y) for x, y in zip((p, m, v), first))
    assert all(torch.equal(x[mid[0]:mid[1]], y) for x, y in zip((p, m, v), mid[2:]))
    assert all(torch.equal(x[last[0]:], y) for x, y in zip((p, m, v), last[1:]))
