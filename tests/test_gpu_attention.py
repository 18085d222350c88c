"""GPU parity of the attention kernels (called through the torch.library ops -> C ABI) against the CPU
oracle on identical seeded inputs: forward O and LSE, backward dQ/dK/dV, the LSE merge, the
kernel-shaped flash_* function set and the zigzag ring schedule.

Tolerances
  * float32 (generic kernels) : 1e-4 relative (stated fp32 bar) with a 1e-5 absolute floor.
  * bfloat16 (MFMA kernels)   : inputs are rounded to bf16 first and the oracle runs in fp32 on those values.
      O, dQ, dK, dV : |err| <= 2e-2 + 2^-8 |want|.  2e-2 is the stated max-abs bar; the second term is half a
                      bf16 ulp of the expected value, the rounding any bf16 output carries (it matters only
                      for |want| > ~5, e.g. dV rows that sum many queries).
      LSE (fp32)    : 1e-4 absolute (scores and row sums are formed in fp32 from the bf16 inputs; measured ~4e-6).
  * reference ring test vectors (fp32, head_dim 3): forward 1e-5, backward 2e-5, the reference's own bars
    (zigzag ring and packed-document ring).
"""
import pytest
import torch

from maltos_amd import ops
from maltos_amd.attention_backend import causal_attention
from maltos_amd.flash_utils import (flash_attn_dense, flash_attn_dense_backward, flash_attn_dense_with_lse,
                                    flash_attn_varlen, flash_attn_varlen_prefix, flash_attn_varlen_prefix_backward,
                                    flash_attn_varlen_prefix_with_lse)
from maltos_amd.llama import HipAttentionCore
from maltos_amd.ring_attention import HipRingAttentionCore, packed_ring_attention, zigzag_ring_attention
from maltos_amd.ring_layout import expected_zigzag_ring_positions
from oracle import attention as oa

pytestmark = pytest.mark.gpu


def check(got: torch.Tensor, want: torch.Tensor, dtype, what: str = "") -> None:
    got, want = got.float().cpu(), want.float().cpu()
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    err = (got - want).abs()
    bound = 1e-4 * want.abs() + 1e-5 if dtype == torch.float32 else 2e-2 + 2.0 ** -8 * want.abs()
    assert (err <= bound).all(), f"{what}: worst excess {(err - bound).max().item():.3e} (max err {err.max().item():.3e})"


def make_docs(B, S, gen, max_len, pad_tail=0):
    pos = torch.zeros(B, S, dtype=torch.long)
    seq = torch.full((B, S), -1, dtype=torch.long)
    for b in range(B):
        i = d = 0
        while i < S - pad_tail:
            L = min(int(torch.randint(1, max_len + 1, (1,), generator=gen)), S - pad_tail - i)
            pos[b, i:i + L] = torch.arange(L)
            seq[b, i:i + L] = d
            i, d = i + L, d + 1
    return pos, seq


def bshd(B, H, S, D, gen, dtype):
    return torch.randn(B, S, H, D, generator=gen).to(dtype).transpose(1, 2)


def run_case(dev, dtype, B, Hq, Hkv, Sq, Sk, D, mode, seed, *, max_doc=None, pad_tail=0, share_ids=True, ids=None):
    """share_ids: queries and keys are described by the same id tensors (self-attention over packed rows) or by separate
    copies (what a ring step or a gathered chunk passes).  ids = (positions, sequence_ids) overrides the drawn documents."""
    gen = torch.Generator().manual_seed(seed)
    q, k, v, do = bshd(B, Hq, Sq, D, gen, dtype), bshd(B, Hkv, Sk, D, gen, dtype), bshd(B, Hkv, Sk, D, gen, dtype), bshd(B, Hq, Sq, D, gen, dtype)
    kw, mask = {}, None
    if mode == ops.MASK_CAUSAL:
        mask = oa.causal_mask(Sq, Sk, "cpu")
    elif mode == ops.MASK_DOC:
        assert Sq == Sk
        pos, seq = ids if ids is not None else make_docs(B, Sq, gen, max_doc or max(2, Sq // 3), pad_tail)
        mask = oa.doc_mask(pos, pos, seq, seq)
        dpos, dseq = pos.to(dev), seq.to(dev)
        kw = dict(q_pos=dpos, k_pos=dpos if share_ids else pos.to(dev), q_seq=dseq, k_seq=dseq if share_ids else seq.to(dev))
    qf, kf, vf = (t.detach().float().clone().requires_grad_(True) for t in (q, k, v))
    want_o, want_lse = oa.attention_with_lse(qf, kf, vf, mask)
    want_o.backward(do.float())
    qg, kg, vg = (t.detach().to(dev).requires_grad_(True) for t in (q, k, v))
    o, lse = ops.attention(qg, kg, vg, mask_mode=mode, return_lse=True, **kw)
    o.backward(do.to(dev))
    tag = f"dtype={dtype} B{B} Hq{Hq} Hkv{Hkv} Sq{Sq} Sk{Sk} D{D} mode{mode}"
    check(o, want_o, dtype, tag + " O")
    fin = torch.isfinite(want_lse)
    assert torch.equal(torch.isfinite(lse.cpu()), fin), tag + " LSE -inf pattern"
    lse_tol = 1e-4
    assert (lse.cpu()[fin] - want_lse[fin]).abs().max() <= lse_tol, tag + " LSE"
    check(qg.grad, qf.grad, dtype, tag + " dQ")
    check(kg.grad, kf.grad, dtype, tag + " dK")
    check(vg.grad, vf.grad, dtype, tag + " dV")
    # explicit FlashAttention-2 backward of the oracle agrees too (pins the formula the kernel implements)
    edq, edk, edv = oa.attention_backward_explicit(do, q, k, v, want_o.detach(), want_lse.detach(), mask)
    check(qg.grad, edq, dtype, tag + " dQ(explicit)")
    return o, lse


CASES = [
    # B, Hq, Hkv, Sq, Sk, D, mode
    (1, 1, 1, 1, 1, 64, ops.MASK_CAUSAL),
    (1, 1, 1, 1, 1, 128, ops.MASK_CAUSAL),
    (2, 2, 2, 33, 65, 128, ops.MASK_NONE),
    (1, 2, 1, 257, 257, 128, ops.MASK_CAUSAL),
    (2, 4, 4, 100, 100, 64, ops.MASK_CAUSAL),
    (1, 2, 2, 256, 256, 128, ops.MASK_CAUSAL),
    (2, 3, 3, 300, 300, 64, ops.MASK_CAUSAL),
    (1, 4, 2, 515, 515, 128, ops.MASK_CAUSAL),
    (1, 2, 1, 200, 333, 128, ops.MASK_NONE),
    (1, 2, 2, 333, 200, 64, ops.MASK_NONE),
    (1, 2, 2, 96, 224, 128, ops.MASK_CAUSAL),  # rectangular, bottom-right aligned
    (2, 4, 2, 515, 515, 128, ops.MASK_DOC),
    (2, 8, 2, 260, 260, 64, ops.MASK_DOC),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "B{}_Hq{}_Hkv{}_Sq{}_Sk{}_D{}_m{}".format(*c))
def test_forward_backward_parity(dev, dtype, case):
    run_case(dev, dtype, *case, seed=sum(case))


@pytest.mark.parametrize("D", [64, 128])
def test_document_mask_many_tiles(dev, D):
    """More than 64 and more than 128 key tiles per row: the kernels find the needed tiles 64 statistics entries at a
    time, so the walk crosses chunk boundaries (and a ragged last tile) here; short documents make most tiles skippable,
    one long document keeps whole chunks needed."""
    run_case(dev, torch.bfloat16, 1, 2, 1, 4300, 4300, D, ops.MASK_DOC, 31 + D, max_doc=300, pad_tail=70)
    S = 8400
    idx = torch.arange(S)
    seq = torch.where(idx < 5000, torch.zeros_like(idx), 1 + (idx - 5000) // 170)
    pos = torch.where(idx < 5000, idx, (idx - 5000) % 170)
    run_case(dev, torch.bfloat16, 1, 1, 1, S, S, D, ops.MASK_DOC, 32 + D, ids=(pos.view(1, S), seq.view(1, S)), share_ids=False)


@pytest.mark.parametrize("D", [64, 128])
def test_document_mask_long_row_equals_causal_attention_per_document(dev, D):
    """A size the oracle does not reach as a whole (32768 tokens): packed documents attend exactly as each document alone
    under the causal mask, forward and backward, so the document kernels are checked against the causal kernels slice by
    slice, and the slices short enough for the oracle (up to 4097 tokens, at the start, in the middle and at the end of
    the row) against the oracle itself."""
    S, Hq, Hkv = 32768, 4, 2
    gen = torch.Generator().manual_seed(7 + D)
    q, k, v, do = (bshd(1, h, S, D, gen, torch.bfloat16).to(dev) for h in (Hq, Hkv, Hkv, Hq))
    cuts = [0, 1, 4097, 4160, 12352, 12353, 20000, 28671, S]  # one-token documents, cuts on and off tile edges
    pos = torch.cat([torch.arange(b - a) for a, b in zip(cuts, cuts[1:])]).view(1, S).int().to(dev)
    seq = torch.cat([torch.full((b - a,), i) for i, (a, b) in enumerate(zip(cuts, cuts[1:]))]).view(1, S).int().to(dev)
    ids = dict(q_pos=pos, k_pos=pos, q_seq=seq, k_seq=seq)
    o, lse = ops.attention_forward(q, k, v, mask_mode=ops.MASK_DOC, **ids)
    dq, dk, dv = ops.attention_backward(do, q, k, v, o, lse, mask_mode=ops.MASK_DOC, **ids)
    for a, b in zip(cuts, cuts[1:]):
        sl = (slice(None), slice(None), slice(a, b))
        o1, lse1 = ops.attention_forward(q[sl], k[sl], v[sl], mask_mode=ops.MASK_CAUSAL)
        g1 = ops.attention_backward(do[sl], q[sl], k[sl], v[sl], o1, lse1, mask_mode=ops.MASK_CAUSAL)
        tag = f"D{D} document [{a}, {b})"
        check(o[sl], o1, torch.bfloat16, tag + " O")
        assert (lse[:, :, a:b] - lse1).abs().max() <= 2e-4, tag + " LSE (two kernel results, each within 1e-4)"
        for got, want, name in zip((dq, dk, dv), g1, ("dQ", "dK", "dV")):
            check(got[sl], want, torch.bfloat16, f"{tag} {name}")
        if b - a <= 4097:
            qc, kc, vc, dc = (t[sl].float().cpu() for t in (q, k, v, do))
            want_o, want_lse = oa.attention_with_lse(qc, kc, vc, oa.causal_mask(b - a, b - a, "cpu"))
            check(o[sl], want_o, torch.bfloat16, tag + " O against the oracle")
            assert (lse[:, :, a:b].cpu() - want_lse).abs().max() <= 1e-4, tag + " LSE against the oracle"
            wants = oa.attention_backward_explicit(dc, qc, kc, vc, want_o, want_lse, oa.causal_mask(b - a, b - a, "cpu"))
            for got, want, name in zip((dq, dk, dv), wants, ("dQ", "dK", "dV")):
                check(got[sl], want, torch.bfloat16, f"{tag} {name} against the oracle")


@pytest.mark.parametrize("seed", range(10))
def test_document_mask_drawn_shapes(dev, seed):
    """Drawn batch sizes, head groupings (1, 2, 3, 4, 8 query heads per KV head: the forward and dQ workgroups take one,
    two or four heads), ragged lengths and document lengths, both head dims, ids shared between the sides or not."""
    gen = torch.Generator().manual_seed(1000 + seed)
    draw = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=gen))
    B, Hkv, group = draw(1, 3), draw(1, 2), (1, 2, 3, 4, 8)[draw(0, 4)]
    S = (draw(1, 63), draw(64, 300), draw(301, 900))[draw(0, 2)]
    D = (64, 128)[seed % 2]
    run_case(dev, torch.bfloat16, B, Hkv * group, Hkv, S, S, D, ops.MASK_DOC, 2000 + seed, max_doc=draw(1, max(1, S // 2)),
             pad_tail=draw(0, min(40, S - 1)), share_ids=bool(seed % 3))


@pytest.mark.parametrize("seed", range(16))
def test_causal_and_unmasked_drawn_shapes(dev, seed):
    """Drawn batch sizes, head groupings, head dims (the MFMA kernels' 64 and 128 and the generic kernels' others), query
    and key lengths that differ either way (bottom-right aligned causal mask: with more queries than keys the first rows
    see nothing and must come out as zeros with LSE = -inf), both dtypes."""
    gen = torch.Generator().manual_seed(3000 + seed)
    draw = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=gen))
    B, Hkv, group = draw(1, 3), draw(1, 2), (1, 2, 4, 8)[draw(0, 3)]
    D = (64, 128, 64, 128, 32, 96, 192, 16)[seed % 8]
    dtype = torch.float32 if seed % 8 == 7 else torch.bfloat16
    Sq = (draw(1, 70), draw(71, 400), draw(401, 1100))[draw(0, 2)]
    Sk = (Sq, draw(1, 1100), Sq + draw(1, 200))[draw(0, 2)]
    mode = ops.MASK_CAUSAL if seed % 2 == 0 else ops.MASK_NONE
    run_case(dev, dtype, B, Hkv * group, Hkv, Sq, Sk, D, mode, 4000 + seed)


@pytest.mark.parametrize("D", [64, 128])
def test_document_plan_is_reused_and_follows_the_ids(dev, D):
    """The plan built for a call's ids (mlts_attn_doc_plan) serves later calls with the same id tensors, gives the results
    of a call that builds its own, bit for bit, and is not used once the ids have changed in place."""
    B, Hq, Hkv, S = 2, 4, 1, 330
    gen = torch.Generator().manual_seed(90 + D)
    q, k, v, do = bshd(B, Hq, S, D, gen, torch.bfloat16), bshd(B, Hkv, S, D, gen, torch.bfloat16), \
        bshd(B, Hkv, S, D, gen, torch.bfloat16), bshd(B, Hq, S, D, gen, torch.bfloat16)
    pos, seq = make_docs(B, S, gen, 90, pad_tail=5)
    dpos, dseq = pos.int().to(dev), seq.int().to(dev)

    def run():
        qg, kg, vg = (t.detach().to(dev).requires_grad_(True) for t in (q, k, v))
        o = ops.attention(qg, kg, vg, mask_mode=ops.MASK_DOC, q_pos=dpos, k_pos=dpos, q_seq=dseq, k_seq=dseq)
        o.backward(do.to(dev))
        return o.detach(), qg.grad, kg.grad, vg.grad

    ops.clear_doc_plan_cache()
    first = run()
    assert len(ops._DOC_PLAN_CACHE) == 1
    again = run()
    assert len(ops._DOC_PLAN_CACHE) == 1
    previous = ops.set_doc_plan_cache_entries(0)
    try:
        own = run()  # forward and backward each build the plan in their workspace
    finally:
        ops.set_doc_plan_cache_entries(previous)
    for a, b_, c in zip(first, again, own):
        assert torch.equal(a, b_) and torch.equal(a, c)
    run()  # (disabling dropped the entry: keep one again, for the old ids)
    assert len(ops._DOC_PLAN_CACHE) == 1
    with torch.inference_mode():  # id tensors without a version counter: served, never kept
        ipos, iseq = pos.int().to(dev), seq.int().to(dev)
        o_inf = ops.attention(q.to(dev), k.to(dev), v.to(dev), mask_mode=ops.MASK_DOC, q_pos=ipos, k_pos=ipos, q_seq=iseq,
                              k_seq=iseq)
    assert torch.equal(o_inf, first[0]) and len(ops._DOC_PLAN_CACHE) == 1
    pos2, seq2 = make_docs(B, S, gen, 40, pad_tail=17)
    dpos.copy_(pos2)
    dseq.copy_(seq2)
    o2 = run()[0]
    assert len(ops._DOC_PLAN_CACHE) == 2  # same tensors, another version: a new plan beside the old one
    want, _ = oa.attention_with_lse(q.float(), k.float(), v.float(), oa.doc_mask(pos2, pos2, seq2, seq2))
    check(o2, want, torch.bfloat16, "O after the ids changed in place")


@pytest.mark.parametrize("ids_form", ["sequence-ids-only", "rank1-int32-host-positions"])
def test_model_step_builds_one_document_plan_for_all_layers(dev, ids_form):
    """A three-layer model step whose batch carries document ids runs the document-mask pre-pass ONCE (counted through
    the library's timer on it): the model canonicalises the ids once per forward, so all layers, forward and backward,
    hand the attention the same tensors; also through flash_attn_varlen, whose run ids are kept with the id tensor."""
    from maltos_amd import _lib
    from maltos_amd.constants import INPUT_IDS_KEY, LABELS_KEY, POSITION_IDS_KEY, SEQUENCE_IDS_KEY
    from maltos_amd.flash_utils import flash_attn_varlen
    from maltos_amd.llama import LlamaConfig, LlamaForCausalLM

    B, S = 2, 200
    gen = torch.Generator().manual_seed(77)
    cfg = LlamaConfig(vocab_size=512, hidden_size=256, intermediate_size=344, num_hidden_layers=3, num_attention_heads=4,
                      num_key_value_heads=2, max_position_embeddings=S)
    torch.manual_seed(5)
    model = LlamaForCausalLM(cfg).to(dev).to(torch.bfloat16)
    ids = torch.randint(0, 512, (B, S + 1), generator=gen)
    pos, seq = make_docs(B, S, gen, 60, pad_tail=0)
    batch = {INPUT_IDS_KEY: ids[:, :-1].to(dev), LABELS_KEY: ids[:, 1:].to(dev), SEQUENCE_IDS_KEY: seq.to(dev)}
    if ids_form == "rank1-int32-host-positions":   # ids that the per-layer canonicalisation would copy afresh per layer
        batch[POSITION_IDS_KEY] = torch.arange(S, dtype=torch.int32)
        batch[SEQUENCE_IDS_KEY] = seq.int()
    ops.clear_doc_plan_cache()
    _lib.kernel_timing(True)
    try:
        model(batch).backward()
        torch.cuda.synchronize()
        _, builds = _lib.kernel_time_ms("attn_doc_prepass")
    finally:
        _lib.kernel_timing(False)
    assert builds == 1, f"{builds} plan builds for 3 layers x (forward + backward)"
    # the varlen provider function: three calls on one id tensor share the run ids and so the plan
    q, k, v = (bshd(B, 2, S, 64, gen, torch.bfloat16).to(dev) for _ in range(3))
    dseq = seq.to(dev)
    ops.clear_doc_plan_cache()
    _lib.kernel_timing(True)
    try:
        outs = [flash_attn_varlen(q, k, v, dseq) for _ in range(3)]
        torch.cuda.synchronize()
        _, builds = _lib.kernel_time_ms("attn_doc_prepass")
    finally:
        _lib.kernel_timing(False)
    assert builds == 1 and torch.equal(outs[0], outs[2])
    dseq[:, S // 2:] += 1   # edited in place: the kept run ids are not used any more
    want, _ = oa.attention_with_lse(q.float().cpu(), k.float().cpu(), v.float().cpu(),
                                    oa.doc_mask(*(2 * [torch.arange(S).repeat(B, 1)]), dseq.cpu(), dseq.cpu()))
    check(flash_attn_varlen(q, k, v, dseq), want, torch.bfloat16, "varlen after the ids changed in place")


@pytest.mark.parametrize("dtype,D,mode", [(torch.bfloat16, 128, ops.MASK_CAUSAL), (torch.bfloat16, 64, ops.MASK_NONE),
                                          (torch.bfloat16, 128, ops.MASK_DOC), (torch.float32, 24, ops.MASK_CAUSAL)])
def test_backward_accumulation_modes(dev, dtype, D, mode):
    """mlts_attn_bwd's output modes against the plain one (everything in the input dtype, overwritten): fp32 gradients
    that are added to (all three, or dQ only with dK / dV written once in the input dtype) and the first block of such
    an accumulation, which overwrites the fp32 dQ instead of adding to it."""
    B, Hq, Hkv, Sq, Sk = 2, 4, 2, 333, 333
    gen = torch.Generator().manual_seed(400 + D)
    q, k, v, do = (bshd(B, h, s, D, gen, dtype).to(dev) for h, s in ((Hq, Sq), (Hkv, Sk), (Hkv, Sk), (Hq, Sq)))
    kw = {}
    if mode == ops.MASK_DOC:
        pos, seq = make_docs(B, Sq, gen, 90, pad_tail=7)
        kw = dict(q_pos=pos.to(dev), k_pos=pos.to(dev), q_seq=seq.to(dev), k_seq=seq.to(dev))
    o, lse = ops.attention_forward(q, k, v, mask_mode=mode, **kw)
    dq0, dk0, dv0 = ops.attention_backward(do, q, k, v, o, lse, mask_mode=mode, **kw)
    nan32 = lambda t: torch.full(t.shape, float("nan"), dtype=torch.float32, device=dev)
    # first block of an accumulation: dq (fp32) and dk, dv (input dtype) are all overwritten
    dq, dk, dv = nan32(q), torch.full_like(k, float("nan")), torch.full_like(v, float("nan"))
    ops.attention_backward_ring_block(do, q, k, v, o, lse, dq, dk, dv, first=True, mask_mode=mode, **kw)
    assert torch.equal(dq.to(dtype), dq0) and torch.equal(dk, dk0) and torch.equal(dv, dv0)
    # a later block: dq is added to, dk and dv are overwritten again
    first = dq.clone()
    dk.fill_(float("nan")), dv.fill_(float("nan"))
    ops.attention_backward_ring_block(do, q, k, v, o, lse, dq, dk, dv, first=False, mask_mode=mode, **kw)
    assert torch.equal(dq, first + first) and torch.equal(dk, dk0) and torch.equal(dv, dv0)
    # everything in fp32, added to
    dq, dk, dv = torch.ones_like(first), torch.ones(k.shape, device=dev), torch.ones(v.shape, device=dev)
    ops.attention_backward_accumulate(do, q, k, v, o, lse, dq, dk, dv, mask_mode=mode, **kw)
    tol = dict(rtol=1e-6, atol=1e-6)
    assert torch.allclose(dq, first + 1, **tol)   # (the product and the addition may be one fused operation)
    if dtype == torch.bfloat16:  # the fp32 values round to what the plain form stored
        assert torch.equal((dk - 1).to(dtype), dk0) or torch.allclose((dk - 1), dk0.float(), rtol=2.0 ** -7, atol=1e-5)
        assert torch.allclose(dv - 1, dv0.float(), rtol=2.0 ** -7, atol=1e-5)
    else:
        assert torch.allclose(dk - 1, dk0, **tol) and torch.allclose(dv - 1, dv0, **tol)


@pytest.mark.parametrize("D", [1, 3, 24, 96, 192])
def test_generic_head_dims(dev, D):
    run_case(dev, torch.float32, 1, 2, 1, 70, 70, D, ops.MASK_CAUSAL, seed=D)
    if D % 8 == 0:
        run_case(dev, torch.bfloat16, 1, 2, 2, 70, 70, D, ops.MASK_DOC, seed=D + 1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_padding_rows_give_zeros_and_no_nan(dev, dtype):
    o, lse = run_case(dev, dtype, 2, 2, 2, 200, 200, 64, ops.MASK_DOC, seed=77, max_doc=50, pad_tail=37)
    assert not o[:, :, -37:].any() and (lse[:, :, -37:] == float("-inf")).all()


@pytest.mark.parametrize("D", [64, 128])
def test_document_mask_irregular_rows(dev, D):
    """The document mask is a rule on (query, key) pairs, whatever the row looks like: ids that fall, an id that returns
    after another document, positions that restart or jump inside a run, padding in the middle, a zigzag order, next to
    a regular packed row in the same batch; with shared and with separate id tensors.  All against the oracle's rule."""
    S = 384
    gen = torch.Generator().manual_seed(5 + D)
    run_case(dev, torch.bfloat16, 2, 4, 2, S, S, D, ops.MASK_DOC, 21, max_doc=150, pad_tail=9, share_ids=False)
    pos_r, seq_r = make_docs(1, S, gen, 120, pad_tail=5)
    rows = [(pos_r[0], seq_r[0])]
    idx = torch.arange(S)
    rows.append((idx % 96, 3 - idx // 96))                                     # ids fall from run to run
    rows.append((idx % 64, (idx // 64) % 2))                                   # ids 0,1,0,1,...: a document in several runs
    rows.append((torch.where(idx < 200, idx, idx - 150), torch.zeros(S, dtype=torch.long)))  # positions restart inside a run
    seq_pad = (idx // 100).clone()
    seq_pad[150:170] = -1                                                      # padding in the middle
    rows.append((idx % 100, seq_pad))
    zig = torch.cat([idx[:96], idx[288:], idx[96:288]])                        # a chunk order that is not ascending
    rows.append((zig, torch.zeros(S, dtype=torch.long)))
    pos = torch.stack([r[0] for r in rows]).long()
    seq = torch.stack([r[1] for r in rows]).long()
    run_case(dev, torch.bfloat16, len(rows), 2, 1, S, S, D, ops.MASK_DOC, 22, ids=(pos, seq))
    run_case(dev, torch.float32, len(rows), 2, 1, 96, 96, 32, ops.MASK_DOC, 23, ids=(pos[:, :96], seq[:, :96]))


def test_reference_known_answers_through_hip(dev, known_answers):
    col = lambda vals: torch.tensor(vals, dtype=torch.float32, device=dev).view(1, 1, -1, 1)
    ka = known_answers["packed_doc_attention"]
    out = HipAttentionCore()(col(ka["q"]), col(ka["k"]), col(ka["v"]), 0, torch.tensor([ka["position_ids"]]),
                             torch.tensor([ka["sequence_ids"]]))
    assert torch.allclose(out.flatten().cpu(), torch.tensor(ka["expected"]), atol=ka["atol"])
    kc = known_answers["cross_chunk_attention"]
    ids = lambda key: torch.tensor([kc[key]], device=dev)
    out = causal_attention(col(kc["q"]), col(kc["k"]), col(kc["v"]), attention_backend="hip", warning_prefix="test",
                           q_positions=ids("q_positions"), k_positions=ids("k_positions"),
                           q_sequence_ids=ids("q_sequence_ids"), k_sequence_ids=ids("k_sequence_ids"),
                           flash_varlen_mode="prefix")
    assert torch.allclose(out.flatten().cpu(), torch.tensor(kc["expected"]), atol=kc["atol"])


def test_hip_backend_agrees_with_sdpa_backend_on_device(dev):
    gen = torch.Generator().manual_seed(5)
    q, k, v = (bshd(2, 4, 129, 64, gen, torch.float32).to(dev) for _ in range(3))
    a = causal_attention(q, k, v, attention_backend="hip", warning_prefix="t")
    b = causal_attention(q, k, v, attention_backend="sdpa_auto", warning_prefix="t")
    assert torch.allclose(a, b, atol=1e-5)
    pos, seq = make_docs(2, 129, gen, 40)
    kw = dict(q_positions=pos.to(dev), k_positions=pos.to(dev), q_sequence_ids=seq.to(dev), k_sequence_ids=seq.to(dev))
    a = causal_attention(q, k, v, attention_backend="hip", warning_prefix="t", **kw)
    b = causal_attention(q, k, v, attention_backend="eager", warning_prefix="t", **kw)
    assert torch.allclose(a, b, atol=1e-5)


def test_empty_and_error_cases(dev):
    z = torch.zeros(0, 2, 8, 64, device=dev, dtype=torch.bfloat16)
    o, lse = ops.attention_forward(z, z, z, mask_mode=ops.MASK_CAUSAL)
    assert o.shape == (0, 2, 8, 64) and lse.shape == (0, 2, 8)
    q = torch.randn(1, 2, 0, 64, device=dev)
    kv = torch.randn(1, 2, 5, 64, device=dev)
    o, lse = ops.attention_forward(q, kv, kv, mask_mode=ops.MASK_NONE)
    assert o.shape == (1, 2, 0, 64)
    q = torch.randn(1, 2, 4, 64, device=dev)
    o, lse = ops.attention_forward(q, kv[:, :, :0], kv[:, :, :0], mask_mode=ops.MASK_NONE)  # no keys: zeros, -inf
    assert not o.any() and (lse == float("-inf")).all()
    # the same on the bf16 MFMA kernels (head_dim 64 and 128), forward and backward
    for D in (64, 128):
        qb = torch.randn(1, 2, 40, D, device=dev).bfloat16()
        kb = torch.randn(1, 2, 0, D, device=dev).bfloat16()
        o, lse = ops.attention_forward(qb, kb, kb, mask_mode=ops.MASK_CAUSAL)
        assert o.dtype == torch.bfloat16 and not o.any() and (lse == float("-inf")).all()
        dq, dk, dv = ops.attention_backward(torch.ones_like(qb), qb, kb, kb, o, lse, mask_mode=ops.MASK_CAUSAL)
        assert not dq.any() and dk.shape == kb.shape and dv.shape == kb.shape
    with pytest.raises(ValueError):
        ops.attention(q, kv.half(), kv.half())
    with pytest.raises(ValueError):
        ops.attention(q, kv, kv, mask_mode=ops.MASK_DOC)  # ids missing
    with pytest.raises(ValueError):
        ops.attention(torch.randn(1, 1, 4, 300, device=dev), torch.randn(1, 1, 4, 300, device=dev), torch.randn(1, 1, 4, 300, device=dev))


@pytest.mark.parametrize("D,blk_dtype", [(128, torch.bfloat16), (64, torch.float32), (3, torch.float32)])
def test_merge_kernel(dev, D, blk_dtype):
    gen = torch.Generator().manual_seed(D)
    B, H, S = 2, 3, 50
    ro = torch.randn(B, H, S, D, generator=gen)
    rl = torch.randn(B, H, S, generator=gen)
    rl[0, 0, :5] = float("-inf")
    ro[0, 0, :5] = 0
    bo = torch.randn(B, S, H, D, generator=gen).to(blk_dtype).transpose(1, 2)
    bl = torch.randn(B, H, S, generator=gen)
    bl[0, 0, 3:8] = float("-inf")
    want_o, want_l = oa.merge_attention_blocks(ro.clone(), rl.clone(), bo, bl)
    go, gl = ro.to(dev), rl.to(dev)
    ops.attention_merge_(go, gl, bo.to(dev), bl.to(dev), 0)
    torch.testing.assert_close(go.cpu(), want_o, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(gl.cpu(), want_l, rtol=1e-5, atol=1e-6)
    # slice form
    want_o2, want_l2 = ro.clone(), rl.clone()
    oa.merge_attention_blocks(want_o2, want_l2, bo[:, :, :20], bl[:, :, :20], q_slice=slice(30, None))
    go, gl = ro.to(dev), rl.to(dev)
    ops.attention_merge_(go, gl, bo[:, :, :20].to(dev), bl[:, :, :20].contiguous().to(dev), 30)
    torch.testing.assert_close(go.cpu(), want_o2, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(gl.cpu(), want_l2, rtol=1e-5, atol=1e-6)
    with pytest.raises(ValueError):
        ops.attention_merge_(go, gl, bo[:, :, :20].to(dev), bl[:, :, :20].contiguous().to(dev), 40)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_block_functions_compose_with_global_lse(dev, dtype):
    """Two key blocks merged == one pass; block backwards fed the GLOBAL out/LSE sum to the full backward."""
    gen = torch.Generator().manual_seed(9)
    B, H, S, D = 1, 2, 192, 64
    q, k, v, do = (bshd(B, H, S, D, gen, dtype).to(dev) for _ in range(4))
    full = flash_attn_dense_with_lse(q, k, v, causal=False)
    a = flash_attn_dense_with_lse(q, k[:, :, :64], v[:, :, :64], causal=False)
    b = flash_attn_dense_with_lse(q, k[:, :, 64:], v[:, :, 64:], causal=False)
    ro = torch.zeros(B, H, S, D, device=dev)
    rl = torch.full((B, H, S), float("-inf"), device=dev)
    ops.attention_merge_(ro, rl, a.out, a.lse)
    ops.attention_merge_(ro, rl, b.out, b.lse)
    check(ro, full.out, dtype, "merged O")
    assert (rl - full.lse).abs().max() <= (1e-5 if dtype == torch.float32 else 1e-4)
    dq, dk, dv = flash_attn_dense_backward(do, q, k, v, full.out, full.lse, causal=False)
    dq1, dk1, dv1 = flash_attn_dense_backward(do, q, k[:, :, :64], v[:, :, :64], full.out, full.lse, causal=False)
    dq2, dk2, dv2 = flash_attn_dense_backward(do, q, k[:, :, 64:], v[:, :, 64:], full.out, full.lse, causal=False)
    check(dq1.float() + dq2.float(), dq, dtype, "dQ sum")
    check(torch.cat([dk1, dk2], 2), dk, dtype, "dK cat")
    check(torch.cat([dv1, dv2], 2), dv, dtype, "dV cat")
    want_o, want_lse = oa.attention_with_lse(q.cpu(), k.cpu(), v.cpu())
    check(full.out, want_o, dtype, "block O vs oracle")
    # differentiable dense causal entry point
    qg = q.clone().requires_grad_(True)
    flash_attn_dense(qg, k, v).backward(do)
    rq = q.cpu().float().requires_grad_(True)
    oa.attention_with_lse(rq, k.cpu(), v.cpu(), oa.causal_mask(S, S, "cpu"))[0].backward(do.cpu().float())
    check(qg.grad, rq.grad, dtype, "flash_attn_dense dQ")


def test_flash_attn_varlen_runs_and_padding(dev):
    gen = torch.Generator().manual_seed(13)
    ids = torch.tensor([[0, 0, 0, 1, 1, -1, 0, 0], [2, 2, 3, 3, 3, 3, -1, -1]])  # id 0 appears in two separate runs
    q, k, v = (bshd(2, 2, 8, 64, gen, torch.float32) for _ in range(3))
    out = flash_attn_varlen(q.to(dev), k.to(dev), v.to(dev), ids.to(dev)).cpu()
    runs = torch.tensor([[0, 0, 0, 1, 1, -1, 2, 2], [0, 0, 1, 1, 1, 1, -1, -1]])
    idx = torch.arange(8).unsqueeze(0).expand(2, -1)
    want, _ = oa.attention_with_lse(q, k, v, oa.doc_mask(idx, idx, runs, runs))
    assert torch.allclose(out, want, atol=1e-5)
    assert not out[0, :, 5].any() and not out[1, :, 6:].any()


def _ring_inputs(world_size, s_loc, B, H, D, dtype, seeds):
    total = s_loc * world_size
    mk = lambda s: torch.randn((B, H, total, D), generator=torch.Generator().manual_seed(s + world_size)).to(dtype)
    all_q, all_k, all_v = mk(seeds["q"]), mk(seeds["k"]), mk(seeds["v"])
    pos = [expected_zigzag_ring_positions(s_loc, rank=r, world_size=world_size, device=torch.device("cpu")) for r in range(world_size)]
    pick = lambda t: [t.index_select(2, p) for p in pos]
    return all_q, all_k, all_v, pos, pick(all_q), pick(all_k), pick(all_v)


@pytest.mark.parametrize("world_size", [2, 4])
def test_zigzag_ring_reference_vectors_fp32(dev, known_answers, world_size):
    spec = known_answers["zigzag_ring_schedule"]
    all_q, all_k, all_v, pos, qc, kc, vc = _ring_inputs(world_size, spec["local_seq_len"], spec["batch"], spec["heads"],
                                                        spec["head_dim"], torch.float32, spec["seed_offsets"])
    total = spec["local_seq_len"] * world_size
    gq, gk, gv = (t.clone().requires_grad_(True) for t in (all_q, all_k, all_v))
    gout, glse = oa.attention_with_lse(gq, gk, gv, oa.causal_mask(total, total, "cpu"))
    dout_all = torch.randn(gout.shape, generator=torch.Generator().manual_seed(99))
    gout.backward(dout_all)
    dk_sum, dv_sum = torch.zeros_like(all_k), torch.zeros_like(all_v)
    for rank in range(world_size):
        q = qc[rank].to(dev).requires_grad_(True)
        chunks = [(k.to(dev).requires_grad_(True), v.to(dev).requires_grad_(True)) for k, v in zip(kc, vc)]
        out, lse = zigzag_ring_attention(q, chunks, rank=rank, world_size=world_size, return_lse=True)
        assert torch.allclose(out.cpu(), gout.detach().index_select(2, pos[rank]), atol=spec["forward_atol"])
        assert torch.allclose(lse.cpu(), glse.detach().index_select(2, pos[rank]), atol=spec["forward_atol"])
        out.backward(dout_all.index_select(2, pos[rank]).to(dev))
        assert torch.allclose(q.grad.cpu(), gq.grad.index_select(2, pos[rank]), atol=spec["backward_atol"])
        for src, (k, v) in enumerate(chunks):
            dk_sum.index_add_(2, pos[src], k.grad.cpu())
            dv_sum.index_add_(2, pos[src], v.grad.cpu())
    assert torch.allclose(dk_sum, gk.grad, atol=spec["backward_atol"])
    assert torch.allclose(dv_sum, gv.grad, atol=spec["backward_atol"])


def test_zigzag_ring_bf16_matches_global_causal(dev):
    world_size, s_loc, B, H, D = 4, 256, 1, 2, 128
    all_q, all_k, all_v, pos, qc, kc, vc = _ring_inputs(world_size, s_loc, B, H, D, torch.bfloat16, dict(q=1, k=2, v=3))
    total = s_loc * world_size
    gq, gk, gv = (t.detach().float().clone().requires_grad_(True) for t in (all_q, all_k, all_v))
    gout, glse = oa.attention_with_lse(gq, gk, gv, oa.causal_mask(total, total, "cpu"))
    dout_all = torch.randn(gout.shape, generator=torch.Generator().manual_seed(7)).bfloat16()
    gout.backward(dout_all.float())
    dk_sum, dv_sum = torch.zeros_like(gk.grad), torch.zeros_like(gv.grad)
    for rank in range(world_size):
        q = qc[rank].to(dev).requires_grad_(True)
        chunks = [(k.to(dev).requires_grad_(True), v.to(dev).requires_grad_(True)) for k, v in zip(kc, vc)]
        core = HipRingAttentionCore(rank=rank, world_size=world_size, kv_source=lambda r, k, v, c=chunks: c)
        out = core(q, chunks[rank][0], chunks[rank][1], 0, pos[rank])
        check(out, gout.detach().index_select(2, pos[rank]), torch.bfloat16, f"ring O rank{rank}")
        out.backward(dout_all.index_select(2, pos[rank]).to(dev))
        check(q.grad, gq.grad.index_select(2, pos[rank]), torch.bfloat16, f"ring dQ rank{rank}")
        for src, (k, v) in enumerate(chunks):
            if k.grad is not None:
                dk_sum.index_add_(2, pos[src], k.grad.float().cpu())
                dv_sum.index_add_(2, pos[src], v.grad.float().cpu())
    # each chunk's dK/dV is the sum of four bf16-rounded rank contributions
    assert ((dk_sum - gk.grad).abs() <= 4 * (2e-2 + 2.0 ** -8 * gk.grad.abs())).all()
    assert ((dv_sum - gv.grad).abs() <= 4 * (2e-2 + 2.0 ** -8 * gv.grad.abs())).all()
    # world_size == 1 degenerates to plain causal attention
    solo = HipRingAttentionCore()(all_q[:, :, :256].to(dev), all_k[:, :, :256].to(dev), all_v[:, :, :256].to(dev), 0)
    want, _ = oa.attention_with_lse(all_q[:, :, :256], all_k[:, :, :256], all_v[:, :, :256], oa.causal_mask(256, 256, "cpu"))
    check(solo, want, torch.bfloat16, "single-rank ring")


def test_packed_ring_reference_scenario_fp32(dev, known_answers):
    """tests/sequence_ids_attention_mask.py:366-434 of the reference: two documents and a PAD token in zigzag order over
    two ranks; every rank's merged output equals global document-masked attention at its tokens."""
    spec = known_answers["packed_ring"]
    w, s_loc, total = spec["world_size"], spec["local_seq_len"], spec["local_seq_len"] * spec["world_size"]
    mk = lambda seed: torch.randn((spec["batch"], spec["heads"], total, spec["head_dim"]), generator=torch.Generator().manual_seed(seed))
    all_q, all_k, all_v = (mk(spec["seeds"][n]) for n in "qkv")
    all_pos = torch.tensor(spec["positions"]).view(1, total)
    all_seq = torch.tensor(spec["sequence_ids"]).view(1, total)
    idx = [expected_zigzag_ring_positions(s_loc, rank=r, world_size=w, device=torch.device("cpu")) for r in range(w)]
    gq, gk, gv = (t.clone().requires_grad_(True) for t in (all_q, all_k, all_v))
    gout, glse = oa.attention_with_lse(gq, gk, gv, oa.doc_mask(all_pos, all_pos, all_seq, all_seq))
    dout_all = torch.randn(gout.shape, generator=torch.Generator().manual_seed(5))
    gout.backward(dout_all)
    dk_sum, dv_sum = torch.zeros_like(all_k), torch.zeros_like(all_v)
    pc = [all_pos.index_select(1, i).to(dev) for i in idx]
    sc = [all_seq.index_select(1, i).to(dev) for i in idx]
    for rank in range(w):
        q = all_q.index_select(2, idx[rank]).to(dev).requires_grad_(True)
        chunks = [(all_k.index_select(2, i).to(dev).requires_grad_(True), all_v.index_select(2, i).to(dev).requires_grad_(True)) for i in idx]
        out, lse = packed_ring_attention(q, chunks, q_positions=pc[rank], q_sequence_ids=sc[rank], kv_positions=pc,
                                         kv_sequence_ids=sc, rank=rank, world_size=w, return_lse=True)
        assert torch.allclose(out.cpu(), gout.detach().index_select(2, idx[rank]), atol=spec["forward_atol"])
        want_lse = glse.index_select(2, idx[rank])
        fin = torch.isfinite(want_lse)
        assert torch.equal(torch.isfinite(lse.cpu()), fin)
        assert torch.allclose(lse.cpu()[fin], want_lse[fin], atol=spec["forward_atol"])
        out.backward(dout_all.index_select(2, idx[rank]).to(dev))
        assert torch.allclose(q.grad.cpu(), gq.grad.index_select(2, idx[rank]), atol=2e-5)
        for src, (k, v) in enumerate(chunks):
            dk_sum.index_add_(2, idx[src], k.grad.cpu())
            dv_sum.index_add_(2, idx[src], v.grad.cpu())
    assert torch.allclose(dk_sum, gk.grad, atol=2e-5)
    assert torch.allclose(dv_sum, gv.grad, atol=2e-5)


def test_prefix_function_set_drives_the_packed_ring_schedule(dev, known_answers):
    """The reference's packed-document ring (runtime/layers/functional.py:823-1009) written against the provider
    functions it calls, flash_attn_varlen_prefix_with_lse / _backward with allow_empty_kv=True, on the scenario of
    tests/sequence_ids_attention_mask.py:366-434: per step one block forward merged into the running state, in the
    backward one block backward from the merged out / LSE; the result is global document-masked attention."""
    spec = known_answers["packed_ring"]
    w, s_loc, total = spec["world_size"], spec["local_seq_len"], spec["local_seq_len"] * spec["world_size"]
    mk = lambda seed: torch.randn((spec["batch"], spec["heads"], total, spec["head_dim"]), generator=torch.Generator().manual_seed(seed))
    all_q, all_k, all_v = (mk(spec["seeds"][n]) for n in "qkv")
    all_pos = torch.tensor(spec["positions"]).view(1, total)
    all_seq = torch.tensor(spec["sequence_ids"]).view(1, total)
    idx = [expected_zigzag_ring_positions(s_loc, rank=r, world_size=w, device=torch.device("cpu")) for r in range(w)]
    gq, gk, gv = (t.clone().requires_grad_(True) for t in (all_q, all_k, all_v))
    gout, glse = oa.attention_with_lse(gq, gk, gv, oa.doc_mask(all_pos, all_pos, all_seq, all_seq))
    dout_all = torch.randn(gout.shape, generator=torch.Generator().manual_seed(5))
    gout.backward(dout_all)
    pc = [all_pos.index_select(1, i).to(dev) for i in idx]
    sc = [all_seq.index_select(1, i).to(dev) for i in idx]
    kc = [all_k.index_select(2, i).to(dev) for i in idx]
    vc = [all_v.index_select(2, i).to(dev) for i in idx]
    dk_sum, dv_sum = torch.zeros_like(all_k), torch.zeros_like(all_v)
    for rank in range(w):
        q = all_q.index_select(2, idx[rank]).to(dev)
        running_out = torch.zeros(q.shape, dtype=torch.float32, device=dev)
        running_lse = torch.full(q.shape[:-1], float("-inf"), dtype=torch.float32, device=dev)
        for step in range(w):
            src = (rank - step) % w
            block = flash_attn_varlen_prefix_with_lse(q, kc[src], vc[src], q_positions=pc[rank], k_positions=pc[src],
                                                      q_sequence_ids=sc[rank], k_sequence_ids=sc[src], allow_empty_kv=True)
            ops.attention_merge_(running_out, running_lse, block.out, block.lse)
        assert torch.allclose(running_out.cpu(), gout.detach().index_select(2, idx[rank]), atol=spec["forward_atol"])
        fin = torch.isfinite(glse.index_select(2, idx[rank]))
        assert torch.equal(torch.isfinite(running_lse.cpu()), fin)
        dout = dout_all.index_select(2, idx[rank]).to(dev)
        dq = torch.zeros_like(q)
        for step in range(w):
            src = (rank - step) % w
            bdq, bdk, bdv = flash_attn_varlen_prefix_backward(dout, q, kc[src], vc[src], running_out, running_lse, q_positions=pc[rank],
                                                              k_positions=pc[src], q_sequence_ids=sc[rank], k_sequence_ids=sc[src],
                                                              allow_empty_kv=True)
            dq += bdq
            dk_sum.index_add_(2, idx[src], bdk.cpu())
            dv_sum.index_add_(2, idx[src], bdv.cpu())
        assert torch.allclose(dq.cpu(), gq.grad.index_select(2, idx[rank]), atol=2e-5)
    assert torch.allclose(dk_sum, gk.grad, atol=2e-5) and torch.allclose(dv_sum, gv.grad, atol=2e-5)


def test_prefix_functions_empty_prefix_and_router_form(dev):
    """A chunk of queries at positions 0, 1, 6, 7 against keys at positions 2..5 (the reference's own empty-prefix vector,
    tests/sequence_ids_attention_mask.py:142-164): queries 0 and 1 see nothing.  allow_empty_kv=True gives zeros and
    LSE = -inf there (runtime/layers/flash_utils.py:810-819), the strict forms raise like the reference's packer; the
    differentiable form agrees with the oracle where every query has keys, GQA and bf16 included."""
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(1, 2, 4, 64, generator=g).to(dev) for _ in range(3))
    q_pos, k_pos = torch.tensor([[0, 1, 6, 7]], device=dev), torch.tensor([[2, 3, 4, 5]], device=dev)
    block = flash_attn_varlen_prefix_with_lse(q, k, v, q_positions=q_pos, k_positions=k_pos, allow_empty_kv=True)
    assert torch.equal(block.out[:, :, :2].cpu(), torch.zeros(1, 2, 2, 64)) and torch.isneginf(block.lse[:, :, :2]).all()
    want, want_lse = oa.attention_with_lse(q[:, :, 2:].cpu(), k.cpu(), v.cpu(), None)
    check(block.out[:, :, 2:], want, torch.float32, "prefix block")
    check(block.lse[:, :, 2:], want_lse, torch.float32, "prefix block LSE")
    dq, dk, dv = flash_attn_varlen_prefix_backward(torch.ones_like(q), q, k, v, block.out, block.lse, q_positions=q_pos, k_positions=k_pos,
                                                   allow_empty_kv=True)
    assert torch.equal(dq[:, :, :2].cpu(), torch.zeros(1, 2, 2, 64)) and torch.isfinite(dk).all() and torch.isfinite(dv).all()
    with pytest.raises(ValueError, match="without any matching key/value prefix"):
        flash_attn_varlen_prefix_with_lse(q, k, v, q_positions=q_pos, k_positions=k_pos)
    with pytest.raises(ValueError, match="without any matching key/value prefix"):
        flash_attn_varlen_prefix(q, k, v, q_positions=q_pos, k_positions=k_pos)
    with pytest.raises(ValueError, match="k_positions shape must match"):
        flash_attn_varlen_prefix(q, k, v, q_positions=q_pos, k_positions=k_pos[:, :3])

    gen = torch.Generator().manual_seed(9)
    B, Hq, Hkv, Sq, Sk, D = 2, 4, 2, 192, 320, 128
    pos, seq = make_docs(B, Sk, gen, 90, pad_tail=11)
    take = torch.arange(Sk - Sq, Sk)  # the queries are the last Sq tokens of the gathered keys
    qb, kb, vb, dob = bshd(B, Hq, Sq, D, gen, torch.bfloat16), bshd(B, Hkv, Sk, D, gen, torch.bfloat16), bshd(B, Hkv, Sk, D, gen, torch.bfloat16), bshd(B, Hq, Sq, D, gen, torch.bfloat16)
    qpos, qseq = pos[:, take], seq[:, take]
    qf, kf, vf = (t.detach().float().clone().requires_grad_(True) for t in (qb, kb, vb))
    want_o, _ = oa.attention_with_lse(qf, kf, vf, oa.doc_mask(qpos, pos, qseq, seq))
    want_o.backward(dob.float())
    qd, kd, vd = (t.to(dev).requires_grad_(True) for t in (qb, kb, vb))
    out = flash_attn_varlen_prefix(qd, kd, vd, q_positions=qpos.to(dev), k_positions=pos.to(dev), q_sequence_ids=qseq.to(dev),
                                   k_sequence_ids=seq.to(dev))
    out.backward(dob.to(dev))
    check(out, want_o.detach(), torch.bfloat16, "prefix O")
    check(qd.grad, qf.grad, torch.bfloat16, "prefix dQ")
    check(kd.grad, kf.grad, torch.bfloat16, "prefix dK")
    check(vd.grad, vf.grad, torch.bfloat16, "prefix dV")


@pytest.mark.parametrize("D", [64, 128])
def test_packed_ring_bf16_matches_global_document_attention(dev, D):
    world_size, s_loc, B, Hq, Hkv = 4, 256, 2, 4, 2
    total = world_size * s_loc
    gen = torch.Generator().manual_seed(40 + D)
    all_q, all_k, all_v = bshd(B, Hq, total, D, gen, torch.bfloat16), bshd(B, Hkv, total, D, gen, torch.bfloat16), bshd(B, Hkv, total, D, gen, torch.bfloat16)
    all_pos, all_seq = make_docs(B, total, gen, 400, pad_tail=37)
    idx = [expected_zigzag_ring_positions(s_loc, rank=r, world_size=world_size, device=torch.device("cpu")) for r in range(world_size)]
    gq, gk, gv = (t.detach().float().clone().requires_grad_(True) for t in (all_q, all_k, all_v))
    gout, _ = oa.attention_with_lse(gq, gk, gv, oa.doc_mask(all_pos, all_pos, all_seq, all_seq))
    dout_all = torch.randn(gout.shape, generator=gen).bfloat16()
    gout.backward(dout_all.float())
    dk_sum, dv_sum = torch.zeros_like(gk.grad), torch.zeros_like(gv.grad)
    pc = [all_pos.index_select(1, i).to(dev) for i in idx]
    sc = [all_seq.index_select(1, i).to(dev) for i in idx]
    for rank in range(world_size):
        q = all_q.index_select(2, idx[rank]).to(dev).requires_grad_(True)
        chunks = [(all_k.index_select(2, i).to(dev).requires_grad_(True), all_v.index_select(2, i).to(dev).requires_grad_(True)) for i in idx]
        core = HipRingAttentionCore(rank=rank, world_size=world_size, kv_source=lambda r, k, v, c=chunks: c,
                                    meta_source=lambda r, p, s: list(zip(pc, sc)))
        out = core(q, chunks[rank][0], chunks[rank][1], 0, pc[rank], sc[rank])
        check(out, gout.detach().index_select(2, idx[rank]), torch.bfloat16, f"packed ring O rank{rank}")
        out.backward(dout_all.index_select(2, idx[rank]).to(dev))
        check(q.grad, gq.grad.index_select(2, idx[rank]), torch.bfloat16, f"packed ring dQ rank{rank}")
        for src, (k, v) in enumerate(chunks):
            dk_sum.index_add_(2, idx[src], k.grad.float().cpu())
            dv_sum.index_add_(2, idx[src], v.grad.float().cpu())
    # each chunk's dK/dV is the sum of four bf16-rounded rank contributions
    assert ((dk_sum - gk.grad).abs() <= 4 * (2e-2 + 2.0 ** -8 * gk.grad.abs())).all()
    assert ((dv_sum - gv.grad).abs() <= 4 * (2e-2 + 2.0 ** -8 * gv.grad.abs())).all()


@pytest.mark.parametrize("packed", [False, True], ids=["positions-only", "packed-documents"])
def test_all_gather_kv_core_matches_global_attention(dev, packed):
    """Every rank's local queries over the gathered keys equal global (document-)causal attention at the rank's tokens,
    forward and backward; chunks are the zigzag split, so the gathered keys are not in position order."""
    from maltos_amd.all_gather_attention import HipAllGatherKvAttentionCore

    world_size, s_loc, B, Hq, Hkv, D = 4, 128, 2, 4, 2, 128
    total = world_size * s_loc
    gen = torch.Generator().manual_seed(77 + packed)
    all_q, all_k, all_v = bshd(B, Hq, total, D, gen, torch.bfloat16), bshd(B, Hkv, total, D, gen, torch.bfloat16), bshd(B, Hkv, total, D, gen, torch.bfloat16)
    if packed:
        all_pos, all_seq = make_docs(B, total, gen, 200, pad_tail=19)
        mask = oa.doc_mask(all_pos, all_pos, all_seq, all_seq)
    else:
        all_pos, all_seq = torch.arange(total).expand(B, total).contiguous(), None
        mask = oa.causal_mask(total, total, "cpu")
    idx = [expected_zigzag_ring_positions(s_loc, rank=r, world_size=world_size, device=torch.device("cpu")) for r in range(world_size)]
    gq, gk, gv = (t.detach().float().clone().requires_grad_(True) for t in (all_q, all_k, all_v))
    gout, _ = oa.attention_with_lse(gq, gk, gv, mask)
    dout_all = torch.randn(gout.shape, generator=gen).bfloat16()
    gout.backward(dout_all.float())
    dk_sum, dv_sum = torch.zeros_like(gk.grad), torch.zeros_like(gv.grad)
    pc = [all_pos.index_select(1, i).to(dev) for i in idx]
    sc = [all_seq.index_select(1, i).to(dev) if packed else None for i in idx]
    for rank in range(world_size):
        q = all_q.index_select(2, idx[rank]).to(dev).requires_grad_(True)
        chunks = [(all_k.index_select(2, i).to(dev).requires_grad_(True), all_v.index_select(2, i).to(dev).requires_grad_(True)) for i in idx]
        core = HipAllGatherKvAttentionCore(rank=rank, world_size=world_size, kv_source=lambda r, k, v, c=chunks: c,
                                           meta_source=lambda r, p, s: list(zip(pc, sc)))
        out = core(q, chunks[rank][0], chunks[rank][1], 0, pc[rank], sc[rank])
        check(out, gout.detach().index_select(2, idx[rank]), torch.bfloat16, f"all-gather O rank{rank}")
        out.backward(dout_all.index_select(2, idx[rank]).to(dev))
        check(q.grad, gq.grad.index_select(2, idx[rank]), torch.bfloat16, f"all-gather dQ rank{rank}")
        for src, (k, v) in enumerate(chunks):
            dk_sum.index_add_(2, idx[src], k.grad.float().cpu())
            dv_sum.index_add_(2, idx[src], v.grad.float().cpu())
    assert ((dk_sum - gk.grad).abs() <= 4 * (2e-2 + 2.0 ** -8 * gk.grad.abs())).all()
    assert ((dv_sum - gv.grad).abs() <= 4 * (2e-2 + 2.0 ** -8 * gv.grad.abs())).all()


def test_tensors_of_more_than_two_to_the_31_elements(dev):
    """q, k, v of 2^31 elements each (B=4, H=32, S=131072, D=128: element offsets past 32 bits): the first and the last
    (batch, head) pair come out exactly as from a call on that pair alone, forward and backward; a size-independent
    property where the oracle cannot go."""
    B, H, S, D = 4, 32, 131072, 128
    gen = torch.Generator(device=dev).manual_seed(11)
    q, k, v, do = (torch.randn(B, S, H, D, generator=gen, device=dev, dtype=torch.bfloat16).transpose(1, 2) for _ in range(4))
    assert q.numel() == 2 ** 31
    o, lse = ops.attention_forward(q, k, v, mask_mode=ops.MASK_CAUSAL)
    dq, dk, dv = ops.attention_backward(do, q, k, v, o, lse, mask_mode=ops.MASK_CAUSAL)
    for b, h in ((0, 0), (B - 1, H - 1)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        o1, lse1 = ops.attention_forward(q[sl], k[sl], v[sl], mask_mode=ops.MASK_CAUSAL)
        assert torch.equal(o[sl], o1) and torch.equal(lse[sl], lse1), (b, h)
        for got, want, name in zip((dq, dk, dv), ops.attention_backward(do[sl], q[sl], k[sl], v[sl], o1, lse1, mask_mode=ops.MASK_CAUSAL),
                                   ("dQ", "dK", "dV")):
            assert torch.equal(got[sl], want), (b, h, name)
    # and the last rows against the oracle: the last 64 queries of the last pair see all 131072 keys
    sl = (slice(B - 1, B), slice(H - 1, H))
    qf, kf, vf = q[sl][:, :, -64:].float().cpu(), k[sl].float().cpu(), v[sl].float().cpu()
    want_o, want_lse = oa.attention_with_lse(qf, kf, vf, oa.causal_mask(64, S, "cpu"))
    check(o[sl][:, :, -64:], want_o, torch.bfloat16, "last rows O")
    assert (lse[sl][:, :, -64:].cpu() - want_lse).abs().max() <= 1e-4
