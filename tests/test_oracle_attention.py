"""Pins oracle/attention.py.

What pins what:
  * attention_with_lse + example_causal_mask : reference known answers (packed_doc_attention,
    cross_chunk_attention), F.scaled_dot_product_attention (library), brute-force per-row softmax.
  * attention_backward_explicit              : torch autograd of the forward (independent derivation),
    including GQA and fully masked rows.
  * merge_attention_blocks                   : splitting the key set in two and merging reproduces the
    unsplit attention; -inf blocks are no-ops; q_slice form equals the full form on the slice.
  * zigzag_positions / zigzag_schedule / zigzag_ring_forward / _backward : reference known answer
    [0,1,6,7], the reference's expected call list, and the invariant "ring == one global causal
    attention at the rank's positions" for W in {2,4} with the reference's seeds (fwd 1e-5, bwd 2e-5).
  * online_softmax_update                    : equals attention_with_lse when fed the keys in two pieces.
  * varlen_metadata                          : reference known answers incl. the post-edit vector.
"""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import attention as oa


def _col(values):
    return torch.tensor(values, dtype=torch.float32).view(1, 1, -1, 1)


def test_packed_doc_known_answer(known_answers):
    ka = known_answers["packed_doc_attention"]
    pos = torch.tensor([ka["position_ids"]])
    seq = torch.tensor([ka["sequence_ids"]])
    mask = oa.example_causal_mask(pos, pos, seq, seq).unsqueeze(1)
    out, _ = oa.attention_with_lse(_col(ka["q"]), _col(ka["k"]), _col(ka["v"]), mask)
    assert torch.allclose(out.flatten(), torch.tensor(ka["expected"]), atol=ka["atol"])


def test_cross_chunk_known_answer(known_answers):
    ka = known_answers["cross_chunk_attention"]
    mask = oa.example_causal_mask(torch.tensor([ka["q_positions"]]), torch.tensor([ka["k_positions"]]),
                                  torch.tensor([ka["q_sequence_ids"]]), torch.tensor([ka["k_sequence_ids"]])).unsqueeze(1)
    out, _ = oa.attention_with_lse(_col(ka["q"]), _col(ka["k"]), _col(ka["v"]), mask)
    assert torch.allclose(out.flatten(), torch.tensor(ka["expected"]), atol=ka["atol"])


def test_mask_brute_force():
    g = torch.Generator().manual_seed(7)
    qp = torch.randint(0, 6, (2, 5), generator=g)
    kp = torch.randint(0, 6, (2, 7), generator=g)
    qs = torch.randint(0, 3, (2, 5), generator=g)
    ks = torch.randint(0, 3, (2, 7), generator=g)
    m = oa.example_causal_mask(qp, kp, qs, ks)
    for b in range(2):
        for i in range(5):
            for j in range(7):
                assert bool(m[b, i, j]) == (kp[b, j] <= qp[b, i] and qs[b, i] == ks[b, j])
    with pytest.raises(ValueError):
        oa.example_causal_mask(qp, kp, qs, None)


@pytest.mark.parametrize("hq,hkv", [(4, 4), (4, 2)])
def test_forward_matches_sdpa_library(hq, hkv):
    g = torch.Generator().manual_seed(11)
    q = torch.randn(2, hq, 33, 16, generator=g)
    k = torch.randn(2, hkv, 33, 16, generator=g)
    v = torch.randn(2, hkv, 33, 16, generator=g)
    out, lse = oa.attention_with_lse(q, k, v, oa.causal_mask(33, 33, "cpu"))
    rep = hq // hkv
    ref = F.scaled_dot_product_attention(q, oa.repeat_kv(k, rep), oa.repeat_kv(v, rep), is_causal=True)
    assert torch.allclose(out, ref, atol=1e-5)
    # brute-force LSE of one row
    s = (q[1, 3, 20] @ oa.repeat_kv(k, rep)[1, 3, :21].T) / math.sqrt(16)
    assert abs(lse[1, 3, 20].item() - torch.logsumexp(s, 0).item()) < 1e-5


def test_fully_masked_rows_are_zero_with_neg_inf_lse():
    q = torch.randn(1, 1, 3, 4)
    k = torch.randn(1, 1, 2, 4)
    v = torch.randn(1, 1, 2, 4)
    mask = torch.tensor([[True, False], [False, False], [True, True]]).view(1, 1, 3, 2)
    out, lse = oa.attention_with_lse(q, k, v, mask)
    assert torch.equal(out[0, 0, 1], torch.zeros(4)) and lse[0, 0, 1] == float("-inf")
    assert torch.isfinite(out).all()


@pytest.mark.parametrize("hq,hkv,masked", [(2, 2, False), (4, 2, True)])
def test_explicit_backward_matches_autograd(hq, hkv, masked):
    g = torch.Generator().manual_seed(5)
    q = torch.randn(2, hq, 9, 8, generator=g, requires_grad=True)
    k = torch.randn(2, hkv, 11, 8, generator=g, requires_grad=True)
    v = torch.randn(2, hkv, 11, 8, generator=g, requires_grad=True)
    do = torch.randn(2, hq, 9, 8, generator=g)
    mask = oa.causal_mask(9, 11, "cpu")
    if masked:
        mask = mask.clone().expand(2, 1, 9, 11).clone()
        mask[0, 0, 4, :] = False  # a fully masked query row
    out, lse = oa.attention_with_lse(q, k, v, mask)
    out.backward(do)
    dq, dk, dv = oa.attention_backward_explicit(do, q.detach(), k.detach(), v.detach(), out.detach(), lse.detach(), mask)
    assert torch.allclose(dq, q.grad, atol=1e-5)
    assert torch.allclose(dk, k.grad, atol=1e-5)
    assert torch.allclose(dv, v.grad, atol=1e-5)


def test_merge_equals_unsplit_attention_and_handles_empty_blocks():
    g = torch.Generator().manual_seed(3)
    q = torch.randn(1, 2, 6, 8, generator=g)
    k = torch.randn(1, 2, 10, 8, generator=g)
    v = torch.randn(1, 2, 10, 8, generator=g)
    full, full_lse = oa.attention_with_lse(q, k, v)
    o1, l1 = oa.attention_with_lse(q, k[:, :, :4], v[:, :, :4])
    o2, l2 = oa.attention_with_lse(q, k[:, :, 4:], v[:, :, 4:])
    ro = torch.zeros_like(full)
    rl = torch.full(full_lse.shape, float("-inf"))
    ro, rl = oa.merge_attention_blocks(ro, rl, o1, l1)
    ro, rl = oa.merge_attention_blocks(ro, rl, o2, l2)
    assert torch.allclose(ro, full, atol=1e-6) and torch.allclose(rl, full_lse, atol=1e-6)
    # an empty block (zeros, lse=-inf) is a no-op, and merging two empties stays empty without NaN
    ro2, rl2 = oa.merge_attention_blocks(ro.clone(), rl.clone(), torch.zeros_like(ro), torch.full_like(rl, float("-inf")))
    assert torch.equal(ro2, ro) and torch.equal(rl2, rl)
    e_o, e_l = oa.merge_attention_blocks(torch.zeros_like(ro), torch.full_like(rl, float("-inf")), torch.zeros_like(ro),
                                         torch.full_like(rl, float("-inf")))
    assert torch.equal(e_o, torch.zeros_like(ro)) and (e_l == float("-inf")).all()
    # q_slice form == full form restricted to the slice
    so, sl = ro.clone(), rl.clone()
    oa.merge_attention_blocks(so, sl, o1[:, :, 3:], l1[:, :, 3:], q_slice=slice(3, None))
    fo, fl = oa.merge_attention_blocks(ro[:, :, 3:], rl[:, :, 3:], o1[:, :, 3:], l1[:, :, 3:])
    assert torch.allclose(so[:, :, 3:], fo) and torch.allclose(sl[:, :, 3:], fl) and torch.equal(so[:, :, :3], ro[:, :, :3])


def test_zigzag_positions_known_answer(known_answers):
    ka = known_answers["zigzag_positions"]
    got = oa.zigzag_positions(ka["local_seq_len"], rank=ka["rank"], world_size=ka["world_size"])
    assert got.tolist() == ka["expected"]
    with pytest.raises(ValueError):
        oa.zigzag_positions(5, rank=0, world_size=2)
    # every position is owned exactly once
    w = 4
    owned = torch.cat([oa.zigzag_positions(6, rank=r, world_size=w) for r in range(w)])
    assert sorted(owned.tolist()) == list(range(6 * w))


def _ring_setup(world_size, spec):
    b, h, s_loc, d = spec["batch"], spec["heads"], spec["local_seq_len"], spec["head_dim"]
    total = s_loc * world_size
    off = spec["seed_offsets"]
    mk = lambda o: torch.randn((b, h, total, d), generator=torch.Generator().manual_seed(o + world_size))
    all_q, all_k, all_v = mk(off["q"]), mk(off["k"]), mk(off["v"])
    pos = [oa.zigzag_positions(s_loc, rank=r, world_size=world_size) for r in range(world_size)]
    pick = lambda t: [t.index_select(2, p) for p in pos]
    return all_q, all_k, all_v, pos, pick(all_q), pick(all_k), pick(all_v)


@pytest.mark.parametrize("world_size", [2, 4])
def test_zigzag_ring_forward_schedule_and_invariant(known_answers, world_size):
    spec = known_answers["zigzag_ring_schedule"]
    all_q, all_k, all_v, pos, qc, kc, vc = _ring_setup(world_size, spec)
    s_loc, half = spec["local_seq_len"], spec["local_seq_len"] // 2
    total = s_loc * world_size
    for rank in range(world_size):
        out, lse, calls = oa.zigzag_ring_forward(qc[rank], list(zip(kc, vc)), rank=rank, world_size=world_size)
        expected_calls = [(s_loc, s_loc, True)] + [
            (s_loc, half, False) if step <= rank else (half, s_loc, False) for step in range(1, world_size)
        ]
        assert calls == expected_calls
        mask = (torch.arange(total)[None, :] <= pos[rank][:, None]).view(1, 1, s_loc, total)
        ref, ref_lse = oa.attention_with_lse(qc[rank], all_k, all_v, mask)
        assert torch.allclose(out, ref, atol=spec["forward_atol"])
        assert torch.allclose(lse, ref_lse, atol=spec["forward_atol"])


@pytest.mark.parametrize("world_size", [2, 4])
def test_zigzag_ring_backward_invariant(known_answers, world_size):
    spec = known_answers["zigzag_ring_schedule"]
    all_q, all_k, all_v, pos, qc, kc, vc = _ring_setup(world_size, spec)
    s_loc = spec["local_seq_len"]
    total = s_loc * world_size
    gq, gk, gv = (t.clone().requires_grad_(True) for t in (all_q, all_k, all_v))
    gout, _ = oa.attention_with_lse(gq, gk, gv, oa.causal_mask(total, total, "cpu"))
    dout_all = torch.randn(gout.shape, generator=torch.Generator().manual_seed(99))
    gout.backward(dout_all)
    dk_sum = torch.zeros_like(all_k)
    dv_sum = torch.zeros_like(all_v)
    for rank in range(world_size):
        out, lse, _ = oa.zigzag_ring_forward(qc[rank], list(zip(kc, vc)), rank=rank, world_size=world_size)
        dq, dkv = oa.zigzag_ring_backward(dout_all.index_select(2, pos[rank]), qc[rank], list(zip(kc, vc)), out, lse,
                                          rank=rank, world_size=world_size)
        assert torch.allclose(dq, gq.grad.index_select(2, pos[rank]), atol=spec["backward_atol"])
        for src, (dk, dv) in dkv.items():
            dk_sum.index_add_(2, pos[src], dk)
            dv_sum.index_add_(2, pos[src], dv)
    assert torch.allclose(dk_sum, gk.grad, atol=spec["backward_atol"])
    assert torch.allclose(dv_sum, gv.grad, atol=spec["backward_atol"])


def _packed_ring_setup(spec):
    """The reference's packed-ring scenario: two documents and a PAD token, spread over the ranks in zigzag order."""
    b, h, s_loc, d, w = spec["batch"], spec["heads"], spec["local_seq_len"], spec["head_dim"], spec["world_size"]
    total = s_loc * w
    mk = lambda seed: torch.randn((b, h, total, d), generator=torch.Generator().manual_seed(seed))
    all_q, all_k, all_v = (mk(spec["seeds"][n]) for n in "qkv")
    all_pos = torch.tensor(spec["positions"]).view(1, total).expand(b, total)
    all_seq = torch.tensor(spec["sequence_ids"]).view(1, total).expand(b, total)
    idx = [oa.zigzag_positions(s_loc, rank=r, world_size=w) for r in range(w)]
    pick = lambda t, dim: [t.index_select(dim, i) for i in idx]
    return all_q, all_k, all_v, all_pos, all_seq, idx, pick


def test_packed_ring_equals_global_document_attention(known_answers):
    spec = known_answers["packed_ring"]
    w = spec["world_size"]
    all_q, all_k, all_v, all_pos, all_seq, idx, pick = _packed_ring_setup(spec)
    qc, kc, vc, pc, sc = pick(all_q, 2), pick(all_k, 2), pick(all_v, 2), pick(all_pos, 1), pick(all_seq, 1)
    gq, gk, gv = (t.clone().requires_grad_(True) for t in (all_q, all_k, all_v))
    gout, glse = oa.attention_with_lse(gq, gk, gv, oa.doc_mask(all_pos, all_pos, all_seq, all_seq))
    # brute force of the rule the reference's test states, independent of doc_mask
    for i in range(all_q.size(2)):
        vis = [j for j in range(all_q.size(2)) if spec["sequence_ids"][i] >= 0
               and spec["sequence_ids"][j] == spec["sequence_ids"][i] and spec["positions"][j] <= spec["positions"][i]]
        if not vis:
            assert gout[0, 0, i].abs().max() == 0
            continue
        p = torch.softmax(all_q[0, 0, i] @ all_k[0, 0, vis].T * all_q.size(-1) ** -0.5, dim=-1)
        assert torch.allclose(gout[0, 0, i], p @ all_v[0, 0, vis], atol=1e-6)
    dout_all = torch.randn(gout.shape, generator=torch.Generator().manual_seed(5))
    gout.backward(dout_all)
    dk_sum, dv_sum = torch.zeros_like(all_k), torch.zeros_like(all_v)
    for rank in range(w):
        out, lse = oa.packed_ring_forward(qc[rank], list(zip(kc, vc)), pc[rank], sc[rank], list(zip(pc, sc)), rank=rank,
                                          world_size=w)
        assert torch.allclose(out, gout.detach().index_select(2, idx[rank]), atol=spec["forward_atol"])
        want_lse = glse.index_select(2, idx[rank])
        assert torch.equal(torch.isfinite(lse), torch.isfinite(want_lse))
        assert torch.allclose(lse[torch.isfinite(lse)], want_lse[torch.isfinite(lse)], atol=spec["forward_atol"])
        dq, dkv = oa.packed_ring_backward(dout_all.index_select(2, idx[rank]), qc[rank], list(zip(kc, vc)), pc[rank],
                                          sc[rank], list(zip(pc, sc)), out, lse, rank=rank, world_size=w)
        assert torch.allclose(dq, gq.grad.index_select(2, idx[rank]), atol=2e-5)
        for src, (dk, dv) in dkv.items():
            dk_sum.index_add_(2, idx[src], dk)
            dv_sum.index_add_(2, idx[src], dv)
    assert torch.allclose(dk_sum, gk.grad, atol=2e-5)
    assert torch.allclose(dv_sum, gv.grad, atol=2e-5)


def test_online_softmax_equals_attention():
    g = torch.Generator().manual_seed(21)
    q = torch.randn(1, 2, 5, 8, generator=g)
    k = torch.randn(1, 2, 12, 8, generator=g)
    v = torch.randn(1, 2, 12, 8, generator=g)
    mask = oa.causal_mask(5, 12, "cpu").expand(1, 2, 5, 12)
    rm = torch.full((1, 2, 5), float("-inf"))
    rs = torch.zeros(1, 2, 5)
    ra = torch.zeros(1, 2, 5, 8)
    for lo, hi in ((0, 7), (7, 12)):
        rm, rs, ra = oa.online_softmax_update(q, k[:, :, lo:hi], v[:, :, lo:hi], mask[..., lo:hi], rm, rs, ra)
    ref, _ = oa.attention_with_lse(q, k, v, mask)
    assert torch.allclose(ra / rs.clamp_min(1e-20).unsqueeze(-1), ref, atol=1e-6)


def test_varlen_metadata_known_answers(known_answers):
    ka = known_answers["varlen_metadata"]
    ids = torch.tensor(ka["sequence_ids"])
    cu, mx, mask = oa.varlen_metadata(ids)
    assert cu.tolist() == ka["cu_seqlens"] and mx == ka["max_seqlen"] and mask.tolist() == ka["token_mask"]
    e = ka["after_edit"]
    ids[e["row"], e["col"]] = e["value"]
    assert oa.varlen_metadata(ids)[0].tolist() == e["cu_seqlens"]
    dense = known_answers["dense_varlen_pack"]
    cu, mx, _ = oa.varlen_metadata(torch.arange(dense["batch"]).unsqueeze(1).expand(-1, dense["seq"]))
    assert cu.tolist() == dense["cu_seqlens"] and mx == dense["max_seqlen"]
    assert oa.varlen_metadata(torch.full((2, 3), -1))[0].tolist() == [0]
