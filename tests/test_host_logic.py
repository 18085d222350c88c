"""CPU tests of the product's host side: the C-ABI library loads and exports every declared symbol,
argument validation raises before any launch, and the host-side mirrors of the reference's helpers
(ids, mask rule, zigzag layout, ring schedule, varlen metadata, backend names, optimizer plumbing)
behave as the reference's tests expect.  No kernel is launched here."""
import ctypes
import re
from pathlib import Path

import pytest
import torch

import maltos_amd
from maltos_amd import _lib, ops
from maltos_amd.attention_backend import (ATTENTION_BACKEND_CHOICES, AttentionBackend, causal_attention,
                                          validate_attention_backend)
from maltos_amd.attn_masking_utils import build_example_causal_mask, canonical_position_ids, canonical_sequence_ids
from maltos_amd.flash_utils import varlen_prefix_metadata, varlen_qkv_metadata
from maltos_amd.optim import FusedAdamW, MasterWeightsOptimizer
from maltos_amd.ring_attention import zigzag_ring_schedule
from maltos_amd.ring_layout import expected_zigzag_ring_positions, has_zigzag_ring_layout

ROOT = Path(__file__).resolve().parent.parent


def _declared_symbols():
    text = (ROOT / "include" / "maltos_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mlts_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert len(names) >= 20
    assert set(names) == set(_lib.SIGNATURES), "include/maltos_hip.h and maltos_amd/_lib.py disagree"
    handle = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in names:
        assert hasattr(handle, name), f"{name} not exported by {_lib.LIB_PATH.name}"
    assert _lib.lib().mlts_abi_version() == 4


def test_entry_points_validate_before_launch():
    L = _lib.lib()
    # no GPU is touched: every call fails validation on the host
    assert L.mlts_adamw_step(None, None, None, None, None, 16, 1e-3, 0.9, 0.95, 1e-8, 0.0, 1, 1.0, None, 0.0, None) == _lib.MLTS_ERR_INVALID
    assert "non-null" in _lib.last_error()
    assert L.mlts_adamw_step(None, None, None, None, None, 0, 1e-3, 0.9, 0.95, 1e-8, 0.0, 1, 1.0, None, 0.0, None) == _lib.MLTS_OK
    assert L.mlts_rmsnorm_fwd(None, None, None, None, 4, 30, 1e-5, _lib.MLTS_BF16, None) == _lib.MLTS_ERR_INVALID
    assert "multiple of 8" in _lib.last_error()
    shape = _lib.AttnShape()
    shape.B, shape.Hq, shape.Hkv, shape.Sq, shape.Sk, shape.D = 1, 3, 2, 8, 8, 64
    shape.dtype, shape.mask_mode, shape.scale = _lib.MLTS_BF16, _lib.MASK_CAUSAL, 0.125
    assert b"multiple of Hkv" in L.mlts_attn_supports(ctypes.byref(shape))
    shape.Hkv = 1
    shape.mask_mode = _lib.MASK_DOC
    assert b"MLTS_MASK_DOC needs" in L.mlts_attn_supports(ctypes.byref(shape))
    shape.mask_mode = _lib.MASK_CAUSAL
    for arr in (shape.q_stride, shape.k_stride, shape.v_stride, shape.o_stride):
        arr[0], arr[1], arr[2] = 8 * 3 * 64, 64, 3 * 64
    assert L.mlts_attn_supports(ctypes.byref(shape)) is None
    assert L.mlts_attn_fwd_workspace_bytes(ctypes.byref(shape)) == 0
    assert L.mlts_attn_bwd_workspace_bytes(ctypes.byref(shape), 0) >= L.mlts_attn_bwd_workspace_bytes(ctypes.byref(shape), 1) > 0
    # the workspace is O(B * Hq * Sq)
    assert L.mlts_attn_bwd_workspace_bytes(ctypes.byref(shape), 0) < 64 * 1024
    shape.D = 128
    for arr in (shape.q_stride, shape.k_stride, shape.v_stride, shape.o_stride):
        arr[0], arr[1], arr[2] = 8 * 3 * 128, 128, 3 * 128
    # rows further apart than 2^24 elements are refused (the MFMA kernels address a tile's rows with 32-bit offsets)
    shape.k_stride[2] = 1 << 24
    assert b"2^24" in L.mlts_attn_supports(ctypes.byref(shape))
    shape.k_stride[2] = 3 * 128
    # the entry point without a workspace refuses shapes beyond its built-in buffer before touching any pointer
    shape.B, shape.Hq, shape.Hkv, shape.Sq, shape.Sk = 1, 64, 64, 32768, 32768
    st = (ctypes.c_int64 * 3)(64 * 32768 * 128, 32768 * 128, 128)
    for arr in (shape.q_stride, shape.k_stride, shape.v_stride, shape.o_stride):
        arr[0], arr[1], arr[2] = st[0], st[1], st[2]
    assert L.mlts_attn_bwd_noalloc(ctypes.byref(shape), None, st, None, None, None, None, None, None, st, None, st, None, st, 0, None) == _lib.MLTS_ERR_INVALID
    assert "built-in scratch" in _lib.last_error()
    with pytest.raises(ValueError):
        _lib.check(_lib.MLTS_ERR_INVALID)
    with pytest.raises(RuntimeError):
        _lib.check(_lib.MLTS_ERR_UNSUPPORTED)


def test_ops_refuse_host_tensors():
    x = torch.randn(4, 8)
    with pytest.raises(RuntimeError, match="no CPU"):
        ops.rms_norm(x, torch.ones(8), 1e-5)
    with pytest.raises(RuntimeError, match="no CPU|GPU only"):
        ops.attention(torch.randn(1, 1, 4, 8), torch.randn(1, 1, 4, 8), torch.randn(1, 1, 4, 8))
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.adamw_step_(torch.zeros(8), torch.zeros(8), torch.zeros(8), torch.zeros(8), lr=1e-3, beta1=0.9, beta2=0.95,
                        eps=1e-8, weight_decay=0.0, step=1)
    with pytest.raises(ValueError):
        ops.attention(torch.randn(1, 3, 4, 8), torch.randn(1, 2, 4, 8), torch.randn(1, 2, 4, 8))
    with pytest.raises(RuntimeError, match="cannot run"):
        causal_attention(x.view(1, 1, 4, 8), x.view(1, 1, 4, 8), x.view(1, 1, 4, 8), attention_backend="hip", warning_prefix="t")


def test_canonical_ids_and_mask_rule(known_answers):
    dev = torch.device("cpu")
    assert canonical_position_ids(None, batch_size=2, seq_len=3, position_offset=5, device=dev).tolist() == [[5, 6, 7]] * 2
    assert canonical_position_ids(torch.tensor([4, 2, 0]), batch_size=2, seq_len=3, position_offset=0, device=dev).tolist() == [[4, 2, 0]] * 2
    assert canonical_sequence_ids(None, batch_size=2, seq_len=3, device=dev) is None
    assert canonical_sequence_ids(torch.tensor([[1, 1, 2]], dtype=torch.int32), batch_size=1, seq_len=3, device=dev).dtype == torch.long
    for bad in (torch.zeros(4), torch.zeros(3, 3), torch.zeros(1, 1, 3)):
        with pytest.raises(ValueError):
            canonical_position_ids(bad, batch_size=2, seq_len=3, position_offset=0, device=dev)
        with pytest.raises(ValueError):
            canonical_sequence_ids(bad, batch_size=2, seq_len=3, device=dev)
    ka = known_answers["cross_chunk_attention"]
    mask = build_example_causal_mask(q_positions=torch.tensor([ka["q_positions"]]), k_positions=torch.tensor([ka["k_positions"]]),
                                     q_sequence_ids=torch.tensor([ka["q_sequence_ids"]]),
                                     k_sequence_ids=torch.tensor([ka["k_sequence_ids"]]))
    assert mask[0].tolist() == [[False, False, False, True, False, False], [False, False, False, True, True, False],
                                [False, False, False, True, True, True]]
    with pytest.raises(ValueError):
        build_example_causal_mask(q_positions=torch.zeros(3), k_positions=torch.zeros(1, 3))
    with pytest.raises(ValueError):
        build_example_causal_mask(q_positions=torch.zeros(1, 3), k_positions=torch.zeros(1, 3), q_sequence_ids=torch.zeros(1, 3))
    # eager backend through the router reproduces the reference known answer on CPU
    col = lambda v: torch.tensor(v, dtype=torch.float32).view(1, 1, -1, 1)
    out = causal_attention(col(ka["q"]), col(ka["k"]), col(ka["v"]), attention_backend="eager", warning_prefix="t",
                           q_positions=torch.tensor([ka["q_positions"]]), k_positions=torch.tensor([ka["k_positions"]]),
                           q_sequence_ids=torch.tensor([ka["q_sequence_ids"]]), k_sequence_ids=torch.tensor([ka["k_sequence_ids"]]))
    assert torch.allclose(out.flatten(), torch.tensor(ka["expected"]), atol=ka["atol"])
    with pytest.raises(ValueError):
        causal_attention(col(ka["q"]), col(ka["k"]), col(ka["v"]), attention_backend="eager", warning_prefix="t",
                         q_sequence_ids=torch.tensor([ka["q_sequence_ids"]]))


def test_backend_names():
    assert set(ATTENTION_BACKEND_CHOICES) == {"eager", "sdpa_auto", "sdpa_flash", "flash_attn", "hip"}
    assert validate_attention_backend("hip") is AttentionBackend.HIP
    assert AttentionBackend.HIP == "hip" and f"{AttentionBackend.SDPA_AUTO}" == "sdpa_auto"
    with pytest.raises(ValueError, match="attention_backend must be one of"):
        validate_attention_backend("cudnn")


def test_zigzag_layout_and_schedule(known_answers):
    ka = known_answers["zigzag_positions"]
    pos = expected_zigzag_ring_positions(ka["local_seq_len"], rank=ka["rank"], world_size=ka["world_size"], device=torch.device("cpu"))
    assert pos.tolist() == ka["expected"]
    with pytest.raises(ValueError):
        expected_zigzag_ring_positions(3, rank=0, world_size=2, device=torch.device("cpu"))
    assert has_zigzag_ring_layout(pos.unsqueeze(0).expand(3, -1), rank=0, world_size=2)
    assert not has_zigzag_ring_layout(pos.unsqueeze(0), rank=1, world_size=2)
    assert not has_zigzag_ring_layout(pos, rank=0, world_size=2)
    for w in (2, 4):
        for rank in range(w):
            plan = zigzag_ring_schedule(rank, w)
            assert [src for src, _ in plan] == [(rank - s) % w for s in range(w)]
            assert [kind for _, kind in plan] == ["causal"] + ["front_kv" if s <= rank else "tail_q" for s in range(1, w)]
    with pytest.raises(ValueError):
        zigzag_ring_schedule(4, 4)


def test_varlen_metadata_known_answers(known_answers):
    ka = known_answers["varlen_metadata"]
    ids = torch.tensor(ka["sequence_ids"])
    meta = varlen_qkv_metadata(ids)
    assert meta.cu_seqlens.tolist() == ka["cu_seqlens"] and meta.cu_seqlens.dtype == torch.int32
    assert meta.max_seqlen == ka["max_seqlen"] and meta.token_mask.tolist() == ka["token_mask"]
    assert varlen_qkv_metadata(ids) is meta  # reused across layers
    e = ka["after_edit"]
    ids[e["row"], e["col"]] = e["value"]
    again = varlen_qkv_metadata(ids)
    assert again is not meta and again.cu_seqlens.tolist() == e["cu_seqlens"]
    empty = varlen_qkv_metadata(torch.full((2, 3), -1))
    assert empty.cu_seqlens.tolist() == [0] and empty.max_seqlen == 0


def _prefix_layout_by_hand(q_pos, k_pos, q_seq, k_seq, allow_empty):
    """Token-by-token walk of the rule stated in the reference (runtime/layers/flash_utils.py:627-690), for small cases."""
    q_idx, k_idx, q_len, k_len = [], [], [], []
    B, Sq = q_pos.shape
    Sk = k_pos.size(1)
    for b in range(B):
        toks = [i for i in range(Sq) if int(q_seq[b, i]) != -1]
        runs, cur = [], []
        for i in toks:
            if cur and (int(q_seq[b, i]) != int(q_seq[b, cur[-1]]) or int(q_pos[b, i]) != int(q_pos[b, cur[-1]]) + 1):
                runs.append(cur)
                cur = []
            cur.append(i)
        if cur:
            runs.append(cur)
        for run in runs:
            sid, end = int(q_seq[b, run[0]]), int(q_pos[b, run[-1]])
            keys = [j for j in range(Sk) if int(k_seq[b, j]) == sid and int(k_seq[b, j]) != -1 and int(k_pos[b, j]) <= end]
            if not keys:
                assert allow_empty
                continue
            q_idx += [b * Sq + i for i in run]
            k_idx += [b * Sk + j for j in keys]
            q_len.append(len(run))
            k_len.append(len(keys))
    return q_idx, k_idx, q_len, k_len


def test_varlen_prefix_metadata_known_answers(known_answers):
    for case in known_answers["varlen_prefix_pack"]["cases"]:
        t = lambda name: None if case[name] is None else torch.tensor(case[name])
        meta = varlen_prefix_metadata(q_positions=t("q_positions"), k_positions=t("k_positions"), q_sequence_ids=t("q_sequence_ids"),
                                      k_sequence_ids=t("k_sequence_ids"), allow_empty_kv=case["allow_empty_kv"])
        assert meta.cu_seqlens_q.tolist() == case["cu_seqlens_q"] and meta.cu_seqlens_q.dtype == torch.int32
        assert meta.cu_seqlens_k.tolist() == case["cu_seqlens_k"] and meta.cu_seqlens_k.dtype == torch.int32
        assert (meta.max_seqlen_q, meta.max_seqlen_k) == (case["max_seqlen_q"], case["max_seqlen_k"])
        assert meta.q_indices.tolist() == case["q_indices"] and meta.k_indices.tolist() == case["k_indices"]
    empty_case = known_answers["varlen_prefix_pack"]["cases"][1]
    with pytest.raises(ValueError, match="without any matching key/value prefix"):
        varlen_prefix_metadata(q_positions=torch.tensor(empty_case["q_positions"]), k_positions=torch.tensor(empty_case["k_positions"]))
    none = varlen_prefix_metadata(q_positions=torch.zeros(2, 3, dtype=torch.long), k_positions=torch.zeros(2, 3, dtype=torch.long),
                                  q_sequence_ids=torch.full((2, 3), -1), k_sequence_ids=torch.zeros(2, 3, dtype=torch.long))
    assert none.cu_seqlens_q.tolist() == [0] and none.max_seqlen_q == 0 and none.q_indices.numel() == 0


def test_varlen_prefix_metadata_against_token_walk():
    gen = torch.Generator().manual_seed(11)
    for trial in range(20):
        B, Sq, Sk = 2, 13, 17
        # shuffled chunks of a few documents with padding: positions and ids drawn so that runs break in every way
        q_seq = torch.randint(-1, 3, (B, Sq), generator=gen)
        k_seq = torch.randint(-1, 3, (B, Sk), generator=gen)
        q_pos = torch.cumsum(torch.randint(0, 3, (B, Sq), generator=gen), 1) % 7
        k_pos = torch.randint(0, 7, (B, Sk), generator=gen)
        want = _prefix_layout_by_hand(q_pos, k_pos, q_seq, k_seq, True)
        meta = varlen_prefix_metadata(q_positions=q_pos, k_positions=k_pos, q_sequence_ids=q_seq, k_sequence_ids=k_seq, allow_empty_kv=True)
        assert meta.q_indices.tolist() == want[0] and meta.k_indices.tolist() == want[1], trial
        assert (meta.cu_seqlens_q[1:] - meta.cu_seqlens_q[:-1]).tolist() == want[2]
        assert (meta.cu_seqlens_k[1:] - meta.cu_seqlens_k[:-1]).tolist() == want[3]
        assert meta.max_seqlen_q == max(want[2], default=0) and meta.max_seqlen_k == max(want[3], default=0)


def test_optimizer_plumbing_on_host():
    with pytest.raises(ValueError):
        FusedAdamW([torch.nn.Parameter(torch.zeros(4))], lr=-1.0)
    with pytest.raises(ValueError):
        FusedAdamW([torch.nn.Parameter(torch.zeros(4))], betas=(1.0, 0.9))
    opt = FusedAdamW([torch.nn.Parameter(torch.zeros(4))], lr=3e-4, betas=(0.9, 0.95), weight_decay=0.1)
    assert opt.param_groups[0]["lr"] == 3e-4 and opt.param_groups[0]["betas"] == (0.9, 0.95)
    with pytest.raises(ValueError, match="GPU"):
        opt.param_groups[0]["params"][0].grad = torch.zeros(4)
        opt.step()
    with pytest.raises(ValueError, match="at least one trainable"):
        MasterWeightsOptimizer([], optimizer_factory=lambda ps: torch.optim.SGD(ps, lr=1.0))
    # the reference's resync scenario with a stock inner optimizer, entirely on the host
    model_param = torch.nn.Parameter(torch.zeros(4, dtype=torch.bfloat16))
    mw = MasterWeightsOptimizer([model_param], optimizer_factory=lambda ps: torch.optim.SGD(ps, lr=1.0))
    with torch.no_grad():
        model_param.fill_(3.0)
    mw.sync_master_params_from_model()
    model_param.grad = torch.zeros_like(model_param)
    mw.step()
    torch.testing.assert_close(model_param, torch.full_like(model_param, 3.0))
    assert mw.model_param_for(mw.master_params[0]) is model_param
    sd = mw.state_dict()
    assert set(sd) == {"inner_optimizer", "master_params", "master_dtype"} and sd["master_dtype"] == "torch.float32"
    mw.zero_grad(set_to_none=True)
    assert model_param.grad is None
    mw.load_state_dict(sd)
    torch.testing.assert_close(model_param, torch.full_like(model_param, 3.0))


def test_adjacent_gradient_columns_are_recognised():
    """The one-product projections take their output gradients as one matrix when these already lie side by side."""
    from maltos_amd.llama import _adjacent_columns

    B, S, D = 2, 5, 4
    joint = torch.arange(B * S * 8 * D, dtype=torch.float32).view(B, S, 8, D)
    q, k, v = (joint[:, :, a:b].reshape(B, S, (b - a) * D) for a, b in ((0, 4), (4, 6), (6, 8)))
    assert q.untyped_storage().data_ptr() == joint.untyped_storage().data_ptr()   # views, as autograd hands them over
    both = _adjacent_columns([q, k, v])
    assert both is not None and both.shape == (B * S, 8 * D) and torch.equal(both, joint.view(B * S, 8 * D))
    assert both.untyped_storage().data_ptr() == joint.untyped_storage().data_ptr()
    assert _adjacent_columns([k, v]) is None                    # rows wider than the two together
    assert _adjacent_columns([q, v, k]) is None                 # another order than the columns
    assert _adjacent_columns([q, k.clone(), v]) is None         # another buffer
    assert _adjacent_columns([q.contiguous(), k.contiguous(), v.contiguous()]) is None
    tail = torch.zeros(B, S, 8, D)[:, :, 4:]
    assert _adjacent_columns([tail[:, :, :2].reshape(B, S, 2 * D), tail[:, :, 2:].reshape(B, S, 2 * D)]) is None
    whole = torch.zeros(3, 6)
    assert _adjacent_columns([whole[:, :2], whole[:, 2:]]).data_ptr() == whole.data_ptr()


def test_shipped_gemm_selection_file_is_well_formed():
    from maltos_amd.gemm_tuning import TUNED_FILE, use_tuned_gemms

    rows = [line.split(",") for line in TUNED_FILE.read_text().splitlines()]
    validators = {r[1] for r in rows if r[0] == "Validator"}
    assert {"PT_VERSION", "HIP_VERSION", "HIPBLASLT_VERSION", "ROCBLAS_VERSION", "GCN_ARCH_NAME"} <= validators
    assert any(r[0] == "Validator" and r[1] == "GCN_ARCH_NAME" and r[2].startswith("gfx950") for r in rows)
    shapes = [r for r in rows if r[0].startswith("Gemm")]
    assert len(shapes) >= 15 and all(len(r) == 4 and float(r[3]) > 0 for r in shapes)
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="needs a GPU"):
            use_tuned_gemms()
