"""The entry point that allocates nothing: mlts_attn_bwd_noalloc keeps its workspace (delta, base-2 LSE, tile
statistics) in a buffer inside the library image instead of taking one from the caller.  Called through the C ABI
and compared bit for bit with mlts_attn_bwd given a caller workspace of exactly mlts_attn_bwd_workspace_bytes (the
same kernels on the same inputs), on two calls in a row, the second on a smaller input, so that whatever the first
call left in the shared buffer is there when the second runs."""
import ctypes as C

import pytest
import torch

from maltos_amd import _lib, ops
from maltos_amd._lib import strides3

pytestmark = pytest.mark.gpu


def _inputs(dev, B, Hq, Hkv, S, D, seed, mode):
    gen = torch.Generator().manual_seed(seed)
    mk = lambda h: torch.randn(B, S, h, D, generator=gen).bfloat16().transpose(1, 2).to(dev)
    q, k, v, do = mk(Hq), mk(Hkv), mk(Hkv), mk(Hq)
    kw = {}
    if mode == ops.MASK_DOC:
        cut = S // 3
        pos = torch.cat([torch.arange(cut), torch.arange(S - cut)]).expand(B, S).contiguous().to(dev)
        seq = torch.cat([torch.zeros(cut, dtype=torch.long), torch.ones(S - cut, dtype=torch.long)]).expand(B, S).contiguous().to(dev)
        kw = dict(q_pos=pos, k_pos=pos, q_seq=seq, k_seq=seq)
    o, lse = ops.attention_forward(q, k, v, mask_mode=mode, **kw)
    return q, k, v, do, o, lse, kw


def _backward_both(dev, q, k, v, do, o, lse, mode, kw):
    L = _lib.lib()
    ids = {n: (t.to(torch.int32).contiguous() if t is not None else None) for n, t in
           dict(q_pos=kw.get("q_pos"), k_pos=kw.get("k_pos"), q_seq=kw.get("q_seq"), k_seq=kw.get("k_seq")).items()}
    shape = ops._attn_shape(q, k, v, o, mode, q.size(-1) ** -0.5, ids["q_pos"], ids["k_pos"], ids["q_seq"], ids["k_seq"])
    assert not L.mlts_attn_supports(C.byref(shape))
    p = lambda t: C.c_void_p(t.data_ptr())
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = []
    for noalloc in (False, True):
        dq, dk, dv = (torch.full_like(t, float("nan")) for t in (q, k, v))
        args = [C.byref(shape), p(do), strides3(do.stride()[:3]), p(q), p(k), p(v), p(o), p(lse), p(dq), strides3(dq.stride()[:3]),
                p(dk), strides3(dk.stride()[:3]), p(dv), strides3(dv.stride()[:3]), 0]
        if noalloc:
            _lib.check(L.mlts_attn_bwd_noalloc(*args, stream))
        else:
            ws_bytes = L.mlts_attn_bwd_workspace_bytes(C.byref(shape), 0)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
            _lib.check(L.mlts_attn_bwd(*args, p(ws), ws_bytes, stream))
        torch.cuda.synchronize()
        outs.append((dq, dk, dv))
    return outs


@pytest.mark.parametrize("mode", [ops.MASK_CAUSAL, ops.MASK_DOC], ids=["causal", "documents"])
def test_noalloc_backward_equals_workspace_backward_twice(dev, mode):
    # first a larger call, then a smaller one: the second finds the first one's data in the shared buffer
    for B, Hq, Hkv, S, D, seed in ((2, 4, 2, 777, 128, 11), (1, 2, 2, 200, 128, 12), (2, 4, 4, 300, 64, 13)):
        q, k, v, do, o, lse, kw = _inputs(dev, B, Hq, Hkv, S, D, seed, mode)
        (dq0, dk0, dv0), (dq1, dk1, dv1) = _backward_both(dev, q, k, v, do, o, lse, mode, kw)
        for name, a, b in (("dQ", dq0, dq1), ("dK", dk0, dk1), ("dV", dv0, dv1)):
            assert torch.isfinite(b.float()).all(), f"{name} S={S}: non-finite"
            assert torch.equal(a, b), f"{name} S={S}: no-alloc result differs from the workspace result"


def test_noalloc_calls_on_two_streams_take_turns(dev):
    """Two calls enqueued back to back on different streams share the one buffer: the second waits for the first (an
    event behind the first call's kernels), so both give the results of the workspace form."""
    L = _lib.lib()
    mode = ops.MASK_CAUSAL
    cases = [_inputs(dev, 2, 8, 8, 1500, 128, 21, mode), _inputs(dev, 1, 4, 4, 900, 128, 22, mode)]
    want = []
    for q, k, v, do, o, lse, kw in cases:
        want.append(ops.attention_backward(do, q, k, v, o, lse, mask_mode=mode))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    got = []
    p = lambda t: C.c_void_p(t.data_ptr())
    for rep in range(3):
        got.clear()
        for (q, k, v, do, o, lse, kw), st in zip(cases, streams):
            shape = ops._attn_shape(q, k, v, o, mode, q.size(-1) ** -0.5, None, None, None, None)
            dq, dk, dv = (torch.full_like(t, float("nan")) for t in (q, k, v))
            st.wait_stream(torch.cuda.current_stream())
            _lib.check(L.mlts_attn_bwd_noalloc(C.byref(shape), p(do), strides3(do.stride()[:3]), p(q), p(k), p(v), p(o), p(lse),
                                               p(dq), strides3(dq.stride()[:3]), p(dk), strides3(dk.stride()[:3]), p(dv),
                                               strides3(dv.stride()[:3]), 0, C.c_void_p(st.cuda_stream)))
            got.append((dq, dk, dv))
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            for a, b in zip(g, w):
                assert torch.equal(a, b), f"repetition {rep}: a call on its own stream differs from the workspace form"


def test_noalloc_rejects_shapes_beyond_its_buffer(dev):
    """B * Hq * Sq rows whose statistics do not fit the built-in buffer are refused before any launch."""
    L = _lib.lib()
    B, H, S, D = 1, 64, 32768, 128   # 2 M query rows: 16 MiB of delta + LSE
    t = torch.empty(1, device=dev, dtype=torch.bfloat16)   # never dereferenced: the size check comes first
    shape = _lib.AttnShape()
    shape.B, shape.Hq, shape.Hkv, shape.Sq, shape.Sk, shape.D = B, H, H, S, S, D
    shape.dtype, shape.mask_mode, shape.scale = _lib.MLTS_BF16, ops.MASK_CAUSAL, D ** -0.5
    for name in ("q_stride", "k_stride", "v_stride", "o_stride"):
        setattr(shape, name, strides3((H * S * D, S * D, D)))
    st = strides3((H * S * D, S * D, D))
    p = C.c_void_p(t.data_ptr())
    rc = L.mlts_attn_bwd_noalloc(C.byref(shape), p, st, p, p, p, p, p, p, st, p, st, p, st, 0, None)
    assert rc == 1
    assert b"built-in scratch" in L.mlts_last_error()
