"""torch.library custom ops over the C ABI of libmaltos_hip.so.

Layering: `torch.ops.maltos.*` (registered here, CUDA/HIP dispatch key only, with fake kernels for
shape inference and autograd formulas) -> ctypes -> `mlts_*` entry points -> HIP kernels on the
current torch stream.  There is deliberately no CPU implementation: calling an op with host
tensors, or without the built library, raises.
"""
from __future__ import annotations

import ctypes as C
import math
import threading

import torch

from . import _lib
from ._lib import MASK_CAUSAL, MASK_DOC, MASK_NONE, MLTS_BF16, MLTS_F32, AttnShape, strides3

# mlts_attn_bwd's accumulate_f32 modes (include/maltos_hip.h)
BWD_OVERWRITE, BWD_ACCUMULATE, BWD_DQ_ACCUMULATE, BWD_DQ_STORE = 0, 1, 2, 3

__all__ = [
    "MASK_NONE", "MASK_CAUSAL", "MASK_DOC",
    "attention", "attention_forward", "attention_backward", "attention_backward_accumulate",
    "attention_backward_ring_block", "attention_merge_",
    "rms_norm", "rope", "rope_pair", "rope_pair_", "swiglu", "cross_entropy",
    "adamw_step_", "sq_norm", "scale_", "grad_to_f32_",
]


# --------------------------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------------------------
def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return MLTS_BF16
    if t.dtype == torch.float32:
        return MLTS_F32
    raise ValueError(f"maltos_amd kernels take float32 or bfloat16 tensors, got {t.dtype}")


def _require_gpu(*tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("maltos_amd ops run on the GPU only (there is no CPU fallback); got a host tensor")


def _p(t: torch.Tensor | None):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def _stream() -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _workspace(nbytes: int, device: torch.device) -> torch.Tensor | None:
    if nbytes <= 0:
        return None
    return torch.empty(int(nbytes), dtype=torch.uint8, device=device)


def _check_attn_inputs(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> None:
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("attention expects q, k, v of shape [batch, heads, seq, head_dim]")
    if k.shape != v.shape:
        raise ValueError(f"k and v must have identical shapes, got {tuple(k.shape)} vs {tuple(v.shape)}")
    if q.size(0) != k.size(0) or q.size(3) != k.size(3):
        raise ValueError(f"q and k disagree on batch or head_dim: {tuple(q.shape)} vs {tuple(k.shape)}")
    if q.size(1) % k.size(1) != 0:
        raise ValueError(f"query heads ({q.size(1)}) must be a multiple of kv heads ({k.size(1)})")
    if not (q.dtype == k.dtype == v.dtype):
        raise ValueError("q, k, v must share a dtype")


def _dense_last(t: torch.Tensor) -> torch.Tensor:
    """Kernels take arbitrary (batch, head, seq) strides but need a contiguous head_dim."""
    return t if t.stride(-1) == 1 or t.size(-1) == 1 else t.contiguous()


def derived_from(t: torch.Tensor, attr: str, build):
    """`build(t)`, kept on the tensor object `t` until `t` is modified in place (its autograd version counter moves).
    Every layer of a model is handed the same id tensors, so what is derived from them (their int32 form, run ids, a
    zero id tensor) is formed once per batch instead of once per layer, and, being the same tensor objects in every
    call, lets the calls share one document-mask plan.  Not kept for inference tensors (no version counter) nor under
    HIP graph capture (a tensor allocated while capturing belongs to the graph's pool)."""
    if t.is_inference() or (t.is_cuda and torch.cuda.is_current_stream_capturing()):
        return build(t)
    hit = t.__dict__.get(attr)
    if hit is not None and hit[0] == t._version:
        return hit[1]
    value = build(t)
    t.__dict__[attr] = (t._version, value)
    return value


def _ids32(t: torch.Tensor | None, batch: int, seq: int, what: str) -> torch.Tensor | None:
    if t is None:
        return None
    if t.shape != (batch, seq):
        raise ValueError(f"{what} must have shape ({batch}, {seq}), got {tuple(t.shape)}")
    if t.dtype == torch.int32 and t.is_contiguous():
        return t
    return derived_from(t, "_maltos_hip_int32", lambda x: x.to(dtype=torch.int32).contiguous())


def _attn_shape(q, k, v, o, mask_mode, scale, q_pos, k_pos, q_seq, k_seq) -> AttnShape:
    s = AttnShape()
    s.B, s.Hq, s.Sq, s.D = q.size(0), q.size(1), q.size(2), q.size(3)
    s.Hkv, s.Sk = k.size(1), k.size(2)
    s.dtype = _dtype_code(q)
    s.mask_mode = int(mask_mode)
    s.scale = float(scale)
    s.q_stride = strides3(q.stride()[:3])
    s.k_stride = strides3(k.stride()[:3])
    s.v_stride = strides3(v.stride()[:3])
    s.o_stride = strides3(o.stride()[:3])
    if mask_mode == MASK_DOC:
        if q_pos is None or k_pos is None or q_seq is None or k_seq is None:
            raise ValueError("document-masked attention needs q/k positions and q/k sequence ids")
        s.q_pos, s.k_pos, s.q_seq, s.k_seq = q_pos.data_ptr(), k_pos.data_ptr(), q_seq.data_ptr(), k_seq.data_ptr()
    return s


# Document-mask plans (mlts_attn_doc_plan): every layer of a model, forward and backward, attends under the same ids, so
# the plan of a call is kept and handed to later calls with the same ids.  "The same" is judged without reading
# device memory: same address, dtype, shape, strides and autograd version of the four id tensors as given by the caller,
# which are kept alive with the plan so that their addresses cannot be handed to other tensors meanwhile (an in-place
# change of the ids through torch bumps the version; writes behind torch's back are not seen: clear_doc_plan_cache()).
_DOC_PLAN_CACHE: list[tuple[tuple, tuple, torch.Tensor]] = []
_DOC_PLAN_CACHE_ENTRIES = 8
_DOC_PLAN_CACHE_BYTES = 1 << 30  # most bytes of plans kept (a plan is B * Sq * Sk / 4 bytes); larger plans are not kept
_DOC_PLAN_LOCK = threading.Lock()  # forward runs on the caller's thread, backward on autograd's device thread


def set_doc_plan_cache_entries(n: int) -> int:
    """Number of document-mask plans kept (0: every call builds its own in its workspace).  Returns the previous value."""
    global _DOC_PLAN_CACHE_ENTRIES
    if n < 0:
        raise ValueError("the number of cached plans is >= 0")
    with _DOC_PLAN_LOCK:
        previous, _DOC_PLAN_CACHE_ENTRIES = _DOC_PLAN_CACHE_ENTRIES, int(n)
        del _DOC_PLAN_CACHE[_DOC_PLAN_CACHE_ENTRIES:]
    return previous


def clear_doc_plan_cache() -> None:
    with _DOC_PLAN_LOCK:
        _DOC_PLAN_CACHE.clear()


def _attach_doc_plan(shape: AttnShape, given: tuple, used: tuple, device: torch.device) -> torch.Tensor | None:
    """Sets shape.doc_plan to a kept plan for these ids, building it first if there is none.  `given`: the caller's id
    tensors, `used`: their int32 forms that shape points at.  Returns the plan (to be kept alive over the launch)."""
    if shape.mask_mode != MASK_DOC or _DOC_PLAN_CACHE_ENTRIES == 0 or torch.cuda.is_current_stream_capturing():
        return None  # (a captured graph must rebuild the plan on every replay: its id buffers are refilled in place)
    L = _lib.lib()
    nbytes = L.mlts_attn_doc_plan_bytes(C.byref(shape))
    if nbytes <= 0 or nbytes > _DOC_PLAN_CACHE_BYTES:
        return None
    if any(t.is_inference() for t in given):
        return None  # (inference tensors carry no version counter: nothing tells a rewritten id tensor from the old one)
    key = (shape.B, shape.Hq, shape.Hkv, shape.Sq, shape.Sk, shape.D, shape.dtype, device, torch.cuda.current_stream().cuda_stream,
           tuple((t.data_ptr(), t._version, t.dtype, tuple(t.shape), tuple(t.stride())) for t in given))
    with _DOC_PLAN_LOCK:
        for i, (k_, _, plan) in enumerate(_DOC_PLAN_CACHE):
            if k_ == key:
                if i:
                    _DOC_PLAN_CACHE.insert(0, _DOC_PLAN_CACHE.pop(i))
                shape.doc_plan = plan.data_ptr()
                return plan
        plan = torch.empty(int(nbytes), dtype=torch.uint8, device=device)
        _lib.check(L.mlts_attn_doc_plan(C.byref(shape), _p(plan), nbytes, _stream()))
        _DOC_PLAN_CACHE.insert(0, (key, tuple(given) + tuple(used), plan))
        del _DOC_PLAN_CACHE[_DOC_PLAN_CACHE_ENTRIES:]
        while sum(e[2].numel() for e in _DOC_PLAN_CACHE) > _DOC_PLAN_CACHE_BYTES:
            _DOC_PLAN_CACHE.pop()
        shape.doc_plan = plan.data_ptr()
        return plan


def _bshd_empty(B: int, H: int, S: int, D: int, like: torch.Tensor, dtype=None) -> torch.Tensor:
    """[B, H, S, D] view over [B, S, H, D] storage: the layout LlamaAttention transposes back to."""
    return torch.empty((B, S, H, D), dtype=dtype or like.dtype, device=like.device).transpose(1, 2)


# --------------------------------------------------------------------------------------------
# raw launches (no autograd)
# --------------------------------------------------------------------------------------------
def attention_forward(q, k, v, *, mask_mode: int, scale: float | None = None, q_pos=None, k_pos=None, q_seq=None,
                      k_seq=None) -> tuple[torch.Tensor, torch.Tensor]:
    """O [B,Hq,Sq,D] (BSHD storage) and LSE [B,Hq,Sq] fp32."""
    _check_attn_inputs(q, k, v)
    _require_gpu(q, k, v, q_pos, k_pos, q_seq, k_seq)
    q, k, v = _dense_last(q), _dense_last(k), _dense_last(v)
    B, Hq, Sq, D = q.shape
    scale = D ** -0.5 if scale is None else scale
    o = _bshd_empty(B, Hq, Sq, D, q)
    lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=q.device)
    if B == 0 or Sq == 0:
        return o, lse
    given = (q_pos, k_pos, q_seq, k_seq)
    q_pos, q_seq = _ids32(q_pos, B, Sq, "q_positions"), _ids32(q_seq, B, Sq, "q_sequence_ids")
    k_pos, k_seq = _ids32(k_pos, B, k.size(2), "k_positions"), _ids32(k_seq, B, k.size(2), "k_sequence_ids")
    shape = _attn_shape(q, k, v, o, mask_mode, scale, q_pos, k_pos, q_seq, k_seq)
    L = _lib.lib()
    why = L.mlts_attn_supports(C.byref(shape))
    if why:
        raise ValueError(f"attention_forward: {why.decode()}")
    plan = _attach_doc_plan(shape, given, (q_pos, k_pos, q_seq, k_seq), q.device)  # noqa: F841 (alive over the launch)
    ws_bytes = L.mlts_attn_fwd_workspace_bytes(C.byref(shape))
    ws = _workspace(ws_bytes, q.device)
    _lib.check(L.mlts_attn_fwd(C.byref(shape), _p(q), _p(k), _p(v), _p(o), _p(lse), _p(ws), ws_bytes, _stream()))
    return o, lse


def _attention_backward_impl(dout, q, k, v, o, lse, dq, dk, dv, accumulate, mask_mode, scale, q_pos, k_pos, q_seq,
                             k_seq) -> None:
    _check_attn_inputs(q, k, v)
    _require_gpu(dout, q, k, v, o, lse, dq, dk, dv, q_pos, k_pos, q_seq, k_seq)
    B, Hq, Sq, D = q.shape
    Sk = k.size(2)
    if B == 0 or Sq == 0 or Sk == 0:
        if accumulate in (BWD_OVERWRITE, BWD_DQ_STORE):
            dq.zero_()
        if accumulate != BWD_ACCUMULATE:
            dk.zero_(), dv.zero_()
        return
    if dout.shape != q.shape or o.shape != q.shape:
        raise ValueError("dout and out must have the shape of q")
    if lse.shape != (B, Hq, Sq) or lse.dtype != torch.float32:
        raise ValueError(f"softmax_lse must be float32 of shape {(B, Hq, Sq)}, got {lse.dtype} {tuple(lse.shape)}")
    lse = lse.contiguous()
    scale = D ** -0.5 if scale is None else scale
    given = (q_pos, k_pos, q_seq, k_seq)
    q_pos, q_seq = _ids32(q_pos, B, Sq, "q_positions"), _ids32(q_seq, B, Sq, "q_sequence_ids")
    k_pos, k_seq = _ids32(k_pos, B, Sk, "k_positions"), _ids32(k_seq, B, Sk, "k_sequence_ids")
    shape = _attn_shape(q, k, v, o, mask_mode, scale, q_pos, k_pos, q_seq, k_seq)
    L = _lib.lib()
    why = L.mlts_attn_supports(C.byref(shape))
    if why:
        raise ValueError(f"attention_backward: {why.decode()}")
    plan = _attach_doc_plan(shape, given, (q_pos, k_pos, q_seq, k_seq), q.device)  # noqa: F841 (alive over the launch)
    ws_bytes = L.mlts_attn_bwd_workspace_bytes(C.byref(shape), int(accumulate))
    ws = _workspace(ws_bytes, q.device)
    _lib.check(
        L.mlts_attn_bwd(C.byref(shape), _p(dout), strides3(dout.stride()[:3]), _p(q), _p(k), _p(v), _p(o), _p(lse),
                        _p(dq), strides3(dq.stride()[:3]), _p(dk), strides3(dk.stride()[:3]), _p(dv),
                        strides3(dv.stride()[:3]), int(accumulate), _p(ws), ws_bytes, _stream())
    )


def attention_backward(dout, q, k, v, o, lse, *, mask_mode: int, scale: float | None = None, q_pos=None, k_pos=None,
                       q_seq=None, k_seq=None):
    """(dq, dk, dv) in the input dtype, as [B, H, S, D] views of [B, S, H, D] storage.  For self-attention (queries and
    keys of one length) the three are the head ranges [0, Hq), [Hq, Hq + Hkv), [Hq + Hkv, Hq + 2 Hkv) of ONE
    [B, S, Hq + 2 Hkv, D] buffer: next to each other exactly as the input gradient of projections that run as one
    product wants them, so that nobody has to copy them together."""
    q, k, v, o, dout = map(_dense_last, (q, k, v, o, dout))
    B, Hq, Sq, D = q.shape
    Hkv = k.size(1)
    if k.size(2) == Sq and k.dtype == q.dtype and v.dtype == q.dtype:
        joint = _bshd_empty(B, Hq + 2 * Hkv, Sq, D, q)
        dq, dk, dv = joint[:, :Hq], joint[:, Hq:Hq + Hkv], joint[:, Hq + Hkv:]
    else:
        dq = _bshd_empty(B, Hq, Sq, D, q)
        dk = _bshd_empty(k.size(0), Hkv, k.size(2), k.size(3), k)
        dv = _bshd_empty(v.size(0), v.size(1), v.size(2), v.size(3), v)
    _attention_backward_impl(dout, q, k, v, o, lse, dq, dk, dv, BWD_OVERWRITE, mask_mode, scale, q_pos, k_pos, q_seq, k_seq)
    return dq, dk, dv


def attention_backward_accumulate(dout, q, k, v, o, lse, dq, dk, dv, *, mask_mode: int, scale: float | None = None,
                                  q_pos=None, k_pos=None, q_seq=None, k_seq=None) -> None:
    """dq += ..., dk += ..., dv += ... into fp32 buffers (ring schedule)."""
    for name, t, ref in (("dq", dq, q), ("dk", dk, k), ("dv", dv, v)):
        if t.dtype != torch.float32 or t.shape != ref.shape or t.stride(-1) != 1:
            raise ValueError(f"{name} must be float32 with the shape of its input and a contiguous head_dim")
    q, k, v, o, dout = map(_dense_last, (q, k, v, o, dout))
    _attention_backward_impl(dout, q, k, v, o, lse, dq, dk, dv, BWD_ACCUMULATE, mask_mode, scale, q_pos, k_pos, q_seq, k_seq)


def attention_backward_ring_block(dout, q, k, v, o, lse, dq, dk, dv, *, first: bool, mask_mode: int, scale: float | None = None,
                                  q_pos=None, k_pos=None, q_seq=None, k_seq=None) -> None:
    """One block of a ring schedule on the rank that owns the queries: dq (fp32) collects every block (`first`: this
    block overwrites it, so nobody has to clear it; later blocks add), while dk and dv of the block's keys (input
    dtype) are written once, since a K/V chunk meets the local queries in exactly one block."""
    if dq.dtype != torch.float32 or dq.shape != q.shape or dq.stride(-1) != 1:
        raise ValueError("dq must be float32 with the shape of q and a contiguous head_dim")
    for name, t, ref in (("dk", dk, k), ("dv", dv, v)):
        if t.dtype != ref.dtype or t.shape != ref.shape or t.stride(-1) != 1:
            raise ValueError(f"{name} must have the dtype and shape of its input and a contiguous head_dim")
    q, k, v, o, dout = map(_dense_last, (q, k, v, o, dout))
    _attention_backward_impl(dout, q, k, v, o, lse, dq, dk, dv, BWD_DQ_STORE if first else BWD_DQ_ACCUMULATE, mask_mode, scale,
                             q_pos, k_pos, q_seq, k_seq)


def attention_merge_(out_acc, lse_acc, o_blk, lse_blk, q_off: int = 0) -> None:
    """In-place log-sum-exp merge of a block into rows [q_off, q_off + q_len) of the running state."""
    _require_gpu(out_acc, lse_acc, o_blk, lse_blk)
    if out_acc.dtype != torch.float32 or lse_acc.dtype != torch.float32 or not out_acc.is_contiguous() or not lse_acc.is_contiguous():
        raise ValueError("running_out / running_lse must be contiguous float32")
    B, H, S, D = out_acc.shape
    q_len = o_blk.size(2)
    if o_blk.shape != (B, H, q_len, D) or lse_blk.shape != (B, H, q_len) or lse_acc.shape != (B, H, S):
        raise ValueError("block shapes do not match the running state")
    o_blk = _dense_last(o_blk)
    lse_blk = lse_blk.to(torch.float32).contiguous()
    _lib.check(
        _lib.lib().mlts_attn_merge(_p(out_acc), _p(lse_acc), _p(o_blk), strides3(o_blk.stride()[:3]), _dtype_code(o_blk),
                                   _p(lse_blk), B, H, S, D, int(q_off), q_len, _stream())
    )


def _rmsnorm_fwd(x, w, eps):
    _require_gpu(x, w)
    hidden = x.size(-1)
    if w.shape != (hidden,) or w.dtype != x.dtype:
        raise ValueError("RMSNorm weight must be [hidden] with the dtype of x")
    x2 = x.contiguous().view(-1, hidden)
    y = torch.empty_like(x2)
    rstd = torch.empty(x2.size(0), dtype=torch.float32, device=x.device)
    w = w.contiguous()   # kept in a local until after the launch
    _lib.check(_lib.lib().mlts_rmsnorm_fwd(_p(x2), _p(w), _p(y), _p(rstd), x2.size(0), hidden, float(eps),
                                           _dtype_code(x), _stream()))
    return y.view(x.shape), rstd


def _rmsnorm_bwd(dy, x, w, rstd):
    _require_gpu(dy, x, w, rstd)
    hidden = x.size(-1)
    x2 = x.contiguous().view(-1, hidden)
    dy2 = dy.contiguous().view(-1, hidden)
    dx = torch.empty_like(x2)
    dw = torch.empty_like(w)
    if x2.size(0) == 0:
        return dx.view(x.shape), dw.zero_()
    L = _lib.lib()
    ws_bytes = L.mlts_rmsnorm_bwd_workspace_bytes(x2.size(0), hidden)
    ws = _workspace(ws_bytes, x.device)
    w = w.contiguous()
    _lib.check(L.mlts_rmsnorm_bwd(_p(dy2), _p(x2), _p(w), _p(rstd), _p(dx), _p(dw), _p(ws), ws_bytes,
                                  x2.size(0), hidden, _dtype_code(x), _stream()))
    return dx.view(x.shape), dw


def _add_rmsnorm_fwd(x, res, w, eps):
    _require_gpu(x, res, w)
    hidden = x.size(-1)
    if w.shape != (hidden,) or w.dtype != x.dtype:
        raise ValueError("RMSNorm weight must be [hidden] with the dtype of x")
    if res.shape != x.shape or res.dtype != x.dtype:
        raise ValueError("the residual must have the shape and dtype of x")
    x2 = x.contiguous().view(-1, hidden)
    r2 = res.contiguous().view(-1, hidden)
    h = torch.empty_like(x2)
    y = torch.empty_like(x2)
    rstd = torch.empty(x2.size(0), dtype=torch.float32, device=x.device)
    w = w.contiguous()
    _lib.check(_lib.lib().mlts_add_rmsnorm_fwd(_p(x2), _p(r2), _p(h), _p(w), _p(y), _p(rstd), x2.size(0), hidden,
                                               float(eps), _dtype_code(x), _stream()))
    return h.view(x.shape), y.view(x.shape), rstd


def _add_rmsnorm_bwd(dy, dres, h, w, rstd):
    _require_gpu(dy, dres, h, w, rstd)
    hidden = h.size(-1)
    h2 = h.contiguous().view(-1, hidden)
    dy2 = dy.contiguous().view(-1, hidden)
    dr2 = dres.contiguous().view(-1, hidden)
    dx = torch.empty_like(h2)
    dw = torch.empty_like(w)
    if h2.size(0) == 0:
        return dx.view(h.shape), dw.zero_()
    L = _lib.lib()
    ws_bytes = L.mlts_rmsnorm_bwd_workspace_bytes(h2.size(0), hidden)
    ws = _workspace(ws_bytes, h.device)
    w = w.contiguous()
    _lib.check(L.mlts_add_rmsnorm_bwd(_p(dy2), _p(h2), _p(w), _p(rstd), _p(dr2), _p(dx), _p(dw), _p(ws), ws_bytes,
                                      h2.size(0), hidden, _dtype_code(h), _stream()))
    return dx.view(h.shape), dw


def _rope(x, cos, sin, positions, position_offset, inverse):
    _require_gpu(x, cos, sin, positions)
    if x.dim() != 4:
        raise ValueError("rope expects [batch, heads, seq, head_dim]")
    B, H, S, D = x.shape
    if cos.shape != sin.shape or cos.dim() != 2 or cos.size(1) * 2 != D:
        raise ValueError(f"cos/sin tables must be [max_pos, {D // 2}], got {tuple(cos.shape)}")
    if cos.dtype != x.dtype or sin.dtype != x.dtype:
        raise ValueError("cos/sin tables must have the activation dtype (the reference casts them first)")
    x = _dense_last(x)
    y = torch.empty_like(x)  # keeps the (possibly transposed) layout of x
    pos32 = None
    if positions is not None:
        pos32 = _ids32(positions, B, S, "position_ids")
    cos, sin = cos.contiguous(), sin.contiguous()
    _lib.check(_lib.lib().mlts_rope(_p(x), strides3(x.stride()[:3]), _p(y), strides3(y.stride()[:3]), _p(cos),
                                    _p(sin), cos.size(0), _p(pos32), int(position_offset), B, H, S, D,
                                    _dtype_code(x), int(bool(inverse)), _stream()))
    return y


def _rope_pair(xa, xb, cos, sin, positions, position_offset, inverse, in_place: bool = False):
    """Both rotations of an attention layer (query and key projections) in one launch."""
    _require_gpu(xa, xb, cos, sin, positions)
    if xa.dim() != 4 or xb.dim() != 4 or xa.size(0) != xb.size(0) or xa.shape[2:] != xb.shape[2:] or xa.dtype != xb.dtype:
        raise ValueError("rope_pair expects two [batch, heads, seq, head_dim] tensors that differ only in heads")
    B, Ha, S, D = xa.shape
    if cos.shape != sin.shape or cos.dim() != 2 or cos.size(1) * 2 != D:
        raise ValueError(f"cos/sin tables must be [max_pos, {D // 2}], got {tuple(cos.shape)}")
    if cos.dtype != xa.dtype or sin.dtype != xa.dtype:
        raise ValueError("cos/sin tables must have the activation dtype (the reference casts them first)")
    if in_place:
        if xa.stride(-1) != 1 or xb.stride(-1) != 1:
            raise ValueError("rope_pair_: the head_dim of both tensors must be contiguous")
        ya, yb = xa, xb
    else:
        xa, xb = _dense_last(xa), _dense_last(xb)
        ya, yb = torch.empty_like(xa), torch.empty_like(xb)
    pos32 = None if positions is None else _ids32(positions, B, S, "position_ids")
    cos, sin = cos.contiguous(), sin.contiguous()
    _lib.check(_lib.lib().mlts_rope_pair(_p(xa), strides3(xa.stride()[:3]), _p(ya), strides3(ya.stride()[:3]), Ha,
                                         _p(xb), strides3(xb.stride()[:3]), _p(yb), strides3(yb.stride()[:3]), xb.size(1),
                                         _p(cos), _p(sin), cos.size(0), _p(pos32), int(position_offset), B, S, D,
                                         _dtype_code(xa), int(bool(inverse)), _stream()))
    return ya, yb


def _swiglu_fwd(gate, up):
    _require_gpu(gate, up)
    if gate.shape != up.shape or gate.dtype != up.dtype:
        raise ValueError("gate and up must match in shape and dtype")
    g, u = gate.contiguous(), up.contiguous()
    h = torch.empty_like(g)
    _lib.check(_lib.lib().mlts_swiglu_fwd(_p(g), _p(u), _p(h), g.numel(), _dtype_code(g), _stream()))
    return h


def _swiglu_bwd(dh, gate, up):
    _require_gpu(dh, gate, up)
    d, g, u = dh.contiguous(), gate.contiguous(), up.contiguous()
    dg, du = torch.empty_like(g), torch.empty_like(u)
    _lib.check(_lib.lib().mlts_swiglu_bwd(_p(d), _p(g), _p(u), _p(dg), _p(du), g.numel(), _dtype_code(g), _stream()))
    return dg, du


def swiglu_rows(gu: torch.Tensor, gate_col: int, up_col: int, cols: int) -> torch.Tensor:
    """round(silu(gate)) * up where gate = gu[..., gate_col : gate_col + cols] and up = gu[..., up_col : up_col + cols] are
    column blocks of one contiguous [..., width] projection output (no autograd: used inside the fused MLP function)."""
    _require_gpu(gu)
    if not gu.is_contiguous():
        raise ValueError("swiglu_rows expects a contiguous projection output")
    width = gu.size(-1)
    rows = gu.numel() // width
    h = torch.empty((*gu.shape[:-1], cols), dtype=gu.dtype, device=gu.device)
    es = gu.element_size()
    _lib.check(_lib.lib().mlts_swiglu_fwd_rows(C.c_void_p(gu.data_ptr() + gate_col * es), C.c_void_p(gu.data_ptr() + up_col * es), width,
                                               _p(h), cols, rows, cols, _dtype_code(gu), _stream()))
    return h


def swiglu_rows_backward(dh: torch.Tensor, gu: torch.Tensor, gate_col: int, up_col: int, cols: int) -> torch.Tensor:
    """d gate and d up of swiglu_rows, written into the same column blocks of a buffer shaped like `gu`; its other
    columns, if there are any, are zero."""
    _require_gpu(dh, gu)
    dh = dh.contiguous()
    width = gu.size(-1)
    rows = gu.numel() // width
    dgu = torch.empty_like(gu) if width == 2 * cols else torch.zeros_like(gu)
    es = gu.element_size()
    _lib.check(_lib.lib().mlts_swiglu_bwd_rows(_p(dh), cols, C.c_void_p(gu.data_ptr() + gate_col * es),
                                               C.c_void_p(gu.data_ptr() + up_col * es), width,
                                               C.c_void_p(dgu.data_ptr() + gate_col * es), C.c_void_p(dgu.data_ptr() + up_col * es), width,
                                               rows, cols, _dtype_code(gu), _stream()))
    return dgu


def _ce_fwd_bwd(logits, labels, ignore_index, overwrite: bool = False):
    """overwrite: the gradient replaces the logits in their own buffer (they must be contiguous)."""
    _require_gpu(logits, labels)
    vocab = logits.size(-1)
    lg = logits.contiguous().view(-1, vocab)
    lb = labels.contiguous().view(-1).to(torch.int64)
    if lb.numel() != lg.size(0):
        raise ValueError(f"labels ({lb.numel()}) do not match logits rows ({lg.size(0)})")
    if overwrite and lg.data_ptr() != logits.data_ptr():
        raise ValueError("cross_entropy(overwrite_logits=True) needs contiguous logits")
    dlogits = lg if overwrite else torch.empty_like(lg)
    loss = torch.empty((), dtype=torch.float32, device=logits.device)
    count = torch.empty((), dtype=torch.int32, device=logits.device)
    L = _lib.lib()
    ws_bytes = L.mlts_ce_workspace_bytes(lg.size(0))
    ws = _workspace(ws_bytes, logits.device)
    _lib.check(L.mlts_ce_fwd_bwd(_p(lg), _p(lb), _p(dlogits), _p(loss), _p(count), _p(ws), ws_bytes, lg.size(0), vocab,
                                 int(ignore_index), _dtype_code(lg), _stream()))
    return loss, dlogits.view(logits.shape), count


# --------------------------------------------------------------------------------------------
# torch.library registration
# --------------------------------------------------------------------------------------------
_LIBRARY = torch.library.Library("maltos", "DEF")
_IDS = "Tensor? q_pos, Tensor? k_pos, Tensor? q_seq, Tensor? k_seq"
_LIBRARY.define(f"attn_fwd(Tensor q, Tensor k, Tensor v, int mask_mode, float scale, {_IDS}) -> (Tensor, Tensor)")
_LIBRARY.define(
    f"attn_bwd(Tensor dout, Tensor q, Tensor k, Tensor v, Tensor o, Tensor lse, int mask_mode, float scale, {_IDS})"
    " -> (Tensor, Tensor, Tensor)"
)
_LIBRARY.define("rmsnorm_fwd(Tensor x, Tensor w, float eps) -> (Tensor, Tensor)")
_LIBRARY.define("rmsnorm_bwd(Tensor dy, Tensor x, Tensor w, Tensor rstd) -> (Tensor, Tensor)")
_LIBRARY.define("add_rmsnorm_fwd(Tensor x, Tensor res, Tensor w, float eps) -> (Tensor, Tensor, Tensor)")
_LIBRARY.define("add_rmsnorm_bwd(Tensor dy, Tensor dres, Tensor h, Tensor w, Tensor rstd) -> (Tensor, Tensor)")
_LIBRARY.define("rope(Tensor x, Tensor cos, Tensor sin, Tensor? positions, int position_offset, bool inverse) -> Tensor")
_LIBRARY.define("rope_pair(Tensor xa, Tensor xb, Tensor cos, Tensor sin, Tensor? positions, int position_offset, bool inverse) -> (Tensor, Tensor)")
_LIBRARY.define("swiglu_fwd(Tensor gate, Tensor up) -> Tensor")
_LIBRARY.define("swiglu_bwd(Tensor dh, Tensor gate, Tensor up) -> (Tensor, Tensor)")
_LIBRARY.define("ce_fwd_bwd(Tensor logits, Tensor labels, int ignore_index) -> (Tensor, Tensor, Tensor)")
_LIBRARY.define("scale_by_scalar(Tensor x, Tensor scale) -> Tensor")
_LIBRARY.define("scale_by_scalar_(Tensor(a!) x, Tensor scale) -> ()")


def _impl(name: str):
    def deco(fn):
        _LIBRARY.impl(name, fn, "CUDA")
        return fn

    return deco


def _cpu_refusal(name: str) -> None:
    def refuse(*args, **kwargs):
        raise RuntimeError(f"maltos::{name} has no CPU implementation; move the tensors to the GPU")

    _LIBRARY.impl(name, refuse, "CPU")


for _name in ("attn_fwd", "attn_bwd", "rmsnorm_fwd", "rmsnorm_bwd", "add_rmsnorm_fwd", "add_rmsnorm_bwd", "rope", "rope_pair", "swiglu_fwd", "swiglu_bwd", "ce_fwd_bwd",
              "scale_by_scalar", "scale_by_scalar_"):
    _cpu_refusal(_name)


@_impl("attn_fwd")
def _attn_fwd_op(q, k, v, mask_mode, scale, q_pos, k_pos, q_seq, k_seq):
    return attention_forward(q, k, v, mask_mode=mask_mode, scale=scale, q_pos=q_pos, k_pos=k_pos, q_seq=q_seq, k_seq=k_seq)


@_impl("attn_bwd")
def _attn_bwd_op(dout, q, k, v, o, lse, mask_mode, scale, q_pos, k_pos, q_seq, k_seq):
    return attention_backward(dout, q, k, v, o, lse, mask_mode=mask_mode, scale=scale, q_pos=q_pos, k_pos=k_pos,
                              q_seq=q_seq, k_seq=k_seq)


_impl("rmsnorm_fwd")(_rmsnorm_fwd)
_impl("rmsnorm_bwd")(_rmsnorm_bwd)
_impl("add_rmsnorm_fwd")(_add_rmsnorm_fwd)
_impl("add_rmsnorm_bwd")(_add_rmsnorm_bwd)
_impl("rope")(_rope)
_impl("rope_pair")(_rope_pair)
_impl("swiglu_fwd")(_swiglu_fwd)
_impl("swiglu_bwd")(_swiglu_bwd)
_impl("ce_fwd_bwd")(_ce_fwd_bwd)


@_impl("scale_by_scalar")
def _scale_by_scalar_op(x, scale):
    _require_gpu(x, scale)
    out = x.contiguous().clone()
    s = scale.to(torch.float32).reshape(1)
    _lib.check(_lib.lib().mlts_scale_by_device_scalar(_p(out), _p(s), out.numel(), _dtype_code(out), _stream()))
    return out


@_impl("scale_by_scalar_")
def _scale_by_scalar_inplace_op(x, scale):
    _require_gpu(x, scale)
    if not x.is_contiguous():
        raise ValueError("scale_by_scalar_ needs a contiguous tensor")
    s = scale.to(torch.float32).reshape(1)
    _lib.check(_lib.lib().mlts_scale_by_device_scalar(_p(x), _p(s), x.numel(), _dtype_code(x), _stream()))


# fake (meta) kernels: shapes/dtypes only, so the ops can be traced or captured
@torch.library.register_fake("maltos::attn_fwd")
def _(q, k, v, mask_mode, scale, q_pos, k_pos, q_seq, k_seq):
    B, H, S, D = q.shape
    return q.new_empty((B, S, H, D)).transpose(1, 2), q.new_empty((B, H, S), dtype=torch.float32)


@torch.library.register_fake("maltos::attn_bwd")
def _(dout, q, k, v, o, lse, mask_mode, scale, q_pos, k_pos, q_seq, k_seq):
    def like(t):
        B, H, S, D = t.shape
        return t.new_empty((B, S, H, D)).transpose(1, 2)

    return like(q), like(k), like(v)


@torch.library.register_fake("maltos::rmsnorm_fwd")
def _(x, w, eps):
    return torch.empty_like(x), x.new_empty((x.numel() // max(1, x.size(-1)),), dtype=torch.float32)


@torch.library.register_fake("maltos::rmsnorm_bwd")
def _(dy, x, w, rstd):
    return torch.empty_like(x), torch.empty_like(w)


@torch.library.register_fake("maltos::add_rmsnorm_fwd")
def _(x, res, w, eps):
    return (torch.empty_like(x), torch.empty_like(x),
            x.new_empty((x.numel() // max(1, x.size(-1)),), dtype=torch.float32))


@torch.library.register_fake("maltos::add_rmsnorm_bwd")
def _(dy, dres, h, w, rstd):
    return torch.empty_like(h), torch.empty_like(w)


@torch.library.register_fake("maltos::rope")
def _(x, cos, sin, positions, position_offset, inverse):
    return torch.empty_like(x)


@torch.library.register_fake("maltos::rope_pair")
def _(xa, xb, cos, sin, positions, position_offset, inverse):
    return torch.empty_like(xa), torch.empty_like(xb)


@torch.library.register_fake("maltos::swiglu_fwd")
def _(gate, up):
    return torch.empty_like(gate)


@torch.library.register_fake("maltos::swiglu_bwd")
def _(dh, gate, up):
    return torch.empty_like(gate), torch.empty_like(up)


@torch.library.register_fake("maltos::ce_fwd_bwd")
def _(logits, labels, ignore_index):
    return (logits.new_empty((), dtype=torch.float32), torch.empty_like(logits),
            logits.new_empty((), dtype=torch.int32))


@torch.library.register_fake("maltos::scale_by_scalar")
def _(x, scale):
    return torch.empty_like(x)


@torch.library.register_fake("maltos::scale_by_scalar_")
def _(x, scale):
    return None


# --------------------------------------------------------------------------------------------
# autograd
# --------------------------------------------------------------------------------------------
def _attn_setup(ctx, inputs, output):
    q, k, v, mask_mode, scale, q_pos, k_pos, q_seq, k_seq = inputs
    o, lse = output
    ctx.save_for_backward(q, k, v, o, lse, q_pos, k_pos, q_seq, k_seq)
    ctx.mask_mode, ctx.scale = mask_mode, scale


def _attn_backward(ctx, do, dlse):
    q, k, v, o, lse, q_pos, k_pos, q_seq, k_seq = ctx.saved_tensors
    dq, dk, dv = torch.ops.maltos.attn_bwd(do, q, k, v, o, lse, ctx.mask_mode, ctx.scale, q_pos, k_pos, q_seq, k_seq)
    return dq, dk, dv, None, None, None, None, None, None


torch.library.register_autograd("maltos::attn_fwd", _attn_backward, setup_context=_attn_setup)


def _rms_setup(ctx, inputs, output):
    x, w, _eps = inputs
    ctx.save_for_backward(x, w, output[1])


def _rms_backward(ctx, dy, _drstd):
    x, w, rstd = ctx.saved_tensors
    dx, dw = torch.ops.maltos.rmsnorm_bwd(dy, x, w, rstd)
    return dx, dw, None


torch.library.register_autograd("maltos::rmsnorm_fwd", _rms_backward, setup_context=_rms_setup)


def _add_rms_setup(ctx, inputs, output):
    _x, _res, w, _eps = inputs
    ctx.save_for_backward(output[0], w, output[2])
    ctx.set_materialize_grads(False)


def _add_rms_backward(ctx, dh, dy, _drstd):
    """dh: gradient of the summed row from its later uses (the residual path), dy: gradient of the normalised row.
    Both addends receive the same gradient."""
    h, w, rstd = ctx.saved_tensors
    if dy is None:
        return dh, dh, None, None
    if dh is None:
        dx, dw = torch.ops.maltos.rmsnorm_bwd(dy, h, w, rstd)
    else:
        dx, dw = torch.ops.maltos.add_rmsnorm_bwd(dy, dh, h, w, rstd)
    return dx, dx, dw, None


torch.library.register_autograd("maltos::add_rmsnorm_fwd", _add_rms_backward, setup_context=_add_rms_setup)


def _rope_setup(ctx, inputs, output):
    _x, cos, sin, positions, position_offset, inverse = inputs
    ctx.save_for_backward(cos, sin, positions)
    ctx.position_offset, ctx.inverse = position_offset, inverse


def _rope_backward(ctx, dy):
    cos, sin, positions = ctx.saved_tensors
    dx = torch.ops.maltos.rope(dy, cos, sin, positions, ctx.position_offset, not ctx.inverse)
    return dx, None, None, None, None, None


torch.library.register_autograd("maltos::rope", _rope_backward, setup_context=_rope_setup)


def _rope_pair_setup(ctx, inputs, output):
    _xa, _xb, cos, sin, positions, position_offset, inverse = inputs
    ctx.save_for_backward(cos, sin, positions)
    ctx.position_offset, ctx.inverse = position_offset, inverse


def _rope_pair_backward(ctx, dya, dyb):
    cos, sin, positions = ctx.saved_tensors
    dxa, dxb = torch.ops.maltos.rope_pair(dya, dyb, cos, sin, positions, ctx.position_offset, not ctx.inverse)
    return dxa, dxb, None, None, None, None, None


torch.library.register_autograd("maltos::rope_pair", _rope_pair_backward, setup_context=_rope_pair_setup)


def _swiglu_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs)


def _swiglu_backward(ctx, dh):
    gate, up = ctx.saved_tensors
    return torch.ops.maltos.swiglu_bwd(dh, gate, up)


torch.library.register_autograd("maltos::swiglu_fwd", _swiglu_backward, setup_context=_swiglu_setup)


def _ce_setup(ctx, inputs, output):
    ctx.save_for_backward(output[1])
    ctx.set_materialize_grads(False)   # no zero tensor of the logits' size for the unused dlogits output
    ctx.dlogits_consumed = False


def _ce_backward(ctx, dloss, _ddlogits, _dcount):
    """d loss / d logits was written by the forward kernel; it is scaled by the upstream gradient in place (the kernel
    returns at once when that is 1, the usual case) and handed on without a copy, so a graph can be walked once."""
    if dloss is None:
        return None, None, None
    if ctx.dlogits_consumed:
        raise RuntimeError("maltos::ce_fwd_bwd: backward ran twice through the same loss; its logits gradient is "
                           "scaled in place by the first pass, so recompute the loss instead of retaining the graph")
    (dlogits,) = ctx.saved_tensors
    torch.ops.maltos.scale_by_scalar_(dlogits, dloss)
    ctx.dlogits_consumed = True
    return dlogits, None, None


torch.library.register_autograd("maltos::ce_fwd_bwd", _ce_backward, setup_context=_ce_setup)


class _CrossEntropyOverLogits(torch.autograd.Function):
    """The loss whose gradient replaces the logits in their buffer: one read and one write of the same addresses (the
    kernel then streams at the rate of an in-place update instead of a copy's) and no second logits-sized tensor.  For
    callers that own the logits and never look at them again; a plain autograd function because an operator that
    overwrites an argument it is differentiated by has no functional form to register."""

    @staticmethod
    def forward(ctx, logits, labels, ignore_index):
        loss, dlogits, _count = _ce_fwd_bwd(logits.detach(), labels, ignore_index, overwrite=True)
        # the kernel wrote through a raw pointer: tell autograd, so that another node that saved these logits for its
        # own backward raises instead of differentiating through the gradient that now stands in their place
        torch.autograd.graph.increment_version(logits)
        ctx.save_for_backward(dlogits)
        ctx.consumed = False
        return loss

    @staticmethod
    def backward(ctx, dloss):
        if ctx.consumed:
            raise RuntimeError("cross_entropy(overwrite_logits=True): backward ran twice through the same loss; its logits "
                               "gradient is scaled in place by the first pass, so recompute the loss instead")
        (dlogits,) = ctx.saved_tensors
        torch.ops.maltos.scale_by_scalar_(dlogits, dloss)
        ctx.consumed = True
        return dlogits, None, None


# --------------------------------------------------------------------------------------------
# public differentiable entry points
# --------------------------------------------------------------------------------------------
def attention(q, k, v, *, mask_mode: int = MASK_CAUSAL, scale: float | None = None, q_pos=None, k_pos=None, q_seq=None,
              k_seq=None, return_lse: bool = False):
    """Differentiable attention; k/v may have fewer heads than q (native GQA)."""
    _check_attn_inputs(q, k, v)
    scale = float(q.size(-1) ** -0.5 if scale is None else scale)
    o, lse = torch.ops.maltos.attn_fwd(q, k, v, int(mask_mode), scale, q_pos, k_pos, q_seq, k_seq)
    return (o, lse) if return_lse else o


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return torch.ops.maltos.rmsnorm_fwd(x, weight, float(eps))[0]


def add_rms_norm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float) -> tuple[torch.Tensor, torch.Tensor]:
    """(h, y) with h = x + residual and y = rms_norm(h), in one pass and with the roundings of the two separate ops."""
    h, y, _ = torch.ops.maltos.add_rmsnorm_fwd(x, residual, weight, float(eps))
    return h, y


def rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, *, positions: torch.Tensor | None = None,
         position_offset: int = 0) -> torch.Tensor:
    return torch.ops.maltos.rope(x, cos, sin, positions, int(position_offset), False)


def rope_pair(xa: torch.Tensor, xb: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, *, positions: torch.Tensor | None = None,
              position_offset: int = 0) -> tuple[torch.Tensor, torch.Tensor]:
    """rope(xa), rope(xb) from one kernel launch (and one in the backward): bit-equal to two `rope` calls."""
    return torch.ops.maltos.rope_pair(xa, xb, cos, sin, positions, int(position_offset), False)


def rope_pair_(xa: torch.Tensor, xb: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, *, positions: torch.Tensor | None = None,
               position_offset: int = 0, inverse: bool = False) -> None:
    """`rope_pair` written over its inputs, outside autograd (`inverse` rotates back: the backward pass).  For buffers
    the caller owns, e.g. the gradients an attention backward has just produced."""
    _rope_pair(xa, xb, cos, sin, positions, int(position_offset), inverse, in_place=True)


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return torch.ops.maltos.swiglu_fwd(gate, up)


def cross_entropy(logits: torch.Tensor, labels: torch.Tensor, ignore_index: int = -100, *,
                  overwrite_logits: bool = False) -> torch.Tensor:
    """fp32 scalar: sum CE over supervised rows / max(1, #supervised rows).  overwrite_logits=True lets the gradient take
    the place of the (contiguous) logits, which the caller must not read afterwards."""
    if overwrite_logits:
        return _CrossEntropyOverLogits.apply(logits, labels, int(ignore_index))
    return torch.ops.maltos.ce_fwd_bwd(logits, labels, int(ignore_index))[0]


# --------------------------------------------------------------------------------------------
# optimizer-step launches (in place, no autograd)
# --------------------------------------------------------------------------------------------
def _flat_f32(t: torch.Tensor, what: str) -> torch.Tensor:
    if t.dtype != torch.float32 or not t.is_contiguous():
        raise ValueError(f"{what} must be a contiguous float32 tensor")
    return t


def adamw_step_(p, g, m, v, *, lr: float, beta1: float, beta2: float, eps: float, weight_decay: float, step: int,
                p_lowp: torch.Tensor | None = None, grad_scale: float = 1.0, sq_norm: torch.Tensor | None = None,
                max_norm: float = 0.0) -> None:
    _require_gpu(p, g, m, v, p_lowp, sq_norm)
    for name, t in (("param", p), ("grad", g), ("exp_avg", m), ("exp_avg_sq", v)):
        _flat_f32(t, name)
        if t.numel() != p.numel():
            raise ValueError("param, grad, exp_avg, exp_avg_sq must have the same number of elements")
    if p_lowp is not None and (p_lowp.dtype != torch.bfloat16 or p_lowp.numel() != p.numel() or not p_lowp.is_contiguous()):
        raise ValueError("p_lowp must be a contiguous bfloat16 tensor matching param")
    if sq_norm is not None and (sq_norm.dtype != torch.float64 or sq_norm.numel() != 1):
        raise ValueError("sq_norm must be a float64 scalar tensor")
    if step < 1:
        raise ValueError("step is the 1-based optimizer step count")
    _lib.check(_lib.lib().mlts_adamw_step(_p(p), _p(g), _p(m), _p(v), _p(p_lowp), p.numel(), lr, beta1, beta2, eps,
                                          weight_decay, int(step), grad_scale, _p(sq_norm), max_norm, _stream()))


def sq_norm(x: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """float64 0-d tensor: sum of squares of a float32 tensor, accumulated in fp64."""
    _require_gpu(x, out)
    _flat_f32(x, "x")
    out = torch.empty((), dtype=torch.float64, device=x.device) if out is None else out
    ws = _workspace(_lib.SQNORM_WS_BYTES, x.device)
    _lib.check(_lib.lib().mlts_sq_norm(_p(x), x.numel(), _p(out), _p(ws), _stream()))
    return out


def scale_(x: torch.Tensor, scale: float) -> torch.Tensor:
    _require_gpu(x)
    _flat_f32(x, "x")
    _lib.check(_lib.lib().mlts_scale(_p(x), float(scale), x.numel(), _stream()))
    return x


def grad_sum_slices(parts: torch.Tensor, out: torch.Tensor | None = None, *, accumulate: bool = False) -> torch.Tensor:
    """parts [slices, ...] -> sum over the slices, added in fp32 and rounded once; with `out` the result is written
    there (accumulate=True: added onto what `out` holds)."""
    _require_gpu(parts, out)
    if parts.dim() < 2 or not parts.is_contiguous():
        raise ValueError("parts must be a contiguous tensor [slices, ...]")
    if out is None:
        if accumulate:
            raise ValueError("accumulate=True needs an output tensor")
        out = torch.empty(parts.shape[1:], dtype=parts.dtype, device=parts.device)
    elif out.dtype != parts.dtype or out.shape != parts.shape[1:] or not out.is_contiguous():
        raise ValueError("out must be contiguous with the dtype and the per-slice shape of parts")
    _lib.check(_lib.lib().mlts_grad_sum_slices(_p(out), _p(parts), _dtype_code(parts), parts.size(0), out.numel(),
                                               int(accumulate), _stream()))
    return out


def grad_to_f32_(dst: torch.Tensor, src: torch.Tensor, *, accumulate: bool = False,
                 sq_out: torch.Tensor | None = None) -> torch.Tensor:
    """dst (=|+=) float(src) over flat buffers, optionally fusing the fp64 sum of squares of dst."""
    _require_gpu(dst, src, sq_out)
    _flat_f32(dst, "dst")
    if src.numel() != dst.numel() or not src.is_contiguous():
        raise ValueError("src must be contiguous and match dst in size")
    ws = _workspace(_lib.SQNORM_WS_BYTES, dst.device) if sq_out is not None else None
    _lib.check(_lib.lib().mlts_grad_to_f32(_p(dst), _p(src), _dtype_code(src), dst.numel(), int(accumulate), _p(sq_out),
                                           _p(ws), _stream()))
    return dst
