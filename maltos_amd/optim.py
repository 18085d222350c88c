"""Optimizer side of the hot path: fused AdamW over flat fp32 buffers and the master-weights wrapper.

Counterparts in the reference:
  * FusedAdamW            <- torch.optim.AdamW(..., fused=True) as built by train/cli.py:420-443; usable
                             as the `optimizer_factory` result RuntimeCore asks for (runtime/core.py:300-325).
  * MasterWeightsOptimizer <- runtime/optim.py:10-104, same constructor, duck-typed methods
                             (copy_master_params, model_param_for, sync_master_params_from_model) and
                             state_dict keys {"inner_optimizer", "master_params", "master_dtype"}.

MI355X-first layout: parameters that are adjacent views of one allocation are stepped as ONE flat
segment (one kernel launch over p/g/m/v), the way the reference's ZeRO plugins lay their shards out
(runtime/plugins/zero1.py:98-164).  MasterWeightsOptimizer builds exactly that layout: one flat fp32
master buffer, one flat fp32 master-grad buffer, and (flat=True) the low-precision model parameters
and their .grad re-pointed into flat buffers too, so that
    copy_master_params  = one bf16->fp32 pass (optionally fused with the fp64 grad-norm), and
    step                = one AdamW pass that also writes the bf16 model copy.
"""
from __future__ import annotations

from collections.abc import Callable, Iterable
from typing import Any

import torch
import torch.nn as nn

from . import ops


# Which parameters received a gradient in this step.  With gradients bound to a flat buffer `param.grad` is never None,
# so "no gradient" (which the reference's optimizers skip, runtime/optim.py:46-50) has to be told another way: whoever
# writes a parameter's gradient says so.  Autograd's own accumulation says it through a post-accumulate-grad hook that
# the flat optimizer layout registers; code that adds into `param.grad` itself (HipLinear.accumulate_into_grad, a
# replayed HIP graph, a reduce-scatter into a shard's gradient) calls notify_grad_written.
_GRAD_WRITE_LISTENERS: list[list] = []


def notify_grad_written(param: torch.Tensor) -> None:
    mark = param.__dict__.get("_maltos_hip_grad_written")
    if mark is not None:
        mark()
    for seen in _GRAD_WRITE_LISTENERS:
        seen.append(param)


class grad_write_listener:
    """`with grad_write_listener() as seen:` collects the parameters whose gradient is reported written inside the block
    (what a recorder of a backward pass keeps, to report the same parameters again after every replay)."""

    def __enter__(self) -> list:
        self._seen: list = []
        _GRAD_WRITE_LISTENERS.append(self._seen)
        return self._seen

    def __exit__(self, *exc) -> None:
        _GRAD_WRITE_LISTENERS.remove(self._seen)


def _is_flat_neighbour(prev: torch.Tensor, nxt: torch.Tensor) -> bool:
    return (prev.untyped_storage().data_ptr() == nxt.untyped_storage().data_ptr()
            and prev.data_ptr() + prev.numel() * prev.element_size() == nxt.data_ptr())


class _Segment:
    """Parameters that live in one flat fp32 allocation (possibly with alignment padding between them)
    and are stepped by a single kernel launch when their grads form the matching flat buffer."""

    def __init__(self, params: list[nn.Parameter], offsets: list[int], flat_p: torch.Tensor,
                 flat_g: torch.Tensor | None = None) -> None:
        self.params = params
        self.offsets = offsets
        self.flat_p = flat_p
        self.numel = flat_p.numel()
        self.bound_grad = flat_g
        self.exp_avg = torch.zeros(self.numel, dtype=torch.float32, device=flat_p.device)
        self.exp_avg_sq = torch.zeros(self.numel, dtype=torch.float32, device=flat_p.device)

    def flat_grad(self) -> torch.Tensor | None:
        """The grads as one flat tensor laid out like flat_p, or None if they are scattered."""
        grads = [p.grad for p in self.params]
        if any(g is None or not g.is_contiguous() or g.dtype != torch.float32 for g in grads):
            return None
        if self.bound_grad is not None:
            base = self.bound_grad.data_ptr()
            if all(g.data_ptr() == base + off * 4 for g, off in zip(grads, self.offsets)):
                return self.bound_grad
            return None
        if any(off != sum(p.numel() for p in self.params[:i]) for i, off in enumerate(self.offsets)):
            return None
        for a, b in zip(grads, grads[1:]):
            if not _is_flat_neighbour(a, b):
                return None
        return grads[0].as_strided((self.numel,), (1,))


class FusedAdamW(torch.optim.Optimizer):
    """AdamW (decoupled weight decay, bias correction, eps added after sqrt) on the HIP kernel.

    Same hyper-parameters, param_groups and per-parameter state keys ("step", "exp_avg", "exp_avg_sq")
    as torch.optim.AdamW, so schedulers and checkpoints carry over.  `lr` is read from the param group at
    every step.  Parameters must be float32 on the GPU (wrap low-precision models in MasterWeightsOptimizer).

    Optional fused extras, used by MasterWeightsOptimizer and the clip helper:
      * set_lowp_shadow(flat_master, flat_lowp): also write bf16(p) for that flat master segment;
      * set_clip(sq_norm, max_norm): scale grads by max_norm / (sqrt(sq_norm) + 1e-6) when that is < 1,
        with sq_norm a device fp64 scalar (no host synchronisation).
    """

    def __init__(self, params, lr: float = 1e-3, betas: tuple[float, float] = (0.9, 0.999), eps: float = 1e-8,
                 weight_decay: float = 1e-2) -> None:
        if lr < 0:
            raise ValueError(f"Invalid learning rate: {lr}")
        if eps <= 0:
            raise ValueError(f"Invalid epsilon value: {eps}")
        if not 0.0 <= betas[0] < 1.0 or not 0.0 <= betas[1] < 1.0:
            raise ValueError(f"Invalid betas: {betas}")
        if weight_decay < 0:
            raise ValueError(f"Invalid weight_decay value: {weight_decay}")
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))
        self._segments: dict[int, list[_Segment]] = {}
        self._shadow: dict[int, torch.Tensor] = {}
        self._clip: tuple[torch.Tensor, float] | None = None
        self._bound = None

    # ---- fused extras ---------------------------------------------------------------------
    def set_lowp_shadow(self, flat_master: torch.Tensor, flat_lowp: torch.Tensor) -> None:
        if flat_lowp.dtype != torch.bfloat16 or flat_lowp.numel() != flat_master.numel():
            raise ValueError("the low-precision shadow must be bfloat16 and match the master segment")
        self._shadow[flat_master.data_ptr()] = flat_lowp

    def set_clip(self, sq_norm: torch.Tensor | None, max_norm: float = 0.0) -> None:
        self._clip = None if sq_norm is None else (sq_norm, float(max_norm))

    # ---- layout ---------------------------------------------------------------------------
    def bind_flat(self, flat_p: torch.Tensor, flat_g: torch.Tensor, params: list[nn.Parameter], offsets: list[int]) -> None:
        """Declare that `params` are views of `flat_p` at element `offsets` and their grads views of `flat_g`
        at the same offsets: they are then stepped by one launch over the whole (padded) buffer."""
        if flat_p.dtype != torch.float32 or flat_g.dtype != torch.float32 or flat_p.numel() != flat_g.numel():
            raise ValueError("bind_flat needs matching float32 flat parameter and gradient buffers")
        self._bound = (flat_p, flat_g, list(params), list(offsets))
        self._segments.clear()

    def _adopt_state(self, seg: _Segment) -> None:
        for p, off in zip(seg.params, seg.offsets):
            st = self.state[p]
            n = p.numel()
            views = (seg.exp_avg[off:off + n].view_as(p), seg.exp_avg_sq[off:off + n].view_as(p))
            if "exp_avg" in st:  # state restored from a checkpoint: keep its values
                views[0].copy_(st["exp_avg"])
                views[1].copy_(st["exp_avg_sq"])
            st["exp_avg"], st["exp_avg_sq"] = views
            if "step" not in st:
                st["step"] = torch.tensor(0.0)
            elif not torch.is_tensor(st["step"]):
                st["step"] = torch.tensor(float(st["step"]))
            else:
                st["step"] = st["step"].detach().to("cpu", torch.float32)

    def _build_segments(self, group_index: int, group: dict[str, Any]) -> list[_Segment]:
        params = [p for p in group["params"] if p.requires_grad]
        for p in params:
            if not p.is_cuda or p.dtype != torch.float32 or not p.is_contiguous():
                raise ValueError("FusedAdamW needs contiguous float32 GPU parameters "
                                 "(use MasterWeightsOptimizer for bf16 models)")
        segments: list[_Segment] = []
        bound = getattr(self, "_bound", None)
        if bound is not None and {id(p) for p in bound[2]} == {id(p) for p in params}:
            segments.append(_Segment(bound[2], bound[3], bound[0], bound[1]))
        else:
            ordered = sorted(params, key=lambda p: p.data_ptr())
            run: list[nn.Parameter] = []

            def close(run_params: list[nn.Parameter]) -> None:
                offs, cur = [], 0
                for q in run_params:
                    offs.append(cur)
                    cur += q.numel()
                segments.append(_Segment(run_params, offs, run_params[0].data.as_strided((cur,), (1,))))

            for p in ordered:
                if run and not _is_flat_neighbour(run[-1].data, p.data):
                    close(run)
                    run = []
                run.append(p)
            if run:
                close(run)
        for seg in segments:
            self._adopt_state(seg)
        return segments

    def load_state_dict(self, state_dict: dict[str, Any]) -> None:
        super().load_state_dict(state_dict)
        self._segments.clear()  # rebuilt (adopting the loaded moments) at the next step

    # ---- step -----------------------------------------------------------------------------
    @torch.no_grad()
    def step(self, closure: Callable[[], float] | None = None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        sq_norm, max_norm = self._clip if self._clip is not None else (None, 0.0)
        for gi, group in enumerate(self.param_groups):
            if gi not in self._segments:
                self._segments[gi] = self._build_segments(gi, group)
            beta1, beta2 = group["betas"]
            hyper = dict(lr=float(group["lr"]), beta1=float(beta1), beta2=float(beta2), eps=float(group["eps"]),
                         weight_decay=float(group["weight_decay"]), sq_norm=sq_norm, max_norm=max_norm)
            for seg in self._segments[gi]:
                flat_g = seg.flat_grad()
                # one launch over the whole segment needs one step count (the bias corrections are launch arguments);
                # the counts differ once a parameter was skipped in an earlier step for want of a gradient
                steps = {float(self.state[p]["step"]) for p in seg.params}
                if flat_g is not None and len(steps) == 1:
                    for p in seg.params:
                        self.state[p]["step"] += 1
                    ops.adamw_step_(seg.flat_p, flat_g, seg.exp_avg, seg.exp_avg_sq, step=int(steps.pop()) + 1,
                                    p_lowp=self._shadow.get(seg.flat_p.data_ptr()), **hyper)
                    continue
                shadow = self._shadow.get(seg.flat_p.data_ptr())
                for p, offset in zip(seg.params, seg.offsets):
                    n = p.numel()
                    if p.grad is not None:
                        g = p.grad
                        if g.dtype != torch.float32 or not g.is_contiguous():
                            g = g.to(torch.float32).contiguous()
                        st = self.state[p]
                        st["step"] += 1
                        ops.adamw_step_(seg.flat_p[offset:offset + n], g.view(-1), seg.exp_avg[offset:offset + n],
                                        seg.exp_avg_sq[offset:offset + n], step=int(st["step"].item()),
                                        p_lowp=None if shadow is None else shadow[offset:offset + n], **hyper)
        return loss


class MasterWeightsOptimizer(torch.optim.Optimizer):
    """Keeps model params in low precision, steps fp32 masters (see module docstring for the layout)."""

    def __init__(self, params: Iterable[nn.Parameter], *, optimizer_factory, master_dtype: torch.dtype = torch.float32,
                 flat: bool = True) -> None:
        model_params = [p for p in params if p.requires_grad]
        if not model_params:
            raise ValueError("MasterWeightsOptimizer requires at least one trainable parameter")
        if master_dtype != torch.float32:
            raise ValueError("the HIP path keeps master weights in float32")
        self.model_params = model_params
        self.master_dtype = master_dtype
        device = model_params[0].device
        total = sum(p.numel() for p in model_params)
        self._gpu = all(p.is_cuda for p in model_params)
        # 16-element padding between parameters keeps every view 16-byte aligned in bf16 and fp32
        self._offsets: list[int] = []
        cursor = 0
        for p in model_params:
            self._offsets.append(cursor)
            cursor += (p.numel() + 15) // 16 * 16
        self._flat_numel = cursor
        self.flat_master = torch.zeros(cursor, dtype=torch.float32, device=device)
        self.flat_master_grad = torch.zeros(cursor, dtype=torch.float32, device=device)
        self.master_params = []
        for p, off in zip(model_params, self._offsets):
            view = self.flat_master[off:off + p.numel()].view_as(p)
            view.copy_(p.detach())
            mp = nn.Parameter(view, requires_grad=True)
            mp.grad = self.flat_master_grad[off:off + p.numel()].view_as(p)
            self.master_params.append(mp)
        self._model_param_by_master_id = {id(m): p for p, m in zip(model_params, self.master_params)}
        lowp_dtypes = {p.dtype for p in model_params}
        self._flat_model = bool(flat) and self._gpu and lowp_dtypes == {torch.bfloat16}
        self.flat_model: torch.Tensor | None = None
        self.flat_model_grad: torch.Tensor | None = None
        if self._flat_model:
            self.flat_model = torch.zeros(cursor, dtype=torch.bfloat16, device=device)
            self.flat_model_grad = torch.zeros(cursor, dtype=torch.bfloat16, device=device)
            for p, off in zip(model_params, self._offsets):
                view = self.flat_model[off:off + p.numel()].view_as(p)
                view.copy_(p.detach())
                p.data = view
            self._bind_model_grads()
        super().__init__(self.master_params, defaults={})
        self._optimizer = optimizer_factory(self.master_params)
        self.param_groups = self._optimizer.param_groups
        self.defaults = self._optimizer.defaults
        self.state = self._optimizer.state
        self._master_grads_copied = False
        self._fused = isinstance(self._optimizer, FusedAdamW)
        if self._fused and self._gpu:
            # padding is stepped too (zeros stay zeros), so the whole buffer is one kernel launch
            self._optimizer.bind_flat(self.flat_master, self.flat_master_grad, self.master_params, self._offsets)
            if self._flat_model:
                self._optimizer.set_lowp_shadow(self.flat_master, self.flat_model)
        self.grad_sq_norm: torch.Tensor | None = None  # device fp64 scalar, filled by copy_master_params(fuse_norm=True)
        del total
        # flat layout: which parameters' gradients were written since the last zero_grad (see notify_grad_written)
        self._grad_written = [False] * len(model_params)
        if self._flat_model:
            for i, p in enumerate(model_params):
                p.__dict__["_maltos_hip_grad_written"] = lambda i=i: self._grad_written.__setitem__(i, True)
                p.register_post_accumulate_grad_hook(notify_grad_written)

    # ---- helpers --------------------------------------------------------------------------
    def _bind_model_grads(self) -> None:
        assert self.flat_model_grad is not None
        for p, off in zip(self.model_params, self._offsets):
            p.grad = self.flat_model_grad[off:off + p.numel()].view_as(p)

    def _grads_are_flat(self) -> bool:
        if not self._flat_model:
            return False
        assert self.flat_model_grad is not None
        base = self.flat_model_grad.data_ptr()
        return all(p.grad is not None and p.grad.data_ptr() == base + off * 2 and p.grad.is_contiguous()
                   for p, off in zip(self.model_params, self._offsets))

    def model_param_for(self, param: nn.Parameter) -> nn.Parameter:
        return self._model_param_by_master_id.get(id(param), param)

    def mark_grads_written(self, params: Iterable[nn.Parameter] | None = None) -> None:
        """For code that fills the bound `.grad` views itself, without autograd: these parameters (default: all) have a
        gradient this step.  Parameters nobody reported are skipped by `step()`, as parameters whose `.grad` is None
        are by the reference (runtime/optim.py:46-50)."""
        if params is None:
            self._grad_written = [True] * len(self.model_params)
            return
        for p in params:
            notify_grad_written(p)

    # ---- reference API ----------------------------------------------------------------------
    def copy_master_params(self, fuse_norm: bool = False) -> None:
        """Upcast model grads into the fp32 master grads, once per step (reference :43-56)."""
        if self._master_grads_copied:
            return
        if self._grads_are_flat():
            sq = None
            if fuse_norm:
                sq = torch.empty((), dtype=torch.float64, device=self.flat_master.device)
            ops.grad_to_f32_(self.flat_master_grad, self.flat_model_grad, sq_out=sq)
            self.grad_sq_norm = sq
            for mp in self.master_params:
                if mp.grad is None:
                    off = self._offsets[self.master_params.index(mp)]
                    mp.grad = self.flat_master_grad[off:off + mp.numel()].view_as(mp)
        else:
            self.grad_sq_norm = None
            for p, mp, off in zip(self.model_params, self.master_params, self._offsets):
                if p.grad is None:
                    mp.grad = None
                    continue
                dst = self.flat_master_grad[off:off + p.numel()]
                if self._gpu and p.grad.is_contiguous() and p.grad.dtype in (torch.bfloat16, torch.float32):
                    ops.grad_to_f32_(dst, p.grad.view(-1))
                else:
                    dst.copy_(p.grad.detach().reshape(-1).to(torch.float32))
                mp.grad = dst.view_as(p)
        self._master_grads_copied = True

    def sync_master_params_from_model(self) -> None:
        """Refresh the fp32 masters after model parameters were loaded externally (reference :58-63)."""
        with torch.no_grad():
            for p, mp in zip(self.model_params, self.master_params):
                mp.copy_(p.to(dtype=mp.dtype))
        self._master_grads_copied = False

    def step(self, closure=None):
        self.copy_master_params()
        partial = self._flat_model and self._grads_are_flat() and not all(self._grad_written)
        if partial:
            # parameters without a gradient this step are left alone (no weight decay, no moment decay, no step count),
            # like parameters whose .grad is None in the reference; the others are then stepped one launch each
            for mp, written in zip(self.master_params, self._grad_written):
                if not written:
                    mp.grad = None
        try:
            loss = self._optimizer.step(closure)
        finally:
            if partial:
                for mp, off in zip(self.master_params, self._offsets):
                    if mp.grad is None:
                        mp.grad = self.flat_master_grad[off:off + mp.numel()].view_as(mp)
        # the fused step has written the bf16 model copy of everything it stepped
        fused_writeback = self._fused and self._flat_model and (partial or all(mp.grad is not None for mp in self.master_params))
        if not fused_writeback:
            with torch.no_grad():
                for p, mp in zip(self.model_params, self.master_params):
                    p.copy_(mp.to(dtype=p.dtype))
        return loss

    def zero_grad(self, set_to_none: bool = True) -> None:
        """Flat layouts keep their grad views and clear the buffers; otherwise as the reference (:73-80)."""
        if self._flat_model:
            assert self.flat_model_grad is not None
            self.flat_model_grad.zero_()
            self._bind_model_grads()
            self._grad_written = [False] * len(self.model_params)
        else:
            for p in self.model_params:
                if set_to_none:
                    p.grad = None
                elif p.grad is not None:
                    p.grad.zero_()
        self._master_grads_copied = False
        self.grad_sq_norm = None

    def state_dict(self) -> dict[str, Any]:
        return {
            "inner_optimizer": self._optimizer.state_dict(),
            "master_params": [mp.detach().cpu().clone() for mp in self.master_params],
            "master_dtype": str(self.master_dtype),
        }

    def load_state_dict(self, state_dict: dict[str, Any]) -> None:
        self._optimizer.load_state_dict(state_dict.get("inner_optimizer", state_dict))
        self.param_groups = self._optimizer.param_groups
        self.defaults = self._optimizer.defaults
        self.state = self._optimizer.state
        saved = state_dict.get("master_params")
        if isinstance(saved, list):
            if len(saved) != len(self.master_params):
                raise ValueError("master_params length does not match this optimizer")
            for mp, t in zip(self.master_params, saved):
                if not torch.is_tensor(t):
                    raise TypeError("master_params entries must be tensors")
                mp.data.copy_(t.to(device=mp.device, dtype=mp.dtype))
        with torch.no_grad():
            for p, mp in zip(self.model_params, self.master_params):
                p.copy_(mp.to(dtype=p.dtype))
        self._master_grads_copied = False
