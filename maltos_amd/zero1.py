"""One rank's side of the reference's ZeRO-1 flat buffers, so that the fused optimizer drops into that layout.

Mirror of `Zero1Plugin._prepare_buffers_and_buckets` and the step phases around it
(runtime/plugins/zero1.py:98-164, 186-260, 283-287; runtime/plugins/zero_common.py:176-193, 293-351):

  * trainable parameters in REVERSE `model.parameters()` order, grouped greedily into buckets of at most
    `bucket_mb_size` MiB (a parameter larger than that gets a bucket of its own), every bucket padded to a multiple
    of `world_size`;
  * one flat `data_buffer` and one flat `grad_buffer` in the parameters' dtype; `param.data` / `param.grad` are
    re-pointed to views of them;
  * per bucket a `local_param`: a clone of this rank's 1 / world_size slice, which is what the optimizer owns.

What moves data between ranks is a seam, not part of this module (everything here runs on one GPU): with
world_size == 1 the reduce-scatter and the all-gather are the local copies the reference itself makes
(`LocalCopyWork`, zero1.py:193-197, 247-249); with world_size > 1 the caller passes `reduce_scatter_avg`,
`all_gather` and `all_reduce_sum` callables.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Callable

import torch
import torch.nn as nn


def build_param_buckets(params: list[nn.Parameter], bucket_byte_size: int) -> list[list[nn.Parameter]]:
    """Greedy grouping in the given order; a bucket is closed when the next parameter would push it past the limit
    (zero_common.py:176-193)."""
    buckets: list[list[nn.Parameter]] = []
    current: list[nn.Parameter] = []
    current_bytes = 0
    for param in params:
        nbytes = param.numel() * param.element_size()
        if current and current_bytes + nbytes > bucket_byte_size:
            buckets.append(current)
            current, current_bytes = [], 0
        current.append(param)
        current_bytes += nbytes
    if current:
        buckets.append(current)
    return buckets


def padded_len(numel: int, world_size: int) -> int:
    """zero_common.py:293-294."""
    return (numel + world_size - 1) // world_size * world_size


def role_params(model: nn.Module) -> list[nn.Parameter]:
    """Trainable parameters, last registered first (zero_common.py:296-302; every LLaMA parameter has the shared role)."""
    return [p for p in model.parameters() if p.requires_grad][::-1]


@dataclass(eq=False)   # a bucket is itself: comparing the tensors it holds field by field is never meant
class Bucket:
    """zero1.py:24-36 without the process-group fields."""

    params: list[nn.Parameter]
    logical_names: list[str]
    start: int
    end: int
    shard_start: int
    shard_end: int
    local_param: nn.Parameter
    # ZeRO-2 only (zero2.py:34-35 of the reference): reductions still to fire in this backward, per-micro-batch buffers
    pending_exec_reductions: int = 0
    exec_states: list = field(default_factory=list)


ReduceScatter = Callable[[torch.Tensor, torch.Tensor], None]   # (out_shard, full_grad): out <- this rank's slice of the mean
AllGather = Callable[[torch.Tensor, torch.Tensor], None]       # (out_full, local_shard)
AllReduceSum = Callable[[torch.Tensor], None]                  # in place, fp64 scalar


class Zero1FlatBuffers:
    """Flat data/grad buffers, buckets and local shards of one rank, with the reference's step phases as methods.

    `optimizer_factory(local_params) -> optimizer` receives the per-bucket `local_param`s, as
    `runtime.create_optimizer` does in the reference (zero1.py:74-76); for bf16 models pass a factory that wraps them
    in `MasterWeightsOptimizer` (runtime/core.py:319-325).
    """

    # ZeRO-1 keeps one gradient buffer laid out like the data buffer; a subclass that brings its own gradient buffers
    # (ZeRO-2: one per bucket and micro-batch) turns this off and `grad_buffer` stays None
    whole_model_grad_buffer = True

    def __init__(self, model: nn.Module, *, optimizer_factory: Callable[[list[nn.Parameter]], torch.optim.Optimizer],
                 world_size: int = 1, rank: int = 0, bucket_mb_size: int = 25,
                 reduce_scatter_avg: ReduceScatter | None = None, all_gather: AllGather | None = None,
                 all_reduce_sum: AllReduceSum | None = None) -> None:
        if world_size < 1 or not 0 <= rank < world_size:
            raise ValueError(f"bad rank {rank} for world_size {world_size}")
        if world_size > 1 and (reduce_scatter_avg is None or all_gather is None or all_reduce_sum is None):
            raise ValueError("world_size > 1 needs reduce_scatter_avg, all_gather and all_reduce_sum")
        self.world_size, self.rank = world_size, rank
        self.bucket_byte_size = bucket_mb_size * 1024 * 1024
        self._reduce_scatter_avg, self._all_gather, self._all_reduce_sum = reduce_scatter_avg, all_gather, all_reduce_sum
        self.data_buffer: torch.Tensor | None = None
        self.grad_buffer: torch.Tensor | None = None
        self.buckets: list[Bucket] = []
        self.grad_norm: float | None = None
        self._prepare_buffers_and_buckets(model)
        self.optimizer = optimizer_factory([b.local_param for b in self.buckets]) if self.buckets else None

    # ---- zero1.py:98-164 ---------------------------------------------------------------------------------------
    def _prepare_buffers_and_buckets(self, model: nn.Module) -> None:
        params = role_params(model)
        if not params:
            return
        dtype, device = params[0].dtype, params[0].device
        names = {id(p): n for n, p in model.named_parameters()}
        param_buckets = build_param_buckets(params, self.bucket_byte_size)
        padded = [padded_len(sum(p.numel() for p in bucket), self.world_size) for bucket in param_buckets]
        total = sum(padded)
        self.data_buffer = torch.zeros(total, dtype=dtype, device=device)
        if self.whole_model_grad_buffer:
            self.grad_buffer = torch.zeros(total, dtype=dtype, device=device)
        offset = 0
        for bucket_params, padded_size in zip(param_buckets, padded):
            cursor = offset
            for param in bucket_params:
                n = param.numel()
                with torch.no_grad():
                    self.data_buffer[cursor:cursor + n].copy_(param.detach().reshape(-1))
                    param.data = self.data_buffer[cursor:cursor + n].view_as(param)
                    if self.grad_buffer is not None:
                        param.grad = self.grad_buffer[cursor:cursor + n].view_as(param)
                cursor += n
            per_rank = padded_size // self.world_size
            shard_start = offset + self.rank * per_rank
            shard_end = shard_start + per_rank
            self.buckets.append(Bucket(
                params=bucket_params, logical_names=[names[id(p)] for p in bucket_params], start=offset,
                end=offset + padded_size, shard_start=shard_start, shard_end=shard_end,
                local_param=nn.Parameter(self.data_buffer[shard_start:shard_end].clone())))
            offset += padded_size

    # ---- PRE_BACKWARD: zero1.py:270-276 -----------------------------------------------------------------------
    def reset_grads(self) -> None:
        """Start of an accumulation window: the flat grad buffer is zeroed (the views stay bound) and the optimizer's
        own gradients are cleared, as the runtime's `optimizer.zero_grad(set_to_none=True)` does between steps (a
        master-weights optimizer also forgets its fp32 copy of the previous step's gradients there)."""
        assert self.grad_buffer is not None
        self.grad_buffer.zero_()
        if self.optimizer is not None:
            self.optimizer.zero_grad(set_to_none=True)

    # ---- POST_BACKWARD: zero1.py:186-212 ----------------------------------------------------------------------
    def reduce_grads(self) -> None:
        """This rank's slice of the mean gradient of every bucket into `local_param.grad`."""
        assert self.grad_buffer is not None
        for bucket in self.buckets:
            if bucket.local_param.grad is None:
                bucket.local_param.grad = torch.empty_like(bucket.local_param.data)
            full_grad = self.grad_buffer[bucket.start:bucket.end]
            if self.world_size == 1:
                bucket.local_param.grad.copy_(full_grad[bucket.shard_start - bucket.start:bucket.shard_end - bucket.start])
            else:
                self._reduce_scatter_avg(bucket.local_param.grad, full_grad)
        # the shards' gradients were filled by hand, not by autograd: tell an optimizer that skips parameters without a
        # gradient that every shard has one (the reference's ZeRO plugins step every shard, zero1.py:214-234)
        mark = getattr(self.optimizer, "mark_grads_written", None)
        if callable(mark):
            mark()

    # ---- PRE_STEP: zero_common.py:307-351, zero1.py:214-234 ---------------------------------------------------
    def local_sq_norm(self) -> torch.Tensor:
        """fp64 sum of squares of this rank's gradient shards (the padding holds zeros; replica factor 1)."""
        device = self.buckets[0].local_param.device
        total = torch.zeros((), dtype=torch.float64, device=device)
        for bucket in self.buckets:
            grad = bucket.local_param.grad
            if grad is not None:
                total += _sq_norm_f64(grad)
        return total

    def clip_local_shards(self, max_norm: float | None) -> float | None:
        """Scales the local gradient shards when max_norm / (global norm + 1e-6) < 1; returns the norm."""
        if max_norm is None or not self.buckets or all(b.local_param.grad is None for b in self.buckets):
            return None
        # An optimizer that keeps fp32 masters (MasterWeightsOptimizer) takes its fp32 copy of the shard gradients
        # here, in the same pass that sums their squares; norm and scaling then act on that copy (the reference
        # scales the low-precision shards and copies afterwards: the same numbers up to one bf16 rounding of g).
        master_grads = getattr(self.optimizer, "flat_master_grad", None)
        fused = master_grads is not None and master_grads.is_cuda
        if fused:
            from .grad_clip import global_grad_sq_norm
            local_sq = global_grad_sq_norm(self.optimizer)
        else:
            local_sq = self.local_sq_norm()
        if self.world_size > 1:
            self._all_reduce_sum(local_sq)
        global_norm = float(local_sq.sqrt().item())
        if not math.isfinite(global_norm):
            bad = [f"bucket={i} names={b.logical_names[:4]}" for i, b in enumerate(self.buckets)
                   if b.local_param.grad is not None and not torch.isfinite(b.local_param.grad).all()]
            details = "; ".join(bad[:8]) or "no local non-finite shard found"
            raise FloatingPointError("non-finite ZeRO gradient norm; refusing optimizer step to avoid inf * 0 -> NaN. "
                                     f"Affected local shards: {details}")
        clip_coef = float(max_norm) / (global_norm + 1e-6)
        if clip_coef < 1.0:
            if fused:
                from . import ops
                ops.scale_(master_grads, clip_coef)
            else:
                for bucket in self.buckets:
                    if bucket.local_param.grad is not None:
                        bucket.local_param.grad.mul_(clip_coef)
        self.grad_norm = global_norm
        return global_norm

    def clip_local_shards_on_device(self, max_norm: float) -> torch.Tensor:
        """The same clip without the host reading the norm: the fp64 sum of squares of all shards stays on the device
        (summed over the ranks by `all_reduce_sum`) and the fused AdamW kernel applies max_norm / (norm + 1e-6) to the
        gradients it reads when that is below 1.  Returns the device scalar (its square root is the norm).  Needs the
        fp32 master copy of `MasterWeightsOptimizer` over `FusedAdamW`; a non-finite norm is not detected here."""
        from .grad_clip import global_grad_sq_norm
        inner = getattr(self.optimizer, "_optimizer", self.optimizer)
        set_clip = getattr(inner, "set_clip", None)
        if not callable(set_clip) or getattr(self.optimizer, "flat_master_grad", None) is None:
            raise TypeError("clip_local_shards_on_device needs MasterWeightsOptimizer over FusedAdamW as the shards' optimizer")
        sq = global_grad_sq_norm(self.optimizer)
        if sq is None:
            raise ValueError("no gradients to clip")
        if self.world_size > 1:
            self._all_reduce_sum(sq)
        set_clip(sq, float(max_norm))
        return sq

    # ---- POST_STEP: zero1.py:236-260 --------------------------------------------------------------------------
    def gather_updated_params(self) -> None:
        """Updated shards back into the flat data buffer (the model's parameters are views of it); grads zeroed."""
        assert self.data_buffer is not None
        if self.grad_buffer is not None:
            self.grad_buffer.zero_()
        with torch.no_grad():
            for bucket in self.buckets:
                local = bucket.local_param.detach().contiguous()
                if self.world_size == 1:
                    self.data_buffer[bucket.start:bucket.end].copy_(local)
                else:
                    self._all_gather(self.data_buffer[bucket.start:bucket.end], local)

    # ---- POST_LOAD: zero1.py:283-287 --------------------------------------------------------------------------
    def sync_local_params_from_data_buffer(self) -> None:
        assert self.data_buffer is not None
        with torch.no_grad():
            for bucket in self.buckets:
                bucket.local_param.data.copy_(self.data_buffer[bucket.shard_start:bucket.shard_end])
        resync = getattr(self.optimizer, "sync_master_params_from_model", None)
        if callable(resync):
            resync()

    # ---- the phases of one optimizer step in the reference's order --------------------------------------------
    def step(self, max_norm: float | None = None, *, clip_on_device: bool = False) -> "float | torch.Tensor | None":
        """Returns the gradient norm as the reference's metadata has it (a host float), or with `clip_on_device` the
        device scalar sum of squares, which nobody has to wait for."""
        self.reduce_grads()
        norm = self.clip_local_shards_on_device(max_norm) if clip_on_device and max_norm is not None else self.clip_local_shards(max_norm)
        assert self.optimizer is not None
        self.optimizer.step()
        self.gather_updated_params()
        return norm


def _sq_norm_f64(grad: torch.Tensor) -> torch.Tensor:
    """sum g^2 in fp64: the fused kernel for fp32 device buffers, torch's own arithmetic otherwise."""
    if grad.is_cuda and grad.dtype == torch.float32 and grad.is_contiguous():
        from . import ops
        return ops.sq_norm(grad.view(-1))
    return grad.detach().double().pow(2).sum()
