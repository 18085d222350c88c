"""One rank's side of the reference's ZeRO-2 buffers: gradients live in per-bucket buffers and are reduced bucket by
bucket while the backward pass is still running.

Mirror of `Zero2Plugin` (runtime/plugins/zero2.py:22-44, 107-176 buffers and buckets, 178-190 and 222-251 the two
hooks, 253-289 the reduction, 345-395 wait / reset) on top of the ZeRO-1 layout of this package (same data buffer, same
buckets, same local shards, same clipping, optimizer step and gather):

  * no gradient buffer of the whole model: every bucket has, per micro-batch of a pipeline schedule (`microbatches`,
    1 without pipelining), an exec state with a `grad_buffer` of the bucket's padded length and a `shard_buffer` of this
    rank's share of it;
  * a tensor hook on every parameter binds the `.grad` of all parameters of its bucket to views of the current exec
    state's `grad_buffer` when the first gradient of the bucket arrives, so autograd accumulates straight into it;
  * a post-accumulate hook counts the bucket's parameters down; the last one fires the bucket's reduction: this rank's
    slice of the mean gradient into `shard_buffer` (world size 1: the local copy the reference makes, zero2.py:258-261);
  * after the backward pass `wait_grad_sync` fires what has not fired (buckets with parameters that took no part) and adds
    every `shard_buffer` into `local_param.grad`, which therefore sums over the micro-steps of an accumulation window.

As in the ZeRO-1 mirror, what moves data between ranks is a seam (`reduce_scatter_avg`, `all_gather`, `all_reduce_sum`
callables); everything here runs on one GPU.

A backward function that adds its gradient into `param.grad` itself and returns None for the parameter
(HipLinear.accumulate_into_grad) still counts: autograd runs the parameter's accumulation node with no gradient, once
every contribution to the parameter is done, and the post-accumulate hook fires there as for any other parameter.  A
replayed HIP graph runs no autograd at all: no bucket fires during the replay, and `wait_grad_sync` reduces them all.
"""
from __future__ import annotations

from dataclasses import dataclass
from functools import partial
from typing import Callable

import torch
import torch.nn as nn

from .zero1 import AllGather, AllReduceSum, Bucket, ReduceScatter, Zero1FlatBuffers


@dataclass(eq=False)
class BucketExecState:
    """zero2.py:38-44; `fired` stands for the reference's pending `work` handle."""

    grad_buffer: torch.Tensor
    shard_buffer: torch.Tensor
    pending: int = 0
    fired: bool = False
    attached: bool = False


class Zero2FlatBuffers(Zero1FlatBuffers):
    whole_model_grad_buffer = False

    def __init__(self, model: nn.Module, *, optimizer_factory: Callable[[list[nn.Parameter]], torch.optim.Optimizer],
                 world_size: int = 1, rank: int = 0, bucket_mb_size: int = 25, microbatches: int = 1,
                 reduce_scatter_avg: ReduceScatter | None = None, all_gather: AllGather | None = None,
                 all_reduce_sum: AllReduceSum | None = None) -> None:
        if microbatches < 1:
            raise ValueError("microbatches must be >= 1")
        self.microbatches = microbatches
        self.microbatch_index = 0          # which exec state the running backward fills (the pipeline schedule sets it)
        self.fired_order: list[int] = []   # bucket indices in the order their reductions fired since the last reset
        self._hook_handles: list = []
        super().__init__(model, optimizer_factory=optimizer_factory, world_size=world_size, rank=rank,
                         bucket_mb_size=bucket_mb_size, reduce_scatter_avg=reduce_scatter_avg, all_gather=all_gather,
                         all_reduce_sum=all_reduce_sum)
        self._add_param_hooks()
        self.reset_buckets(grad_accum_start=True)

    # ---- zero2.py:107-176 ---------------------------------------------------------------------------------------
    def _prepare_buffers_and_buckets(self, model: nn.Module) -> None:
        super()._prepare_buffers_and_buckets(model)
        for bucket in self.buckets:
            dtype, device = bucket.local_param.dtype, bucket.local_param.device
            bucket.exec_states = [
                BucketExecState(grad_buffer=torch.zeros(bucket.end - bucket.start, dtype=dtype, device=device),
                                shard_buffer=torch.zeros(bucket.local_param.numel(), dtype=dtype, device=device))
                for _ in range(self.microbatches)]
            for param in bucket.params:
                param.grad = None   # bound to an exec state's buffer when the bucket's first gradient arrives

    # ---- zero2.py:178-190, 222-251 ------------------------------------------------------------------------------
    def _add_param_hooks(self) -> None:
        for bucket in self.buckets:
            for param in bucket.params:
                self._hook_handles.append(param.register_hook(partial(self._attach_hook, bucket)))
                self._hook_handles.append(param.register_post_accumulate_grad_hook(partial(self._grad_sync_hook, bucket)))

    def remove_hooks(self) -> None:
        for handle in self._hook_handles:
            handle.remove()
        self._hook_handles.clear()

    def _exec_state(self, bucket: Bucket) -> BucketExecState:
        return bucket.exec_states[0 if len(bucket.exec_states) == 1 else self.microbatch_index]

    def _attach_hook(self, bucket: Bucket, grad: "torch.Tensor | None") -> "torch.Tensor | None":
        state = self._exec_state(bucket)
        if not state.attached:
            self._attach_bucket_grad_buffer(bucket, state)
            state.attached = True
        return grad

    @staticmethod
    def _attach_bucket_grad_buffer(bucket: Bucket, state: BucketExecState) -> None:
        offset = 0
        for param in bucket.params:
            param.grad = state.grad_buffer[offset:offset + param.numel()].view_as(param)
            offset += param.numel()

    def _grad_sync_hook(self, bucket: Bucket, _param: torch.Tensor) -> None:
        state = self._exec_state(bucket)
        state.pending -= 1
        if state.pending == 0:
            self._fire(bucket, state)
            bucket.pending_exec_reductions -= 1

    # ---- zero2.py:253-289 ---------------------------------------------------------------------------------------
    def _fire(self, bucket: Bucket, state: BucketExecState) -> None:
        """This rank's slice of the bucket's mean gradient into the state's shard buffer."""
        if bucket.local_param.grad is None:
            bucket.local_param.grad = torch.zeros_like(bucket.local_param.data)
        full_grad = state.grad_buffer[:bucket.end - bucket.start]
        with torch.no_grad():
            if self.world_size == 1:
                state.shard_buffer.copy_(full_grad[:bucket.local_param.numel()])
            else:
                self._reduce_scatter_avg(state.shard_buffer, full_grad)
        state.fired = True
        self.fired_order.append(self.buckets.index(bucket))

    def _wait_state(self, bucket: Bucket, state: BucketExecState) -> None:
        """zero2.py:386-390: the reduced slice joins the shard's gradient."""
        with torch.no_grad():
            bucket.local_param.grad.add_(state.shard_buffer)
        state.fired = False

    # ---- POST_BACKWARD at a step boundary: zero2.py:345-355 -----------------------------------------------------
    def wait_grad_sync(self) -> None:
        for bucket in self.buckets:
            if not bucket.exec_states:
                raise RuntimeError("ZeRO2 bucket has no exec_states after backward")
            for state in bucket.exec_states:
                if not state.fired:     # parameters that took no part in this backward left the count above zero
                    self._fire(bucket, state)
                self._wait_state(bucket, state)
        mark = getattr(self.optimizer, "mark_grads_written", None)
        if callable(mark):
            mark()

    # ---- PRE_BACKWARD: zero2.py:357-381 -------------------------------------------------------------------------
    def reset_buckets(self, *, grad_accum_start: bool, backward_start: bool = True) -> None:
        if grad_accum_start:
            if self.optimizer is not None:
                self.optimizer.zero_grad(set_to_none=True)   # a master-weights optimizer forgets its fp32 gradients here
            for bucket in self.buckets:
                if bucket.local_param.grad is None:
                    bucket.local_param.grad = torch.zeros_like(bucket.local_param.data)
                else:
                    bucket.local_param.grad.zero_()
        if backward_start:
            self.fired_order.clear()
            for bucket in self.buckets:
                bucket.pending_exec_reductions = len(bucket.exec_states)
        for bucket in self.buckets:
            state = self._exec_state(bucket)
            if state.fired:   # the previous micro-step's reduction of this state is taken in before its buffers are cleared
                self._wait_state(bucket, state)
            state.grad_buffer.zero_()
            state.shard_buffer.zero_()
            state.pending = len(bucket.params)
            state.attached = False
            if self.microbatches > 1 and any(p.grad is not None for p in bucket.params):
                # a backward function that adds into an existing `.grad` (HipLinear.accumulate_into_grad) does so before
                # any hook of the parameter runs: it must find this micro-batch's buffer bound, not the one before
                self._attach_bucket_grad_buffer(bucket, state)
                state.attached = True

    # ---- the ZeRO-1 names of the same phases, so that a training loop can take either layout ---------------------
    def reset_grads(self) -> None:
        self.reset_buckets(grad_accum_start=True)

    def reduce_grads(self) -> None:
        self.wait_grad_sync()
