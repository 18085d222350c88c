"""Forward + backward of a model recorded once into a HIP graph and replayed per step.

A LLaMA-50M step is some six hundred kernel launches of ten to twenty microseconds each, so the eager step is bound
by the host's launch rate rather than by the GPU.  Recording `loss = model(batch); loss.backward()` into one graph
removes that bound: a step becomes a copy of the batch into the static input tensors, one graph launch, and the
(eager, few-launch) clip + optimizer step + gradient clear that follow.

Requirements, checked where they can be:
  * every tensor of the batch keeps its shape, dtype and device from step to step;
  * the parameters' `.grad` tensors exist before recording and keep their storage (the flat layouts of
    `MasterWeightsOptimizer(flat=True)` and `Zero1FlatBuffers` do: their `zero_grad` / `reset_grads` clear in place),
    so the recorded in-place accumulation lands in the memory the optimizer reads;
  * nothing in the forward or backward depends on host-side reads of device data.

What stays outside the graph, on purpose:
  * the token embedding and its gradient.  torch's embedding gradient for more than a few thousand indices sorts them
    with library routines whose temporary storage does not survive into a replay (the replayed kernel faults), so the
    lookup runs eagerly in front of the graph, the graph starts from a static copy of the hidden states, and the
    embedding's backward runs eagerly behind it on the gradient the graph left for those hidden states;
  * the optimizer step: its bias corrections and learning rate are host scalars that change every step.
"""
from __future__ import annotations

from typing import Callable, Mapping

import torch


class CapturedForwardBackward:
    """`step = CapturedForwardBackward(model, example_batch, embed=model.embed_tokens); loss = step(batch)`.

    `embed` maps `batch[input_key]` to hidden states; the model is then called with `hidden_key` in place of
    `input_key` (LlamaForCausalLM accepts that form).  `loss` is a static tensor overwritten by every replay; read or
    clone it before the next call.  Gradients are accumulated into the existing `.grad` tensors exactly as the eager
    `loss.backward()` would.
    """

    def __init__(self, model: torch.nn.Module, example_batch: Mapping[str, torch.Tensor], *,
                 embed: Callable[[torch.Tensor], torch.Tensor] | None = None, input_key: str = "input_ids",
                 hidden_key: str = "hidden_states", warmup: int = 2, clear_grads: Callable[[], None] | None = None) -> None:
        params = [p for p in model.parameters() if p.requires_grad]
        if not params or not all(p.is_cuda for p in params):
            raise RuntimeError("CapturedForwardBackward needs a model on the GPU")
        missing = [n for n, p in model.named_parameters() if p.requires_grad and p.grad is None]
        if missing:
            raise RuntimeError("parameters without a bound .grad cannot be recorded (their gradient would be allocated "
                               f"inside the graph's private pool): {missing[:4]}")
        if embed is None and any(isinstance(m, torch.nn.Embedding) and m.weight.requires_grad for m in model.modules()):
            raise RuntimeError("the model has a trainable nn.Embedding: pass embed=<that module> so that its lookup and "
                               "gradient run outside the graph (torch's embedding gradient is not safe to replay)")
        self._model, self._embed, self._input_key = model, embed, input_key
        self._params = params
        self._grad_ptrs = [p.grad.data_ptr() for p in params]
        self._static = {k: v.clone() for k, v in example_batch.items() if embed is None or k != input_key}
        self._hidden = None
        if embed is not None:
            with torch.no_grad():
                self._hidden = embed(example_batch[input_key]).clone().requires_grad_(True)
            self._hidden.grad = torch.zeros_like(self._hidden)
            self._static[hidden_key] = self._hidden
        clear = clear_grads or (lambda: [p.grad.zero_() for p in params])

        def forward_backward() -> torch.Tensor:
            if self._hidden is not None:
                self._hidden.grad.zero_()      # a fill kernel, recorded as the graph's first node
            loss = model(self._static)
            loss.backward()
            return loss

        from .optim import grad_write_listener, notify_grad_written
        self._notify_grad_written = notify_grad_written
        # warm-up on a side stream (workspaces, lazily created module state, library handles), then record on the SAME
        # stream: autograd ties each parameter's gradient accumulator to the stream of the forward pass that created it
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(max(1, warmup)):
                forward_backward()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self._check_grads_in_place()
        self.graph = torch.cuda.CUDAGraph()
        # the parameters whose gradient the recorded backward writes: reported again after every replay, for optimizers
        # that skip parameters without a gradient (a replay runs no Python, so nobody else would tell them)
        with grad_write_listener() as seen, torch.cuda.graph(self.graph, stream=side):
            # detached: nobody differentiates through the static loss, and an autograd graph kept alive here would tie
            # the parameters' gradient accumulators to the recording stream for later eager passes
            self.loss = forward_backward().detach()
        self._written = list({id(p): p for p in seen}.values())
        self._check_grads_in_place()
        clear()            # the warm-up passes ran for real; recording itself executes nothing

    def _check_grads_in_place(self) -> None:
        for p, ptr in zip(self._params, self._grad_ptrs):
            if p.grad is None or p.grad.data_ptr() != ptr:
                raise RuntimeError("a parameter's .grad was re-allocated during warm-up or recording; bind gradients "
                                   "to persistent buffers (flat layout) before capturing")

    def __call__(self, batch: Mapping[str, torch.Tensor]) -> torch.Tensor:
        hidden = None
        if self._embed is not None:
            hidden = self._embed(batch[self._input_key])
            if hidden.shape != self._hidden.shape or hidden.dtype != self._hidden.dtype:
                raise ValueError(f"embedded batch is {tuple(hidden.shape)} {hidden.dtype}, recorded "
                                 f"{tuple(self._hidden.shape)} {self._hidden.dtype}")
            with torch.no_grad():
                self._hidden.copy_(hidden)
        for key, dst in self._static.items():
            if dst is self._hidden:
                continue
            if key not in batch:
                raise ValueError(f"batch lacks the recorded key {key!r}")
            src = batch[key]
            if src.shape != dst.shape or src.dtype != dst.dtype:
                raise ValueError(f"batch[{key!r}] is {tuple(src.shape)} {src.dtype}, recorded {tuple(dst.shape)} {dst.dtype}")
            if src.data_ptr() != dst.data_ptr():
                dst.copy_(src, non_blocking=True)
        self._check_grads_in_place()
        self.graph.replay()
        for p in self._written:
            self._notify_grad_written(p)
        if hidden is not None and hidden.requires_grad:
            hidden.backward(self._hidden.grad)      # eager: the embedding's own gradient
        return self.loss
