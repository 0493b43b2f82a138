"""Mixed-precision training of a bf16 model against fp32 master weights.

Under `torch.autocast` every projection of every layer casts its fp32 weight, bias and input to bf16 on the way in and
its gradients back on the way out: at the size of the reference's training script (train.py:22-50: dim 512, depth 6,
1024 tokens) that is ~270 of a step's ~940 kernel launches, and the step is bound by its launches, not by the GPU.
Here the model itself is bf16 (no casts inside the step) and the optimizer works on fp32 copies of its parameters:
one multi-tensor copy takes the bf16 gradients to the masters, one takes the updated masters back.  The arithmetic is
the same as under autocast - bf16 operands rounded from fp32 masters, fp32 accumulation, fp32 update - and the loss
curve agrees with the fp32 oracle as closely.

`GraphedStep` goes one further for fixed shapes: the forward and backward of the bf16 model are recorded once into a HIP
graph and replayed per step (one launch instead of ~700); the optimizer stays outside the graph.
"""
from __future__ import annotations

import torch
from torch import nn


class Fp32Masters:
    """`model` (its parameters still fp32, freshly initialised or loaded) is cast to bf16 in place; `self.masters` are the
    fp32 originals, to be handed to any torch optimizer.  Per step: `loss.backward()`, then `step(optimizer)`."""

    def __init__(self, model: nn.Module):
        self.masters = [p.detach().clone().float() for p in model.parameters()]
        model.bfloat16()
        self.params = list(model.parameters())
        for m in self.masters:
            m.requires_grad_(True)

    @torch.no_grad()
    def step(self, optimizer: torch.optim.Optimizer) -> None:
        live = [(m, p) for m, p in zip(self.masters, self.params) if p.grad is not None]
        for m, p in zip(self.masters, self.params):
            if p.grad is None:
                m.grad = None               # no gradient this step: the optimizer skips it
            elif m.grad is None:
                m.grad = torch.empty_like(m)
        torch._foreach_copy_([m.grad for m, _ in live], [p.grad for _, p in live])
        optimizer.step()
        torch._foreach_copy_(self.params, self.masters)
        for p in self.params:
            p.grad = None


class GraphedStep:
    """Forward + backward of `model(ids, return_loss=True)` (or of `loss_fn(model, ids)`) as one replayed HIP graph, for a
    bf16 model (e.g. under `Fp32Masters`) and inputs of one fixed shape.

        step = GraphedStep(model, example_ids)
        loss = step(ids)            # gradients are in p.grad of the model's parameters afterwards
        masters.step(optimizer)     # or optimizer.step() on the model's own parameters

    The graph holds no memset node of a library reduction (their replays gave wrong bias gradients on this platform):
    while it is recorded every bias gradient is a column sum by this library's kernel (ops.colsum_supported) and the
    feed-forward projections go through ops.linear (Transformer._feed_forward).  The gradient tensors are the graph's own:
    every call re-attaches them to the parameters (an optimizer helper may have set `p.grad = None`) and every replay
    overwrites them, so gradients do not accumulate across calls.  `loss` is a tensor that the next call overwrites.
    Create it before the model's first normally launched training step (a `Transformer` that has been stepped is refused:
    recording one ended the process here); replays and launched steps may be mixed freely afterwards."""

    def __init__(self, model: nn.Module, example_ids: torch.Tensor, warmup: int = 3, loss_fn=None):
        # loss_fn(model, ids) -> scalar loss; default: the Transformer's own `model(ids, return_loss=True)`
        self.loss_fn = loss_fn if loss_fn is not None else (lambda m, ids: m(ids, return_loss=True))
        if not example_ids.is_cuda:
            raise RuntimeError("GraphedStep needs device tensors")
        if torch.is_autocast_enabled() or any(p.requires_grad and p.is_floating_point() and p.dtype != torch.bfloat16 for p in model.parameters()):
            # under autocast / with fp32 parameters the projections run through the library's own autograd, whose bias
            # gradients are the sums that replay wrongly
            raise RuntimeError("GraphedStep records a bf16 model outside autocast (cast it with Fp32Masters or .bfloat16())")
        if getattr(model, "_launched_grad_steps", False):
            # recording after normally launched training steps of the same model ended the process (segmentation fault inside
            # the recording) on this platform, with backward() and with autograd.grad() alike; a model that has not been
            # stepped yet records and replays correctly, also next to other models trained in the same process
            raise RuntimeError("GraphedStep must be created before the model's first normally launched training step "
                               "(build the model, then GraphedStep, then train through it)")
        self.model = model
        self.params = [p for p in model.parameters()]
        self.ids = example_ids.clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        # torch.autograd.grad, not backward(): the gradients come back as the recording's own tensors instead of passing
        # through the parameters' gradient accumulator nodes (which belong to the stream that created them)
        wanted = [p for p in self.params if p.requires_grad]
        model._recording_warmup = True
        try:
            with torch.cuda.stream(side):                # allocator and library warm-up outside the recording
                for _ in range(max(1, warmup)):
                    torch.autograd.grad(self.loss_fn(model, self.ids), wanted, allow_unused=True)
        finally:
            model._recording_warmup = False
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            loss = self.loss_fn(model, self.ids)
            grads = torch.autograd.grad(loss, wanted, allow_unused=True)
            self.loss = loss.detach()
        by_param = dict(zip(map(id, wanted), grads))
        self.grads = [by_param.get(id(p)) for p in self.params]

    def __call__(self, ids: torch.Tensor) -> torch.Tensor:
        if ids.shape != self.ids.shape or ids.dtype != self.ids.dtype:
            raise RuntimeError(f"GraphedStep was recorded for ids of shape {tuple(self.ids.shape)}, got {tuple(ids.shape)}")
        for p, g in zip(self.params, self.grads):
            p.grad = g
        self.ids.copy_(ids)
        self.graph.replay()
        return self.loss
