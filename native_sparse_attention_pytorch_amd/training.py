"""Mixed-precision training of a bf16 model against fp32 master weights.

Under `torch.autocast` every projection of every layer casts its fp32 weight, bias and input to bf16 on the way in and
its gradients back on the way out: at the size of the reference's training script (train.py:22-50: dim 512, depth 6,
1024 tokens) that is ~270 of a step's ~940 kernel launches, and the step is bound by its launches, not by the GPU.
Here the model itself is bf16 (no casts inside the step) and the optimizer works on fp32 copies of its parameters:
one multi-tensor copy takes the bf16 gradients to the masters, one takes the updated masters back.  The arithmetic is
the same as under autocast - bf16 operands rounded from fp32 masters, fp32 accumulation, fp32 update - and the loss
curve agrees with the fp32 oracle as closely.
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
