"""Dense backward through the whole forward graph: the path the scan step is checked against.

Module and names of reference backward/autograd.py:11-28 (the reference's training loop imports
``AutogradEngine`` from the package for its dense runs, train/runners.py).  Plain ``loss.backward()``; no
kernel of this package is involved.
"""
from __future__ import annotations

from typing import Any

import torch
from torch import nn

from .base import ADResult, GradMap, collect_named_grads


def autograd_backward_step(model: nn.Module, *, ce_loss: torch.Tensor) -> GradMap:
    """Named gradients of every trainable parameter from one dense backward of ``ce_loss``; gradients left on
    the parameters from an earlier step are dropped first."""
    for param in model.parameters():
        param.grad = None
    ce_loss.backward()
    return collect_named_grads(model)


class AutogradEngine:
    """The dense step behind the engine interface (``backward(model=, loss=, cache=)``); the cache is not read."""

    name = "autograd"

    def backward(self, *, model: nn.Module, loss: torch.Tensor, cache: Any | None = None) -> ADResult:
        return ADResult(grad_map=autograd_backward_step(model, ce_loss=loss))


__all__ = ["AutogradEngine", "autograd_backward_step"]
