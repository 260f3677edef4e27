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


class AutogradEngine:
    """``backward(model=, loss=, cache=)`` clears the gradients, runs ``loss.backward()`` and returns the
    named gradients; the cache is not read."""

    name = "autograd"

    def backward(self, *, model: nn.Module, loss: torch.Tensor, cache: Any | None = None) -> ADResult:
        model.zero_grad(set_to_none=True)
        loss.backward()
        return ADResult(grad_map=collect_named_grads(model))


def autograd_backward_step(model: nn.Module, *, ce_loss: torch.Tensor) -> GradMap:
    return AutogradEngine().backward(model=model, loss=ce_loss).grad_map


__all__ = ["AutogradEngine", "autograd_backward_step"]
