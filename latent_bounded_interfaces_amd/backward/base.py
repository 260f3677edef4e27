"""Result records and gradient-map helpers of the backward engines.

Same names, fields and behaviour as reference backward/base.py:10-90 so that code written
against the reference's ``backward`` package finds them here: ``ADResult``,
``LBIBackwardResult``, the structural model protocol ``ScanBackpropModel`` and the three
helpers that move gradients between ``param.grad`` and a ``{name: grad}`` map.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Protocol, runtime_checkable

import torch
from torch import nn

GradMap = dict  # {parameter name: gradient tensor or None}


@dataclass
class ADResult:
    """What an engine's ``backward`` returns (reference backward/base.py:13-16)."""

    grad_map: GradMap
    diagnostics: dict[str, Any] = field(default_factory=dict)


@dataclass
class LBIBackwardResult:
    """What the scan backward step returns (reference backward/base.py:19-23)."""

    grad_map: GradMap
    interface_scan_rms: float
    interface_jacobian_stats: dict[str, float] | None = None


@runtime_checkable
class ScanBackpropModel(Protocol):
    """Members the scan engines use on a model (reference backward/base.py:27-49)."""

    num_regions: int
    region_ranges: list
    interface: Any
    region_backend: Any

    def named_parameters(self, *args: Any, **kwargs: Any) -> Any: ...

    def zero_grad(self, *args: Any, **kwargs: Any) -> None: ...

    def output_head_vjp_parameters(self) -> list: ...

    def canvas_vjp_parameters(self) -> list: ...

    def shared_local_vjp_parameters(self) -> list: ...


class ADEngine(Protocol):
    """An engine turns a loss (and a forward cache) into a gradient map (reference backward/base.py:52-62)."""

    name: str

    def backward(self, *, model: nn.Module, loss: torch.Tensor, cache: Any | None = None) -> ADResult: ...


def _trainable(model: nn.Module):
    return ((name, p) for name, p in model.named_parameters() if p.requires_grad)


def collect_named_grads(model: nn.Module) -> GradMap:
    """Detached copies of every trainable parameter's ``.grad`` (``None`` where unset)."""
    return {name: (None if p.grad is None else p.grad.detach().clone()) for name, p in _trainable(model)}


def assign_grad_map(model: nn.Module, grad_map: GradMap) -> None:
    """Writes a gradient map into ``param.grad``; names missing from the map clear the gradient."""
    for name, p in _trainable(model):
        grad = grad_map.get(name)
        p.grad = None if grad is None else grad.detach().clone()


def store_named_grads(grad_map: GradMap, param_name_map: dict[int, str], params, grads) -> None:
    """Files ``grads`` (as ``torch.autograd.grad`` returns them for ``params``) under the parameters' names."""
    for p, grad in zip(params, grads):
        grad_map[param_name_map[id(p)]] = None if grad is None else grad.detach().clone()


__all__ = [
    "ADEngine",
    "ADResult",
    "GradMap",
    "LBIBackwardResult",
    "ScanBackpropModel",
    "assign_grad_map",
    "collect_named_grads",
    "store_named_grads",
]
