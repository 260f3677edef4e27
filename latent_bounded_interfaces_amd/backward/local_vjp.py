"""Region-local parameter VJPs on the forward graph.

``TorchAutogradLocalVJPProvider`` is the provider the reference's scan step falls back to when
the caller passes none (reference backward/scan.py:28; class backward/local_vjp.py:66-185): every
gradient is one ``torch.autograd.grad`` call whose seed is either the loss or a state adjoint the
scan produced, so no gradient ever crosses a region boundary through the graph.  It holds no
kernel of its own; it is here so that the engine entries keep the reference's defaults.
"""
from __future__ import annotations

from typing import Any

import torch

from .base import GradMap, store_named_grads


class TorchAutogradLocalVJPProvider:
    """Local VJPs by ``torch.autograd.grad``; same method names and keywords as the reference's."""

    name = "torch_autograd"

    @staticmethod
    def _names(model: Any) -> dict[int, str]:
        return {id(p): n for n, p in model.named_parameters() if p.requires_grad}

    def new_grad_map(self, model: Any) -> GradMap:
        return {n: None for n, p in model.named_parameters() if p.requires_grad}

    def _grads_into(self, model: Any, grad_map: GradMap, params: list, target: torch.Tensor,
                    seed: torch.Tensor | None, retain: bool = True) -> None:
        if not params:
            return
        grads = torch.autograd.grad(target, params, grad_outputs=seed, retain_graph=retain, create_graph=False,
                                    allow_unused=True)
        store_named_grads(grad_map, self._names(model), params, grads)

    def store_output_head_grads(self, *, model: Any, loss: torch.Tensor, grad_map: GradMap) -> None:
        self._grads_into(model, grad_map, list(model.output_head_vjp_parameters()), loss, None)

    def state_adjoint_from_loss(self, *, loss: torch.Tensor, state: torch.Tensor) -> torch.Tensor:
        (g,) = torch.autograd.grad(loss, state, retain_graph=True, create_graph=False, allow_unused=False)
        return g.detach().to(device=state.device, dtype=state.dtype)

    def store_initial_interface_grads(self, *, model: Any, state0: torch.Tensor, state0_adjoint: torch.Tensor,
                                      grad_map: GradMap) -> None:
        seed = state0_adjoint.to(device=state0.device, dtype=state0.dtype)
        self._grads_into(model, grad_map, list(model.interface.initial_vjp_parameters()), state0, seed)

    def store_region_grads(self, *, model: Any, loss: torch.Tensor, states: list, region_index: int, num_regions: int,
                           state_adjoints: list, grad_map: GradMap) -> None:
        params = [*model.region_backend.parameters_for_region(region_index),
                  *model.interface.region_vjp_parameters(region_index)]
        if region_index < num_regions - 1:
            # parameters of region r reach the loss only through its output state s_{r+1}
            target = states[region_index + 1]
            seed = state_adjoints[region_index + 1].to(device=target.device, dtype=target.dtype)
            self._grads_into(model, grad_map, params, target, seed)
        else:
            # the last region feeds the readout directly (its output state is never used)
            self._grads_into(model, grad_map, params, loss, None)

    def store_shared_canvas_grads(self, *, model: Any, loss: torch.Tensor, grad_map: GradMap) -> None:
        # last use of the graph in a step: it is released here, as the reference does (:176-184)
        self._grads_into(model, grad_map, list(model.shared_local_vjp_parameters()), loss, None, retain=False)


__all__ = ["TorchAutogradLocalVJPProvider"]
