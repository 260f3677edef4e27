"""Structural contracts between this package and the program it plugs into.

Nothing here is a base class: the reference program keeps its own protocol and cache types
(backward/pullbacks.py:9-18, backward/local_vjp.py:10-63, backward/base.py:13-62,
backends/base.py:10-50, backends/transformer.py:17-85) and this package is duck-typed on their
attribute names.  The protocols below say, in checkable form, which of those names are used:

* what this package OFFERS: ``HipTransformerLowering`` is a ``TransformerLowering``,
  ``StructuredInterfacePullbackProvider`` is an ``InterfacePullbackProvider``;
* what it NEEDS from the caller: the methods ``lbi_scan_backward_step`` calls on the local-VJP
  provider, and the cache fields the region pullback reads.

``isinstance`` against these protocols checks the presence of the members only
(``typing.runtime_checkable``), which is all duck typing asks for.
"""
from __future__ import annotations

from typing import Any, Protocol, runtime_checkable

import torch


@runtime_checkable
class InterfacePullbackProvider(Protocol):
    """Builds the K transposed state Jacobians ``Jt_r [B, d, d]`` the suffix scan composes
    (``g_in = Jt @ g_out``; reference backward/pullbacks.py:9-18, convention :53-64)."""

    name: str

    def materialize_state_jacobian_t(self, *, model: Any, cache: dict[str, Any]) -> list[torch.Tensor]: ...


@runtime_checkable
class TransformerLowering(Protocol):
    """Region derivative contracts of the Transformer backend (reference backends/transformer.py:64-85),
    plus the attention-level entry of its CUDA lowering (backends/transformer_cuda.py:23-43)."""

    name: str

    def attention_input_pullback_basis(self, *, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                                       output_cotangent_basis: torch.Tensor, softmax_scale: float,
                                       causal: bool = True, kernel_mode: str = "fa2_mma_pblock4"
                                       ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]: ...

    def input_pullback_basis(self, *, backend: Any, cache: Any, output_cotangent_basis: torch.Tensor
                             ) -> torch.Tensor: ...

    def parameter_vjp(self, *, backend: Any, cache: Any, output_cotangent: torch.Tensor
                      ) -> dict[str, torch.Tensor]: ...


@runtime_checkable
class LocalVJPProvider(Protocol):
    """The calls ``lbi_scan_backward_step`` makes, in this order (reference backward/local_vjp.py:10-63,
    call sites backward/scan.py:29-96)."""

    def new_grad_map(self, model: Any) -> dict: ...

    def store_output_head_grads(self, *, model: Any, loss: torch.Tensor, grad_map: dict) -> None: ...

    def state_adjoint_from_loss(self, *, loss: torch.Tensor, state: torch.Tensor) -> torch.Tensor: ...

    def store_initial_interface_grads(self, *, model: Any, state0: torch.Tensor, state0_adjoint: torch.Tensor,
                                      grad_map: dict) -> None: ...

    def store_region_grads(self, *, model: Any, loss: torch.Tensor, states: list, region_index: int,
                           num_regions: int, state_adjoints: list, grad_map: dict) -> None: ...

    def store_shared_canvas_grads(self, *, model: Any, loss: torch.Tensor, grad_map: dict) -> None: ...


# Fields of the reference's forward caches that the region pullback and the parameter VJP read
# (reference backends/transformer.py:17-61, backends/base.py:10-13).  Everything else in those
# dataclasses is ignored, so a caller may leave it unset.
ATTENTION_CACHE_FIELDS = ("norm_input", "norm_output", "q_rope", "k_expanded", "v_expanded", "out_proj_input")
MLP_CACHE_FIELDS = ("norm_input", "norm_output", "fc1_output", "down_input")
LAYER_CACHE_FIELDS = ("layer_index", "attention", "mlp")
REGION_CACHE_FIELDS = ("layer_range", "layer_caches", "region_input")

__all__ = [
    "ATTENTION_CACHE_FIELDS",
    "InterfacePullbackProvider",
    "LAYER_CACHE_FIELDS",
    "LocalVJPProvider",
    "MLP_CACHE_FIELDS",
    "REGION_CACHE_FIELDS",
    "TransformerLowering",
]
