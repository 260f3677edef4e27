"""Interface state Jacobians built from structured pullbacks instead of autograd graphs.

An ``InterfacePullbackProvider`` (reference backward/pullbacks.py:9-18) hands the scan
one matrix per region, ``Jt[b, i, j] = d s_out[j] / d s_in[i]`` (reference
backward/pullbacks.py:53-64).  The reference's two providers obtain it from
``torch.autograd.grad`` (graph walk, or recompute of the region with the batch replicated
per basis direction, :37-146).  The provider here composes the three structured pieces the
reference's interfaces and backends already expose:

1. ``interface.apply_update_jacobian_t_to_region_output``  (interfaces/base.py:69-76;
   interfaces/vector_mlp.py:223-253): identity basis on ``s_out`` -> cotangents of the
   region output ``[B, P, T, D]`` and the skip term ``[B, P, d]``;
2. ``region_backend.input_pullback_basis``  (backends/transformer.py:248-258): region
   output cotangents -> region input cotangents, which with ``HipTransformerLowering``
   as the backend's lowering runs on the HIP kernels;
3. ``interface.apply_decode_jacobian_t_to_state_input``  (interfaces/base.py:78-85;
   interfaces/vector_mlp.py:255-270): region input cotangents -> ``[B, P, d]``;

and sums skip and decode terms, which is ``apply_region_transition_jacobian_t``
(interfaces/base.py:87-106).  The forward activations are those of the cache: no region is
run again.
"""
from __future__ import annotations

from typing import Any

import torch


class StructuredInterfacePullbackProvider:
    """Builds ``Jt`` per region from the interface's and the backend's structured pullbacks."""

    name = "structured"

    def __init__(self, *, basis_chunk: int = 0, position_constant_update: str = "verify_once") -> None:
        # directions pulled back per call; 0 = all d at once
        if int(basis_chunk) < 0:
            raise ValueError("basis_chunk must be >= 0.")
        if position_constant_update not in {"verify_once", "verify", "off"}:
            raise ValueError("position_constant_update must be one of: verify_once, verify, off")
        self.basis_chunk = int(basis_chunk)
        self.position_constant_update = position_constant_update
        self._constant_over_positions: dict[type, bool] = {}

    def _region_output_cotangent(self, interface: Any, g_region_output: torch.Tensor) -> torch.Tensor:
        """An interface that pools the region output with a mean over positions sends the same cotangent to
        every position (reference interfaces/vector_mlp.py:111-116 materialises it as a dense [B,P,T,D]
        tensor).  When that holds the tensor is handed on as a stride-0 view of its first position, which lets
        the region pullback run the last block's first product on one row per direction.  Whether it holds is
        a property of the interface class: it is checked on the device (one host synchronisation) the first
        time a class is seen (``verify_once``), on every call (``verify``), or never used (``off``)."""
        if self.position_constant_update == "off" or g_region_output.dim() != 4 or g_region_output.shape[2] <= 1:
            return g_region_output
        if g_region_output.stride(2) == 0:
            return g_region_output
        first = g_region_output[:, :, :1].expand_as(g_region_output)
        known = self._constant_over_positions.get(type(interface)) if self.position_constant_update == "verify_once" else None
        if known is None:
            known = bool(torch.equal(first, g_region_output))
            self._constant_over_positions[type(interface)] = known
        return first if known else g_region_output

    def region_state_jacobian_t(self, *, model: Any, region_cache: Any) -> torch.Tensor:
        state_in = region_cache.state_in
        if state_in.dim() != 2:
            raise ValueError("interface state inputs must be [B, R].")
        bsz, rank = state_in.shape
        chunk = self.basis_chunk or rank
        eye = torch.eye(rank, device=state_in.device, dtype=state_in.dtype)
        cols: list[torch.Tensor] = []
        with torch.no_grad():
            for start in range(0, rank, chunk):
                basis = eye[start:start + chunk].unsqueeze(0).expand(bsz, -1, rank)
                update = model.interface.apply_update_jacobian_t_to_region_output(
                    region_cache=region_cache, state_out_cotangent_basis=basis)
                g_region_output = self._region_output_cotangent(model.interface, update["g_region_output"])
                g_region_input = model.region_backend.input_pullback_basis(
                    cache=region_cache.backend_cache, output_cotangent_basis=g_region_output)
                decode = model.interface.apply_decode_jacobian_t_to_state_input(
                    region_cache=region_cache, region_input_cotangent_basis=g_region_input)
                total = update["g_state_skip"] + decode["g_state_input"]  # [B, P, d_in]
                cols.append(total.transpose(1, 2))                        # [B, d_in, P]
        return torch.cat(cols, dim=-1).to(device=state_in.device, dtype=state_in.dtype).contiguous()

    def materialize_state_jacobian_t(self, *, model: Any, cache: dict[str, Any]) -> list[torch.Tensor]:
        region_caches = cache["region_caches"]
        if len(region_caches) != model.num_regions:
            raise ValueError("cache has invalid region_caches length.")
        return [self.region_state_jacobian_t(model=model, region_cache=rc) for rc in region_caches]


def build_interface_pullback_provider(mode: str, *, basis_chunk: int = 0,
                                      position_constant_update: str = "verify_once") -> StructuredInterfacePullbackProvider:
    """Name lookup in the style of reference backward/pullbacks.py:185-197; the autograd
    providers of the reference stay in the reference."""
    normalized = str(mode).strip().lower().replace("-", "_")
    if normalized in {"structured", "hip", "structured_hip"}:
        return StructuredInterfacePullbackProvider(basis_chunk=basis_chunk,
                                                   position_constant_update=position_constant_update)
    raise ValueError("interface pullback provider must be one of: structured, hip")
