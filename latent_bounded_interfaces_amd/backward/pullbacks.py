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

    def __init__(self, *, basis_chunk: int = 0) -> None:
        # directions pulled back per call; 0 = all d at once
        if int(basis_chunk) < 0:
            raise ValueError("basis_chunk must be >= 0.")
        self.basis_chunk = int(basis_chunk)

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
                g_region_input = model.region_backend.input_pullback_basis(
                    cache=region_cache.backend_cache, output_cotangent_basis=update["g_region_output"])
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


def build_interface_pullback_provider(mode: str, *, basis_chunk: int = 0) -> StructuredInterfacePullbackProvider:
    """Name lookup in the style of reference backward/pullbacks.py:185-197; the autograd
    providers of the reference stay in the reference."""
    normalized = str(mode).strip().lower().replace("-", "_")
    if normalized in {"structured", "hip", "structured_hip"}:
        return StructuredInterfacePullbackProvider(basis_chunk=basis_chunk)
    raise ValueError("interface pullback provider must be one of: structured, hip")
