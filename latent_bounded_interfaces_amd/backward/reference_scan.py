"""Scan backward step configured by mode name.

Counterpart of reference backward/reference_scan.py:12-34 (same name, keywords and defaults,
and the same re-exports): builds the interface-pullback provider from ``state_jacobian_mode``
and runs ``lbi_scan_backward_step`` with the default local-VJP provider.  Besides the
reference's ``graph`` / ``recompute`` modes, ``structured`` selects the provider whose region
pullback runs on the HIP kernels.
"""
from __future__ import annotations

from typing import Any

import torch

from .base import LBIBackwardResult
from .pullbacks import build_interface_pullback_provider
from .scan import ReferenceScanEngine, ScanADEngine, lbi_scan_backward_step


def lbi_reference_scan_backward_step(
    model: Any,
    *,
    ce_loss: torch.Tensor,
    cache: dict[str, Any],
    state_jacobian_mode: str = "graph",
    state_jacobian_basis_chunk: int = 1,
    compute_interface_jacobian_stats: bool = False,
    include_interface_jacobian_suffix: bool = False,
) -> LBIBackwardResult:
    """Run exact LBI scan backprop with a configured interface-pullback provider."""
    provider = build_interface_pullback_provider(state_jacobian_mode, basis_chunk=state_jacobian_basis_chunk)
    return lbi_scan_backward_step(
        model,
        ce_loss=ce_loss,
        cache=cache,
        pullback_provider=provider,
        compute_interface_jacobian_stats=compute_interface_jacobian_stats,
        include_interface_jacobian_suffix=include_interface_jacobian_suffix,
    )


__all__ = ["ReferenceScanEngine", "ScanADEngine", "lbi_reference_scan_backward_step", "lbi_scan_backward_step"]
