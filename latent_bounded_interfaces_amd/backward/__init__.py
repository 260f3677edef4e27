"""Backward-engine side callers of the scan kernel (counterpart of reference backward/)."""
from .suffix_scan import (
    apply_jacobian_t,
    compose_suffix_jacobian_t,
    interface_state_jacobian_t_stats,
    propagate_state_adjoint_from_last_region_input,
    propagate_state_adjoint_with_jacobian_scan,
)

__all__ = [
    "apply_jacobian_t",
    "compose_suffix_jacobian_t",
    "interface_state_jacobian_t_stats",
    "propagate_state_adjoint_from_last_region_input",
    "propagate_state_adjoint_with_jacobian_scan",
]
