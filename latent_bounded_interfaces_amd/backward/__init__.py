"""Backward-engine side callers of the HIP kernels (counterpart of reference backward/)."""
from .pullbacks import StructuredInterfacePullbackProvider, build_interface_pullback_provider
from .scan import LBIBackwardResult, lbi_scan_backward_step
from .suffix_scan import (
    apply_jacobian_t,
    compose_suffix_jacobian_t,
    interface_state_jacobian_t_stats,
    propagate_state_adjoint_from_last_region_input,
    propagate_state_adjoint_with_jacobian_scan,
)

__all__ = [
    "LBIBackwardResult",
    "StructuredInterfacePullbackProvider",
    "apply_jacobian_t",
    "build_interface_pullback_provider",
    "compose_suffix_jacobian_t",
    "interface_state_jacobian_t_stats",
    "lbi_scan_backward_step",
    "propagate_state_adjoint_from_last_region_input",
    "propagate_state_adjoint_with_jacobian_scan",
]
