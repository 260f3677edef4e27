"""Backward-engine side callers of the HIP kernels (counterpart of reference backward/)."""
from .base import (
    ADEngine,
    ADResult,
    GradMap,
    LBIBackwardResult,
    ScanBackpropModel,
    assign_grad_map,
    collect_named_grads,
    store_named_grads,
)
from .local_vjp import TorchAutogradLocalVJPProvider
from .pullbacks import (
    StructuredInterfacePullbackProvider,
    TorchGraphInterfacePullbackProvider,
    TorchRecomputeInterfacePullbackProvider,
    build_interface_pullback_provider,
)
from .reference_scan import ReferenceScanEngine, ScanADEngine, lbi_reference_scan_backward_step, lbi_scan_backward_step
from .suffix_scan import (
    apply_jacobian_t,
    compose_suffix_jacobian_t,
    interface_state_jacobian_t_stats,
    propagate_state_adjoint_by_autograd_chain,
    propagate_state_adjoint_from_last_region_input,
    propagate_state_adjoint_with_jacobian_scan,
)

__all__ = [
    "ADEngine",
    "ADResult",
    "GradMap",
    "LBIBackwardResult",
    "ReferenceScanEngine",
    "ScanADEngine",
    "ScanBackpropModel",
    "StructuredInterfacePullbackProvider",
    "TorchAutogradLocalVJPProvider",
    "TorchGraphInterfacePullbackProvider",
    "TorchRecomputeInterfacePullbackProvider",
    "apply_jacobian_t",
    "assign_grad_map",
    "build_interface_pullback_provider",
    "collect_named_grads",
    "compose_suffix_jacobian_t",
    "interface_state_jacobian_t_stats",
    "lbi_reference_scan_backward_step",
    "lbi_scan_backward_step",
    "propagate_state_adjoint_by_autograd_chain",
    "propagate_state_adjoint_from_last_region_input",
    "propagate_state_adjoint_with_jacobian_scan",
    "store_named_grads",
]
