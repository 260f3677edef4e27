"""Exact scan backward step of an LBI model on the HIP scan kernels, and the engine around it.

Counterparts of ``lbi_scan_backward_step`` and ``ScanADEngine`` / ``ReferenceScanEngine``
(reference backward/scan.py:18-97, :100-171): same arguments, defaults, results and diagnostics
keys, same order of calls into the local-VJP provider, same edge cases (no region:
``RuntimeError``; one region: no Jacobian is built).  What differs is the middle:

* the state adjoints are every suffix matrix applied to the last cotangent in ONE launch
  (``lbi_suffix_apply``; the reference spends K mat-vec launches, backward/suffix_scan.py:49-53);
* the last region's state Jacobian, which the reference builds and then drops (its output state never reaches the
  loss), is not built when the provider can leave it out and the Jacobian statistics are off: one region pullback
  less per step;
* ``interface_scan_rms`` (logged by the reference's training loop as ``scan_align``) is reported
  on every step as the reference does (:63-72): the RMS difference between those adjoints and the
  sequential chain ``g_r = Jt_r g_{r+1}`` (the reference's ``g_manual``), which comes from a kernel of its
  own (``lbi_suffix_cotangents``: one pass over the matrices, no matrix product).  The two sides share no
  intermediate result whatever form the scan takes (one chain per column block, or chunks side by side),
  so the figure checks the scan and is tiny but not zero.  ``check_scan=False`` skips it (no suffix
  matrix is formed, no host synchronisation, 0.0 reported) for callers that do not log it.
"""
from __future__ import annotations

from typing import Any

import torch
from torch import nn

from ..hip.interface import suffix_apply, suffix_scan_cotangents, suffix_scan_pullbacks
from .base import ADResult, LBIBackwardResult, ScanBackpropModel, assign_grad_map
from .local_vjp import TorchAutogradLocalVJPProvider, build_local_vjp_provider
from .pullbacks import STRUCTURED_MODE_NAMES, build_interface_pullback_provider
from .suffix_scan import (
    _stack_for_chain,
    interface_state_jacobian_t_stats,
    propagate_state_adjoint_from_last_region_input,
)


def _adjoints_and_scan_rms(state_jacobians_t, g_last_input: torch.Tensor) -> tuple[list[torch.Tensor], float]:
    """State adjoints of every region input plus the RMS difference between the two ways of getting them."""
    stacked = _stack_for_chain(state_jacobians_t[:-1])            # the last region's output state is unused
    count = stacked.shape[1]
    # suffix[b, r] @ g[b] for all (b, r) at once (the identity tail returns g): the adjoints the step uses,
    # formed the way the reference forms them (backward/suffix_scan.py:49-53)
    applied = suffix_apply(suffix_scan_pullbacks(stacked), g_last_input)
    # the sequential chain from a kernel that shares nothing with the scan (the reference's g_manual, :63-69)
    chain = suffix_scan_cotangents(stacked, g_last_input)
    # mean over the count + 1 regions of the per-region mean square
    rms = torch.sqrt(((applied - chain) ** 2).mean())
    adjoints = [applied[:, r].to(g_last_input.dtype) for r in range(count + 1)]
    return adjoints, float(rms.item())


def lbi_scan_backward_step(
    model: Any,
    *,
    ce_loss: torch.Tensor,
    cache: dict[str, Any],
    pullback_provider: Any,
    local_vjp_provider: Any | None = None,
    compute_interface_jacobian_stats: bool = False,
    include_interface_jacobian_suffix: bool = False,
    check_scan: bool = True,
) -> LBIBackwardResult:
    """Exact scan backward for an LBI model using a supplied interface-pullback provider."""
    local_vjp_provider = local_vjp_provider or TorchAutogradLocalVJPProvider()
    bind_cache = getattr(local_vjp_provider, "bind_cache", None)
    if bind_cache is not None:
        bind_cache(cache)                # a provider that works from the cache (the protocol's calls do not pass it)
    grad_map = local_vjp_provider.new_grad_map(model)
    states = list(cache["states"])
    num_regions = len(list(cache["region_ranges"]))
    if num_regions == 0:
        raise RuntimeError("LBI scan backward requires at least one region.")

    local_vjp_provider.store_output_head_grads(model=model, loss=ce_loss, grad_map=grad_map)

    interface_scan_rms = 0.0
    interface_jacobian_stats = None
    if num_regions == 1:
        g_state_inputs = [local_vjp_provider.state_adjoint_from_loss(loss=ce_loss, state=states[0])]
    else:
        g_last_input = local_vjp_provider.state_adjoint_from_loss(loss=ce_loss, state=states[-2])
        # The last region's Jacobian is read by the statistics only (the reference builds it every step and drops
        # it, backward/suffix_scan.py:71-74): a provider that can leave it out is asked to.
        if not compute_interface_jacobian_stats and getattr(pullback_provider, "can_skip_last_region", False):
            state_jacobians_t = pullback_provider.materialize_state_jacobian_t(model=model, cache=cache, skip_last=True)
        else:
            state_jacobians_t = pullback_provider.materialize_state_jacobian_t(model=model, cache=cache)
        g_last_input = g_last_input.to(device=state_jacobians_t[0].device, dtype=state_jacobians_t[0].dtype)
        if compute_interface_jacobian_stats:
            interface_jacobian_stats = interface_state_jacobian_t_stats(
                state_jacobians_t, include_suffix=include_interface_jacobian_suffix)
        if len(state_jacobians_t) != num_regions:
            raise ValueError("state_jacobians_t length mismatch.")
        if check_scan:
            g_state_inputs, interface_scan_rms = _adjoints_and_scan_rms(state_jacobians_t, g_last_input)
        else:
            g_state_inputs = propagate_state_adjoint_from_last_region_input(
                state_jacobians_t, g_last_input, num_regions=num_regions)

    local_vjp_provider.store_initial_interface_grads(
        model=model, state0=states[0], state0_adjoint=g_state_inputs[0], grad_map=grad_map)
    for region_index in range(num_regions):
        local_vjp_provider.store_region_grads(
            model=model, loss=ce_loss, states=states, region_index=region_index, num_regions=num_regions,
            state_adjoints=g_state_inputs, grad_map=grad_map)
    local_vjp_provider.store_shared_canvas_grads(model=model, loss=ce_loss, grad_map=grad_map)
    return LBIBackwardResult(grad_map=grad_map, interface_scan_rms=interface_scan_rms,
                             interface_jacobian_stats=interface_jacobian_stats)


class ScanADEngine:
    """The engine the reference's training loop builds every step (train/runners.py:368-372): holds the two
    providers and the diagnostics switches, ``backward`` runs the step and writes ``param.grad``.  Constructor
    and ``from_config`` take the reference's arguments (backward/scan.py:103-136); ``state_jacobian_mode``
    also accepts ``"structured"`` for the provider that runs on the HIP region pullback."""

    name = "scan"

    def __init__(
        self,
        *,
        pullback_provider: Any | None = None,
        local_vjp_provider: Any | None = None,
        state_jacobian_mode: str = "graph",
        state_jacobian_basis_chunk: int | None = None,
        compute_interface_jacobian_stats: bool = False,
        include_interface_jacobian_suffix: bool = False,
        local_vjp_mode: str = "autograd",
    ) -> None:
        # ``state_jacobian_basis_chunk=None``: the provider's own default, which is the reference's 1 for its
        # autograd modes and "all d directions in one call" for the structured provider

        self.pullback_provider = pullback_provider or build_interface_pullback_provider(
            state_jacobian_mode, basis_chunk=state_jacobian_basis_chunk)
        # ``local_vjp_mode="structured"``: region parameter VJPs on the HIP kernels instead of the forward graph
        self.local_vjp_provider = local_vjp_provider or build_local_vjp_provider(local_vjp_mode)
        self.compute_interface_jacobian_stats = bool(compute_interface_jacobian_stats)
        self.include_interface_jacobian_suffix = bool(include_interface_jacobian_suffix)

    @classmethod
    def from_config(cls, cfg: Any, *, compute_interface_jacobian_stats: bool = False) -> "ScanADEngine":
        """Reads ``interface_jacobian_mode``, ``jacobian_basis_chunk`` and ``log_interface_jacobian_suffix``
        of the reference's training configuration (train/config.py:164-171).

        ``jacobian_basis_chunk`` is the reference's memory knob for its autograd providers (copies of the batch
        per recompute pass; default 1, values <= 0 rejected by its validator, train/config.py:169, :330) and is
        passed to those only.  The structured provider has no replicated batch: it pulls all ``d`` directions
        back in one call per region unless the configuration carries ``structured_basis_chunk`` (directions per
        call; absent or 0 = all), so a reference configuration object with its defaults gets the fast form.
        ``local_vjp_mode`` (absent = ``autograd``, the reference's provider) selects the local-VJP provider."""
        mode = str(cfg.interface_jacobian_mode)
        if mode.strip().lower().replace("-", "_") in STRUCTURED_MODE_NAMES:
            chunk = int(getattr(cfg, "structured_basis_chunk", 0) or 0)
        else:
            chunk = int(cfg.jacobian_basis_chunk)
        return cls(
            pullback_provider=build_interface_pullback_provider(mode, basis_chunk=chunk),
            local_vjp_provider=build_local_vjp_provider(str(getattr(cfg, "local_vjp_mode", "autograd"))),
            compute_interface_jacobian_stats=compute_interface_jacobian_stats,
            include_interface_jacobian_suffix=bool(cfg.log_interface_jacobian_suffix),
        )

    def backward(self, *, model: nn.Module, loss: torch.Tensor, cache: Any | None = None) -> ADResult:
        if not isinstance(model, ScanBackpropModel):
            raise TypeError("ScanADEngine requires a model satisfying ScanBackpropModel")
        if cache is None:
            raise ValueError("ScanADEngine requires a forward cache")
        model.zero_grad(set_to_none=True)
        result = lbi_scan_backward_step(
            model,
            ce_loss=loss,
            cache=cache,
            pullback_provider=self.pullback_provider,
            local_vjp_provider=self.local_vjp_provider,
            compute_interface_jacobian_stats=self.compute_interface_jacobian_stats,
            include_interface_jacobian_suffix=self.include_interface_jacobian_suffix,
        )
        assign_grad_map(model, result.grad_map)
        diagnostics: dict[str, Any] = {
            "interface_scan_rms": result.interface_scan_rms,
            "interface_pullback_provider": self.pullback_provider.name,
            "local_vjp_provider": self.local_vjp_provider.name,
        }
        if result.interface_jacobian_stats is not None:
            diagnostics["interface_jacobian_stats"] = dict(result.interface_jacobian_stats)
        return ADResult(grad_map=result.grad_map, diagnostics=diagnostics)


# The reference names the same class by its role as well (backward/scan.py:170-171).
ReferenceScanEngine = ScanADEngine


def lbi_reference_scan_backward_step(model: Any, *, ce_loss: torch.Tensor, cache: dict[str, Any],
                                     state_jacobian_mode: str = "graph",
                                     state_jacobian_basis_chunk: int | None = None,
                                     compute_interface_jacobian_stats: bool = False,
                                     include_interface_jacobian_suffix: bool = False) -> LBIBackwardResult:
    """The step configured by mode name (reference backward/reference_scan.py:12-34: same keywords):
    the provider comes from ``build_interface_pullback_provider``, the local VJPs from the default autograd
    provider.  Besides the reference's ``graph`` / ``recompute``, ``structured`` selects the provider whose region
    pullback runs on the HIP kernels (``state_jacobian_basis_chunk`` then counts directions per call, 0 = all).
    ``state_jacobian_basis_chunk=None`` is the reference's default of 1 for its own modes and all directions in
    one call for ``structured``."""
    return lbi_scan_backward_step(
        model, ce_loss=ce_loss, cache=cache,
        pullback_provider=build_interface_pullback_provider(state_jacobian_mode, basis_chunk=state_jacobian_basis_chunk),
        compute_interface_jacobian_stats=compute_interface_jacobian_stats,
        include_interface_jacobian_suffix=include_interface_jacobian_suffix)


__all__ = ["LBIBackwardResult", "ReferenceScanEngine", "ScanADEngine", "lbi_reference_scan_backward_step",
           "lbi_scan_backward_step"]
