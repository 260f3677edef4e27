"""Region-local parameter VJPs: on the forward graph, or on the HIP region kernels.

``TorchAutogradLocalVJPProvider`` is the provider the reference's scan step falls back to when
the caller passes none (reference backward/scan.py:28; class backward/local_vjp.py:66-185): every
gradient is one ``torch.autograd.grad`` call whose seed is either the loss or a state adjoint the
scan produced, so no gradient ever crosses a region boundary through the graph.  It holds no
kernel of its own; it is here so that the engine entries keep the reference's defaults.

``StructuredLocalVJPProvider`` fills the same protocol (reference backward/local_vjp.py:10-63) from
the forward CACHE: a region's parameter gradients are ``region_backend.parameter_vjp`` of the
cotangent of its output (reference backends/transformer.py:270-280), which with
``HipTransformerLowering`` is one backward sweep on the HIP kernels, and the small interface maps
around the region (pooling + encoder + normalisation on the way out, decoder on the way in) are
re-run on detached inputs and differentiated by autograd on their own.  The forward graph is walked
only from the loss to the last region's output (readout) and from the canvas features to the canvas
parameters (embedding).
"""
from __future__ import annotations

from typing import Any

import torch

from ..contracts import LocalVJPProvider
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


def _wide(t: torch.Tensor) -> torch.Tensor:
    """16-bit cotangents are accumulated in fp32; fp32 and fp64 ones as they are."""
    return t if t.dtype in (torch.float32, torch.float64) else t.float()


def _add(total: torch.Tensor | None, term: torch.Tensor | None) -> torch.Tensor | None:
    if term is None:
        return total
    return term if total is None else total + term


class StructuredLocalVJPProvider:
    """The local-VJP protocol of the scan step (reference backward/local_vjp.py:10-63) on the forward cache.

    Per region ``r`` with seed ``g = state_adjoints[r + 1]`` on its output state (the last region: the loss's own
    cotangent of its output instead, reference backward/local_vjp.py:158-175):

    1. update side: ``interface.update(state_in, region_output, r)`` re-run on detached inputs, one
       ``autograd.grad`` for the cotangent of the region output and the gradients of the interface parameters
       that act there (encoder, normalisation, the shared update scale);
    2. region: ``lowering.parameter_vjp_with_input_cotangent`` (one sweep for the block parameters and the
       cotangent of the region input; a lowering without it gets ``parameter_vjp`` and ``input_pullback_basis``
       with one direction, the two calls of the reference's protocol);
    3. decode side: ``interface.decode(state_in, r)`` re-run, seeded with the region-input cotangent summed over
       positions (the condition is broadcast to every position, reference models/lbi_language_model.py:171), for
       the decoder gradients; the region-input cotangent itself is the region's share of the canvas cotangent.

    The methods of the protocol do not receive the cache, so the provider is bound to it: ``cache=`` at
    construction (the reference builds its engine anew every step, train/runners.py:368) or ``bind_cache(cache)``,
    which ``lbi_scan_backward_step`` of this package calls when the method exists.  A model whose readout shares
    a parameter with the canvas (tied embeddings) gets its shared gradients by autograd on the full graph, as the
    reference does (backward/local_vjp.py:176-184); everything else is as above."""

    name = "structured"

    def __init__(self, *, cache: dict[str, Any] | None = None) -> None:
        self.bind_cache(cache)

    def bind_cache(self, cache: dict[str, Any] | None) -> None:
        self._cache = cache
        self._g_last_output: torch.Tensor | None = None          # d loss / d output of the last region
        self._g_canvas: torch.Tensor | None = None               # cotangent of the canvas features, summed
        self._shared: dict[int, torch.Tensor] = {}                # id(param) -> gradient of interface-shared params
        self._last_region: dict[str, Any] | None = None           # the last region's sweep, run once
        self._model: Any | None = None                            # set by the first call of a step

    # -- helpers ----------------------------------------------------------------------------------------------
    @staticmethod
    def _names(model: Any) -> dict[int, str]:
        return {id(p): n for n, p in model.named_parameters() if p.requires_grad}

    def _region_caches(self) -> list:
        if self._cache is None:
            raise RuntimeError("StructuredLocalVJPProvider needs the forward cache: pass cache= or call bind_cache")
        return list(self._cache["region_caches"])

    def new_grad_map(self, model: Any) -> GradMap:
        return {n: None for n, p in model.named_parameters() if p.requires_grad}

    def _store(self, model: Any, grad_map: GradMap, params: list, grads: list) -> None:
        names = self._names(model)
        for p, g in zip(params, grads):
            if id(p) in names:
                grad_map[names[id(p)]] = None if g is None else g.detach().to(p.dtype)

    def _region_sweep(self, model: Any, region_cache: Any, g_region_output: torch.Tensor
                      ) -> tuple[dict[int, torch.Tensor], torch.Tensor]:
        """Block-parameter gradients (by ``id``) and the region-input cotangent ``[B, T, D]`` for one region."""
        backend = model.region_backend
        lowering = getattr(backend, "lowering", None)
        fused = getattr(lowering, "parameter_vjp_with_input_cotangent", None)
        if fused is not None:
            by_name, g_in = fused(backend=backend, cache=region_cache.backend_cache, output_cotangent=g_region_output)
        else:
            by_name = backend.parameter_vjp(cache=region_cache.backend_cache, output_cotangent=g_region_output)
            g_in = backend.input_pullback_basis(cache=region_cache.backend_cache,
                                                output_cotangent_basis=g_region_output.unsqueeze(1))[:, 0]
        params = dict(backend.named_parameters())
        return {id(params[n]): g for n, g in by_name.items()}, g_in

    def _decode_side(self, model: Any, region_cache: Any, g_region_input: torch.Tensor
                     ) -> tuple[torch.Tensor, dict[int, torch.Tensor]]:
        """Region-input cotangent -> (cotangent of the region's input state, decoder gradients by ``id``)."""
        r = region_cache.region_index
        params = [p for p in model.interface.region_vjp_parameters(r) if p.requires_grad]
        with torch.enable_grad():
            state = region_cache.state_in.detach().requires_grad_(True)
            condition = model.interface.decode(state, r)
            seed = g_region_input.sum(dim=1).to(condition.dtype)
            grads = torch.autograd.grad(condition, [state, *params], grad_outputs=seed, allow_unused=True)
        return grads[0].detach(), {id(p): g for p, g in zip(params, grads[1:]) if g is not None}

    def _update_side(self, model: Any, region_cache: Any, seed: torch.Tensor
                     ) -> tuple[torch.Tensor, dict[int, torch.Tensor]]:
        """Cotangent of the output state -> (cotangent of the region output ``[B, T, D]``, gradients by ``id`` of
        the region's and the shared interface parameters acting in the update)."""
        r = region_cache.region_index
        params = [p for p in (*model.interface.region_vjp_parameters(r), *model.interface.shared_vjp_parameters())
                  if p.requires_grad]
        with torch.enable_grad():
            region_output = region_cache.region_output.detach().requires_grad_(True)
            state_out = model.interface.update(region_cache.state_in.detach(), region_output, r).state
            grads = torch.autograd.grad(state_out, [region_output, *params],
                                        grad_outputs=seed.to(device=state_out.device, dtype=state_out.dtype),
                                        allow_unused=True)
        return grads[0].detach(), {id(p): g for p, g in zip(params, grads[1:]) if g is not None}

    def _run_last_region(self, model: Any) -> dict[str, Any]:
        if self._last_region is None:
            if self._g_last_output is None:
                raise RuntimeError("store_output_head_grads must run before the last region's gradients are formed")
            region_cache = self._region_caches()[-1]
            block_grads, g_in = self._region_sweep(model, region_cache, self._g_last_output)
            g_state, decoder_grads = self._decode_side(model, region_cache, g_in)
            self._g_canvas = _add(self._g_canvas, _wide(g_in))
            self._last_region = {"grads": {**block_grads, **decoder_grads}, "g_state": g_state}
        return self._last_region

    # -- the protocol, in the order the scan step calls it (reference backward/scan.py:29-96) -------------------
    def store_output_head_grads(self, *, model: Any, loss: torch.Tensor, grad_map: GradMap) -> None:
        self._model = model          # ``state_adjoint_from_loss``, the next call of a step, is not handed the model
        params = [p for p in model.output_head_vjp_parameters() if p.requires_grad]
        last_output = self._region_caches()[-1].region_output
        # one walk from the loss through the readout: its parameters and the cotangent the last region starts from
        grads = torch.autograd.grad(loss, [*params, last_output], retain_graph=True, create_graph=False,
                                    allow_unused=True)
        self._store(model, grad_map, params, grads[:-1])
        self._g_last_output = grads[-1].detach()

    def state_adjoint_from_loss(self, *, loss: torch.Tensor, state: torch.Tensor) -> torch.Tensor:
        region_caches = self._region_caches()
        if state is not region_caches[-1].state_in or self._model is None:
            # not the state the last region read: the graph answers
            (g,) = torch.autograd.grad(loss, state, retain_graph=True, create_graph=False, allow_unused=False)
            return g.detach().to(device=state.device, dtype=state.dtype)
        return self._run_last_region(self._model)["g_state"].to(device=state.device, dtype=state.dtype)

    def store_initial_interface_grads(self, *, model: Any, state0: torch.Tensor, state0_adjoint: torch.Tensor,
                                      grad_map: GradMap) -> None:
        params = [p for p in model.interface.initial_vjp_parameters() if p.requires_grad]
        with torch.enable_grad():
            canvas = self._cache["canvas_features"].detach().requires_grad_(True)
            state = model.interface.initialize(canvas)
            grads = torch.autograd.grad(state, [canvas, *params],
                                        grad_outputs=state0_adjoint.to(device=state.device, dtype=state.dtype),
                                        allow_unused=True)
        self._g_canvas = _add(self._g_canvas, None if grads[0] is None else _wide(grads[0].detach()))
        self._store(model, grad_map, params, grads[1:])

    def store_region_grads(self, *, model: Any, loss: torch.Tensor, states: list, region_index: int, num_regions: int,
                           state_adjoints: list, grad_map: GradMap) -> None:
        region_cache = self._region_caches()[region_index]
        params = [*model.region_backend.parameters_for_region(region_index),
                  *model.interface.region_vjp_parameters(region_index)]
        shared_ids = {id(p) for p in model.interface.shared_vjp_parameters()}
        if region_index == num_regions - 1:
            # the last region feeds the readout directly; its output state is never used
            by_id = self._run_last_region(model)["grads"]
        else:
            g_output, by_id = self._update_side(model, region_cache, state_adjoints[region_index + 1])
            for key in [k for k in by_id if k in shared_ids]:
                self._shared[key] = _add(self._shared.get(key), by_id.pop(key))
            block_grads, g_in = self._region_sweep(model, region_cache, g_output)
            _, decoder_grads = self._decode_side(model, region_cache, g_in)
            self._g_canvas = _add(self._g_canvas, _wide(g_in))
            by_id = {**by_id, **block_grads}
            for key, g in decoder_grads.items():
                by_id[key] = _add(by_id.get(key), g)
        self._store(model, grad_map, params, [by_id.get(id(p)) for p in params])

    def store_shared_canvas_grads(self, *, model: Any, loss: torch.Tensor, grad_map: GradMap) -> None:
        canvas_params = [p for p in model.canvas_vjp_parameters() if p.requires_grad]
        head_ids = {id(p) for p in model.output_head_vjp_parameters()}
        tied = getattr(model, "tie_embeddings", False) or any(id(p) in head_ids for p in canvas_params)
        interface_shared = [p for p in model.interface.shared_vjp_parameters() if p.requires_grad]
        self._store(model, grad_map, interface_shared, [self._shared.get(id(p)) for p in interface_shared])
        if not canvas_params:
            return
        if tied:
            grads = torch.autograd.grad(loss, canvas_params, retain_graph=False, create_graph=False, allow_unused=True)
        elif self._g_canvas is None:
            grads = [None] * len(canvas_params)
        else:
            features = self._cache["canvas_features"]
            grads = torch.autograd.grad(features, canvas_params, grad_outputs=self._g_canvas.to(features.dtype),
                                        retain_graph=False, create_graph=False, allow_unused=True)
        self._store(model, grad_map, canvas_params, grads)


def build_local_vjp_provider(mode: str = "autograd", *, cache: dict[str, Any] | None = None):
    """``autograd`` / ``torch_autograd``: the reference's provider; ``structured`` / ``hip``: the provider that
    runs region parameter VJPs on the HIP kernels (bound to ``cache`` if given)."""
    normalized = str(mode).strip().lower().replace("-", "_")
    if normalized in {"autograd", "torch_autograd", "torch", "graph"}:
        return TorchAutogradLocalVJPProvider()
    if normalized in {"structured", "hip", "structured_hip"}:
        return StructuredLocalVJPProvider(cache=cache)
    raise ValueError("local VJP provider must be one of: autograd, torch_autograd, structured, hip")


__all__ = ["LocalVJPProvider", "StructuredLocalVJPProvider", "TorchAutogradLocalVJPProvider",
           "build_local_vjp_provider"]
