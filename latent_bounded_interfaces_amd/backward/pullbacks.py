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

import weakref
from typing import Any

import torch

from ..contracts import InterfacePullbackProvider


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
        # (interface instance, region length) -> True once a non-zero cotangent was seen to be constant
        self._constant_over_positions: "weakref.WeakKeyDictionary[Any, dict[int, bool]]" = weakref.WeakKeyDictionary()

    def _region_output_cotangent(self, interface: Any, g_region_output: torch.Tensor) -> torch.Tensor:
        """An interface that pools the region output with a mean over positions sends the same cotangent to
        every position (reference interfaces/vector_mlp.py:111-116 materialises it as a dense [B,P,T,D]
        tensor).  When that holds the tensor is handed on as a stride-0 view of its first position, which lets
        the region pullback run the last block's first product on one row per direction.

        An interface may declare the property (attribute ``region_output_cotangent_constant_over_positions``:
        True / False); otherwise it is checked on the device (one host synchronisation): on every call
        (``verify``), or until a call has shown it for this interface object and this region length with a
        cotangent that is not all zero (``verify_once``: an all-zero cotangent, e.g. from a zero-initialised gate,
        is constant trivially and proves nothing about later steps).  A negative finding is never cached."""
        if self.position_constant_update == "off" or g_region_output.dim() != 4 or g_region_output.shape[2] <= 1:
            return g_region_output
        if g_region_output.stride(2) == 0:
            return g_region_output
        declared = getattr(interface, "region_output_cotangent_constant_over_positions", None)
        if declared is False:
            return g_region_output
        first = g_region_output[:, :, :1].expand_as(g_region_output)
        seq_len = int(g_region_output.shape[2])
        if self.position_constant_update == "verify_once":
            try:
                seen = self._constant_over_positions.setdefault(interface, {})
            except TypeError:  # an interface object that cannot be weakly referenced: check every time
                seen = {}
            if seen.get(seq_len):
                return first
            flags = torch.stack([(first == g_region_output).all(), (g_region_output != 0).any()]).cpu().tolist()
            if flags[0] and flags[1]:
                seen[seq_len] = True
            return first if flags[0] else g_region_output
        return first if bool(torch.equal(first, g_region_output)) else g_region_output

    def region_state_jacobian_t(self, *, model: Any, region_cache: Any, out: torch.Tensor | None = None,
                                dtype: torch.dtype | None = None) -> torch.Tensor:
        """``Jt`` of one region, ``[B, d, d]``; written into ``out`` (any strides) when given.  ``dtype``: dtype of
        the cotangent basis and of the result (default: that of ``out``, else of the region's input state)."""
        state_in = region_cache.state_in
        if state_in.dim() != 2:
            raise ValueError("interface state inputs must be [B, R].")
        bsz, rank = state_in.shape
        chunk = self.basis_chunk or rank
        dtype = dtype or (out.dtype if out is not None else state_in.dtype)
        eye = torch.eye(rank, device=state_in.device, dtype=dtype)
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
                if out is not None:
                    out[:, :, start:start + total.shape[1]].copy_(total.transpose(1, 2))
                else:
                    cols.append(total.transpose(1, 2))                    # [B, d_in, P]
        if out is not None:
            return out
        return torch.cat(cols, dim=-1).to(device=state_in.device, dtype=dtype).contiguous()

    #: ``materialize_state_jacobian_t`` takes ``skip_last=True``: the scan backward step asks for that when nothing
    #: reads the last region's Jacobian (one region pullback less per step)
    can_skip_last_region = True

    def materialize_state_jacobian_t(self, *, model: Any, cache: dict[str, Any],
                                     skip_last: bool = False) -> list[torch.Tensor]:
        """One ``[B, d, d]`` tensor per region.  The first K - 1 of them are slices of ONE dense ``[B, K-1, d, d]``
        buffer, in order: the scan backward step composes exactly those (the last region's output state never
        reaches the loss, reference backward/suffix_scan.py:71), and ``backward.suffix_scan`` hands such a list to
        the kernels as it lies, without the stacking copy (reference backward/suffix_scan.py:17).

        ``skip_last=True`` leaves the last region's Jacobian out (``None`` in its place): the reference builds it
        and drops it (backward/scan.py:44, backward/suffix_scan.py:71-74); only the Jacobian statistics read it."""
        region_caches = cache["region_caches"]
        count = len(region_caches)
        if count != model.num_regions:
            raise ValueError("cache has invalid region_caches length.")
        if count < 2:
            if skip_last:
                return [None for _ in region_caches]
            return [self.region_state_jacobian_t(model=model, region_cache=rc) for rc in region_caches]
        state = region_caches[0].state_in
        bsz, rank = state.shape
        # one dtype for all regions: a forward under autocast can leave the first state 16-bit and the others fp32
        dtype = state.dtype
        for rc in region_caches[1:]:
            dtype = torch.promote_types(dtype, rc.state_in.dtype)
        inner = torch.empty((bsz, count - 1, rank, rank), device=state.device, dtype=dtype)
        result = [self.region_state_jacobian_t(model=model, region_cache=rc, out=inner[:, r])
                  for r, rc in enumerate(region_caches[:-1])]
        result.append(None if skip_last else
                      self.region_state_jacobian_t(model=model, region_cache=region_caches[-1], dtype=dtype))
        return result


class TorchGraphInterfacePullbackProvider:
    """``Jt`` per region from the forward graph held by ``cache["states"]`` (the reference's default provider,
    backward/pullbacks.py:37-81, 152-165): ``d`` vector-Jacobian products of ``s_{r+1}`` with respect to
    ``s_r``, batched through ``is_grads_batched`` where every operator on the way supports it, one at a time
    otherwise.  Plain ``torch.autograd`` on whatever device the states live on; no kernel of this package is
    involved until the matrices reach the scan."""

    name = "torch_graph"

    def __init__(self, *, basis_chunk: int = 1) -> None:
        self.basis_chunk = int(basis_chunk)

    #: see ``StructuredInterfacePullbackProvider.can_skip_last_region``
    can_skip_last_region = True

    def materialize_state_jacobian_t(self, *, model: Any, cache: dict[str, Any],
                                     skip_last: bool = False) -> list[torch.Tensor]:
        states = cache["states"]
        if len(states) != model.num_regions + 1:
            raise ValueError("cache has invalid states length.")
        result = []
        for index, (s_in, s_out) in enumerate(zip(states[:-1], states[1:])):
            if s_in.dim() != 2 or s_out.dim() != 2:
                raise ValueError("interface states must be [B, R].")
            if skip_last and index == len(states) - 2:
                result.append(None)  # never read by the scan backward step
                break
            bsz, rank = s_out.shape
            eye = torch.eye(rank, device=s_out.device, dtype=s_out.dtype)

            def vjp(seed, batched):
                return torch.autograd.grad(s_out, s_in, grad_outputs=seed, retain_graph=True, create_graph=False,
                                           allow_unused=False, is_grads_batched=batched)[0]

            try:
                rows = vjp(eye.unsqueeze(1).expand(rank, bsz, rank), True)        # [j, B, i]
                result.append(rows.permute(1, 2, 0).contiguous())
            except (TypeError, RuntimeError) as exc:
                if isinstance(exc, RuntimeError) and "doesn't have storage" not in str(exc):
                    raise
                cols = [vjp(eye[j].expand(bsz, rank), False) for j in range(rank)]
                result.append(torch.stack(cols, dim=-1))
        return result


class TorchRecomputeInterfacePullbackProvider:
    """``Jt`` per region by re-running the region on a replicated batch (the reference's ``recompute`` mode,
    backward/pullbacks.py:84-149, 168-182): ``basis_chunk`` copies of the batch go through decode -> region ->
    update again, and one backward pass seeded with that many basis vectors yields as many columns.  Needs
    no forward graph in the cache.  Plain ``torch.autograd``, as above."""

    name = "torch_recompute"

    def __init__(self, *, basis_chunk: int = 1) -> None:
        self.basis_chunk = int(basis_chunk)

    @staticmethod
    def _state_map(model: Any, region_index: int, canvas: torch.Tensor, state: torch.Tensor) -> torch.Tensor:
        condition = model.interface.decode(state, region_index)
        region_output, _ = model.region_backend.forward_region(region_input=canvas + condition.unsqueeze(1),
                                                               region_index=region_index)
        return model.interface.update(state, region_output, region_index).state

    #: see ``StructuredInterfacePullbackProvider.can_skip_last_region``
    can_skip_last_region = True

    def materialize_state_jacobian_t(self, *, model: Any, cache: dict[str, Any],
                                     skip_last: bool = False) -> list[torch.Tensor]:
        if self.basis_chunk <= 0:
            raise ValueError("basis_chunk must be > 0.")
        region_caches = cache["region_caches"]
        if len(region_caches) != model.num_regions:
            raise ValueError("cache has invalid region_caches length.")
        result = []
        for index, rc in enumerate(region_caches):
            if skip_last and index == len(region_caches) - 1:
                result.append(None)  # never read by the scan backward step
                break
            state, canvas = rc.state_in.detach(), rc.canvas_features.detach()
            if state.dim() != 2:
                raise ValueError("interface state inputs must be [B, R].")
            if canvas.dim() != 3:
                raise ValueError("canvas_features must be [B, L, D].")
            bsz, rank = state.shape
            if canvas.shape[0] != bsz:
                raise ValueError("canvas_features and state batch sizes do not match.")
            eye = torch.eye(rank, device=state.device, dtype=state.dtype)
            cols = []
            for start in range(0, rank, self.basis_chunk):
                basis = eye[start:start + self.basis_chunk]
                n = int(basis.shape[0])
                with torch.enable_grad():
                    state_rep = state.repeat(n, 1).requires_grad_(True)               # copy c holds rows c*B..c*B+B-1
                    out_rep = self._state_map(model, rc.region_index, canvas.repeat(n, 1, 1), state_rep)
                    seed = basis.repeat_interleave(bsz, dim=0).to(device=out_rep.device, dtype=out_rep.dtype)
                    (g_in,) = torch.autograd.grad(out_rep, state_rep, grad_outputs=seed)
                cols.append(g_in.reshape(n, bsz, rank).permute(1, 2, 0))
            result.append(torch.cat(cols, dim=-1).to(device=state.device, dtype=state.dtype).contiguous())
        return result


def materialize_interface_state_jacobian_t_graph(*, model: Any, cache: dict[str, Any]) -> list[torch.Tensor]:
    """Function form of the graph provider (reference backward/pullbacks.py:37-81)."""
    return TorchGraphInterfacePullbackProvider().materialize_state_jacobian_t(model=model, cache=cache)


def materialize_interface_state_jacobian_t_recompute(*, model: Any, cache: dict[str, Any],
                                                     basis_chunk: int = 1) -> list[torch.Tensor]:
    """Function form of the recompute provider (reference backward/pullbacks.py:84-149)."""
    return TorchRecomputeInterfacePullbackProvider(basis_chunk=basis_chunk).materialize_state_jacobian_t(
        model=model, cache=cache)


#: normalised mode names that select the structured provider
STRUCTURED_MODE_NAMES = frozenset({"structured", "hip", "structured_hip"})


def build_interface_pullback_provider(mode: str, *, basis_chunk: int | None = None,
                                      position_constant_update: str = "verify_once"):
    """Provider by name.  ``graph`` / ``recompute`` and their aliases are the reference's modes
    (backward/pullbacks.py:185-197; the values its configuration field ``interface_jacobian_mode`` takes) and
    give the autograd providers above; ``structured`` (aliases ``hip``, ``structured_hip``) gives the provider
    that runs the region pullback on the HIP kernels, for which ``basis_chunk`` counts directions per call.
    ``basis_chunk=None`` means the reference's default of 1 for the autograd providers and 0 (all ``d``
    directions in one call) for the structured one."""
    normalized = str(mode).strip().lower().replace("-", "_")
    if normalized in STRUCTURED_MODE_NAMES:
        return StructuredInterfacePullbackProvider(basis_chunk=0 if basis_chunk is None else basis_chunk,
                                                   position_constant_update=position_constant_update)
    basis_chunk = 1 if basis_chunk is None else basis_chunk
    if normalized in {"graph", "torch_graph", "pytorch_graph"}:
        return TorchGraphInterfacePullbackProvider(basis_chunk=basis_chunk)
    if normalized in {"recompute", "torch_recompute", "pytorch_recompute"}:
        return TorchRecomputeInterfacePullbackProvider(basis_chunk=basis_chunk)
    raise ValueError("interface pullback provider must be one of: graph, recompute, torch_graph, torch_recompute, "
                     "structured, hip")


__all__ = ["InterfacePullbackProvider", "STRUCTURED_MODE_NAMES", "StructuredInterfacePullbackProvider",
           "TorchGraphInterfacePullbackProvider", "TorchRecomputeInterfacePullbackProvider",
           "build_interface_pullback_provider", "materialize_interface_state_jacobian_t_graph",
           "materialize_interface_state_jacobian_t_recompute"]
