"""State-adjoint propagation through the interface chain, on the HIP scan kernels.

Counterpart of reference backward/suffix_scan.py with the same function names,
arguments, results and exceptions.  ``Jt[b, i, j] = d s_out[j] / d s_in[i]`` and
``g_in = Jt @ g_out`` (reference backward/pullbacks.py:53-64).
"""
from __future__ import annotations

from collections.abc import Sequence

import torch

from ..hip.interface import matrix_norms, suffix_apply, suffix_scan_cotangents
from ..hip.interface import suffix_scan_pullbacks as suffix_scan_jacobian_t


def compose_suffix_jacobian_t(state_jacobians_t: Sequence[torch.Tensor]) -> list[torch.Tensor]:
    """All suffix products of the K matrices plus the identity, as K+1 tensors ``[B, d, d]``.

    Same contract as reference backward/suffix_scan.py:10-21.
    """
    count = len(state_jacobians_t)
    if count == 0:
        return []
    bsz, rank, rank2 = state_jacobians_t[0].shape
    if rank != rank2:
        raise ValueError("interface state Jacobian-transpose tensors must be square.")
    stacked = _stack_for_chain(state_jacobians_t)
    suffix = suffix_scan_jacobian_t(stacked)
    if suffix.shape != (bsz, count + 1, rank, rank):
        raise ValueError("suffix scan returned an unexpected shape")
    return [suffix[:, region_index].contiguous() for region_index in range(count + 1)]


def apply_jacobian_t(
    jacobian_t: torch.Tensor,
    cotangent: torch.Tensor,
    *,
    out_dtype: torch.dtype | None = None,
) -> torch.Tensor:
    """``result[b] = jacobian_t[b] @ cotangent[b]`` (reference backward/suffix_scan.py:24-38).

    Runs as a one-step cotangent chain on the device.  The reference multiplies in
    ``promote_types(jacobian_t.dtype, cotangent.dtype)``; here the kernel reads fp32 / fp16 / bf16
    matrices as stored, accumulates in fp32 and the result is cast to ``out_dtype`` (default: the
    cotangent's dtype).  Any other matrix dtype (fp64 included) is accepted and converted to fp32 first,
    so an fp64 call keeps the reference's result dtype but carries fp32 accuracy.
    """
    if jacobian_t.dim() != 3 or cotangent.dim() != 2:
        raise ValueError("jacobian_t must be [B, d, d] and cotangent [B, d]")
    if out_dtype is None:
        out_dtype = cotangent.dtype
    if jacobian_t.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        jacobian_t = jacobian_t.to(torch.float32)
    chain = suffix_scan_cotangents(jacobian_t.unsqueeze(1), cotangent.to(device=jacobian_t.device))
    return chain[:, 0].to(device=cotangent.device, dtype=out_dtype)


def _dense_stack_view(mats: Sequence[torch.Tensor]) -> torch.Tensor | None:
    """The list as one ``[B, K, d, d]`` tensor WITHOUT a copy, if its members are, in order, the K slices
    ``buf[:, r]`` of one dense ``[B, K, d, d]`` buffer (what ``StructuredInterfacePullbackProvider`` returns for
    the matrices the scan composes); else None."""
    first = mats[0]
    count = len(mats)
    bsz, rank, _ = first.shape
    item, step = first.element_size(), rank * rank
    want_strides = (count * step, rank, 1)
    for r, m in enumerate(mats):
        if (m.shape != first.shape or m.dtype != first.dtype or m.device != first.device
                or (bsz > 1 and m.stride() != want_strides) or m.stride()[1:] != want_strides[1:]
                or m.data_ptr() != first.data_ptr() + r * step * item
                or m.untyped_storage().data_ptr() != first.untyped_storage().data_ptr()):
            return None
    need = first.storage_offset() + (bsz - 1) * count * step + count * step
    if first.untyped_storage().nbytes() < need * item:
        return None
    return torch.as_strided(first, (bsz, count, rank, rank), (count * step, step, rank, 1))


def _stack_for_chain(state_jacobians_t: Sequence[torch.Tensor]) -> torch.Tensor:
    bsz, rank, rank2 = state_jacobians_t[0].shape
    if rank != rank2:
        raise ValueError("interface state Jacobian-transpose tensors must be square.")
    dense = _dense_stack_view(state_jacobians_t)
    if dense is not None:
        return dense
    return torch.stack(list(state_jacobians_t), dim=1).contiguous()


def propagate_state_adjoint_with_jacobian_scan(
    state_jacobians_t: Sequence[torch.Tensor],
    g_top_state: torch.Tensor,
    *,
    materialize_suffix: bool = False,
) -> list[torch.Tensor]:
    """K+1 state cotangents ``[suffix[r] @ g for r < K] + [g]``.

    Same results as reference backward/suffix_scan.py:41-56.  By default the
    cotangent-only kernel is used (one pass over the matrices, no ``d x d``
    product); ``materialize_suffix=True`` forms the suffix matrices first, as the
    reference does.
    """
    count = len(state_jacobians_t)
    if count == 0:
        # The reference reaches its length check with an empty suffix list here.
        raise ValueError("suffix length mismatch.")
    if materialize_suffix:
        suffix = suffix_scan_jacobian_t(_stack_for_chain(state_jacobians_t))
        if suffix.shape[1] != count + 1:
            raise ValueError("suffix length mismatch.")
        g_top_state = g_top_state.to(device=suffix.device, dtype=suffix.dtype)
        applied = suffix_apply(suffix, g_top_state)   # the K mat-vecs of the reference (and the identity) in one launch
        g_states = [applied[:, region_index] for region_index in range(count)]
        g_states.append(g_top_state)
        return g_states
    stacked = _stack_for_chain(state_jacobians_t)
    chain = suffix_scan_cotangents(stacked, g_top_state)
    return [chain[:, region_index] for region_index in range(count + 1)]


def propagate_state_adjoint_from_last_region_input(
    state_jacobians_t: Sequence[torch.Tensor],
    g_last_input_state: torch.Tensor,
    *,
    num_regions: int,
    materialize_suffix: bool = False,
) -> list[torch.Tensor]:
    """Cotangents of every region's input state given the one of the last region's input.

    Same contract as reference backward/suffix_scan.py:59-79: the last matrix is
    dropped (the last region's output state never reaches the loss), length
    mismatch raises ``ValueError``, ``num_regions`` 0 / 1 return ``[]`` / ``[g]``.
    """
    if len(state_jacobians_t) != num_regions:
        raise ValueError("state_jacobians_t length mismatch.")
    if num_regions == 0:
        return []
    if num_regions == 1:
        return [g_last_input_state]
    return propagate_state_adjoint_with_jacobian_scan(
        state_jacobians_t[:-1], g_last_input_state, materialize_suffix=materialize_suffix
    )


def propagate_state_adjoint_by_autograd_chain(
    *,
    states: Sequence[torch.Tensor],
    top_state_adjoint: torch.Tensor,
) -> list[torch.Tensor]:
    """Diagnostic of the reference (backward/suffix_scan.py:82-102): the same adjoints walked through an
    existing autograd graph, one ``torch.autograd.grad`` per region; no kernel of this package is involved."""
    if len(states) < 2:
        raise ValueError("at least two interface states are required.")
    g_states = [torch.zeros_like(states[0]) for _ in states]
    g_states[-1] = top_state_adjoint
    for region_index in reversed(range(len(states) - 1)):
        (g_states[region_index],) = torch.autograd.grad(
            states[region_index + 1], states[region_index], grad_outputs=g_states[region_index + 1],
            retain_graph=True, create_graph=False, allow_unused=False)
    return g_states


def interface_state_jacobian_t_stats(
    state_jacobians_t: Sequence[torch.Tensor],
    *,
    include_suffix: bool,
) -> dict[str, float]:
    """Frobenius / spectral norm diagnostics (reference backward/suffix_scan.py:105-134): same keys and
    values, from one ``lbi_matrix_norms`` launch per group of matrices instead of a singular value
    decomposition per matrix; the only host synchronisation is the final read of the seven scalars."""
    if not state_jacobians_t:
        return {}
    with torch.no_grad():
        dense = torch.stack([jt.detach() for jt in state_jacobians_t], dim=1)
        if dense.dtype not in (torch.float32, torch.float16, torch.bfloat16):
            dense = dense.float()
        spec, frob = matrix_norms(dense)
        rank = max(1, int(dense.shape[-1]))
        values = [spec.mean(), spec.max(), frob.mean(), frob.max(), (frob / (rank ** 0.5)).mean()]
        keys = ["jac_local_spec_mean", "jac_local_spec_max", "jac_local_frob_mean", "jac_local_frob_max",
                "jac_local_frob_normed_mean"]
        if include_suffix:
            suffix_spec, _ = matrix_norms(suffix_scan_jacobian_t(dense.contiguous()))
            values += [suffix_spec.mean(), suffix_spec.max()]
            keys += ["jac_suffix_spec_mean", "jac_suffix_spec_max"]
        host = torch.stack(values).cpu().tolist()
        return dict(zip(keys, (float(v) for v in host)))


__all__ = ["apply_jacobian_t", "compose_suffix_jacobian_t", "interface_state_jacobian_t_stats",
           "propagate_state_adjoint_by_autograd_chain", "propagate_state_adjoint_from_last_region_input",
           "propagate_state_adjoint_with_jacobian_scan"]
