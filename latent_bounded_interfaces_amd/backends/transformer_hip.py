"""HIP lowering for Transformer region derivative contracts.

Counterpart of reference backends/transformer_cuda.py (``CudaTransformerLowering``)
and an implementation of the ``TransformerLowering`` protocol of reference
backends/transformer.py:64-85.
"""
from __future__ import annotations

from typing import Any

import torch

from ..hip.transformer import attention_input_pullback_basis as hip_attention_input_pullback_basis
from ..hip.transformer.region import (region_input_pullback_basis, region_parameter_vjp,
                                      region_parameter_vjp_with_input_cotangent)


class HipTransformerLowering:
    """HIP lowering for Transformer region derivative contracts."""

    name = "hip"

    def __init__(self, *, reference_lowering: Any | None = None) -> None:
        # The reference's class can delegate the region-level methods to its autograd lowering
        # (allow_reference_fallback=True).  Here both run the HIP path; a caller who passes a
        # `reference_lowering` gets parameter_vjp from it instead.
        self.reference_lowering = reference_lowering
        self.allow_reference_fallback = reference_lowering is not None

    def attention_input_pullback_basis(
        self,
        *,
        q: torch.Tensor,
        k: torch.Tensor,
        v: torch.Tensor,
        output_cotangent_basis: torch.Tensor,
        softmax_scale: float,
        causal: bool = True,
        kernel_mode: str = "fa2_mma_pblock4",
    ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """Same keyword-only contract and default mode as reference backends/transformer_cuda.py:23-43 (the
        default therefore keeps that mode's limit of four directions per call, a ``ValueError`` beyond it);
        ``kernel_mode="hip"`` is the mode without a limit.  Every mode runs the same HIP kernels."""
        return hip_attention_input_pullback_basis(
            q,
            k,
            v,
            output_cotangent_basis,
            softmax_scale=float(softmax_scale),
            causal=causal,
            use_cuda=True,
            kernel_mode=kernel_mode,
        )

    def input_pullback_basis(self, *, backend: Any, cache: Any, output_cotangent_basis: torch.Tensor) -> torch.Tensor:
        """Region input pullback ``[B, P, T, D] -> [B, P, T, D]`` on the GPU.

        The method the reference leaves as the "CUDA kernel target"
        (backends/transformer_cuda.py:45-64); same result as its autograd lowering
        (backends/transformer.py:284-330).  ``backend`` and ``cache`` are the reference's
        ``TransformerRegionBackend`` and ``TransformerRegionCache`` (or objects with the same
        attribute names).
        """
        if output_cotangent_basis.dim() != 4:
            raise ValueError("output_cotangent_basis must have shape [B, P, T, D]")
        return region_input_pullback_basis(backend, cache, output_cotangent_basis, kernel_mode="hip")

    def parameter_vjp(self, *, backend: Any, cache: Any, output_cotangent: torch.Tensor) -> dict[str, torch.Tensor]:
        """Parameter gradients of the region for ``output_cotangent [B, T, D]`` on the GPU, keyed
        like ``backend.named_parameters()`` (reference backends/transformer_cuda.py:66-83 leaves
        this unimplemented; autograd version backends/transformer.py:332-355)."""
        if self.reference_lowering is not None:
            return self.reference_lowering.parameter_vjp(backend=backend, cache=cache, output_cotangent=output_cotangent)
        return region_parameter_vjp(backend, cache, output_cotangent, kernel_mode="hip")

    def parameter_vjp_with_input_cotangent(self, *, backend: Any, cache: Any, output_cotangent: torch.Tensor
                                           ) -> tuple[dict[str, torch.Tensor], torch.Tensor]:
        """``parameter_vjp`` plus the cotangent of the region input ``[B, T, D]`` (fp32) from the same sweep; not
        part of the reference's lowering protocol, used by ``StructuredLocalVJPProvider`` when present."""
        if self.reference_lowering is not None:
            grads = self.reference_lowering.parameter_vjp(backend=backend, cache=cache, output_cotangent=output_cotangent)
            g_in = region_input_pullback_basis(backend, cache, output_cotangent.unsqueeze(1), kernel_mode="hip")[:, 0]
            return grads, g_in
        return region_parameter_vjp_with_input_cotangent(backend, cache, output_cotangent, kernel_mode="hip")
