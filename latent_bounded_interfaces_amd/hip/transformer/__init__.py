"""Transformer attention input-pullback for P cotangent basis directions on the GPU.

Counterpart of reference cuda/transformer/__init__.py: same function name, arguments
and result.  ``q, k, v [B, H, T, Dh]`` and ``output_cotangent_basis [B, P, H, T, Dh]``
give ``(dq, dk, dv)``, each ``[B, P, H, T, Dh]`` in the input dtype; slice ``p`` is the
attention backward for cotangent ``output_cotangent_basis[:, p]``.

All work is done by ``lbi_attn_pullback`` of liblbi_hip.so, which recomputes the
softmax statistics itself (the reference wrapper re-runs a flash forward for them,
cuda/transformer/__init__.py:248-256).  Every ``kernel_mode`` of the reference is
accepted, with its limit on P, and all of them run the same HIP kernels; ``"hip"``
is the unrestricted mode.  There is no torch or CPU execution path here.
"""
from __future__ import annotations

import torch

from ... import _lib

# kernel_mode -> largest basis size the reference accepts for it (None: any).
# reference cuda/transformer/__init__.py:104,165,226-228
_MODE_BASIS_LIMIT = {
    "hip": None,
    "fa2_loop": None,
    "simple": None,
    "fa2_p1": 1,
    "fa2_mma_p1": 1,
    "fa2_mma_pblock4": 4,
}


# what the matrix-core kernels take (the generic kernels take any length and head dim up to 256)
_MFMA_SEQ_MULTIPLE = 64
_MFMA_HEAD_DIMS = (64, 128)
# longest sequence the single-launch kernel takes, by head dim (any length up to it)
_SINGLE_LAUNCH_MAX_SEQ = {64: 256, 128: 128}


def _validate(q, k, v, output_cotangent_basis) -> None:
    # reference cuda/transformer/__init__.py:21-26
    if q.dim() != 4 or k.shape != q.shape or v.shape != q.shape:
        raise ValueError("q, k, and v must have matching shape [B, H, T, Dh]")
    if output_cotangent_basis.dim() != 5:
        raise ValueError("output_cotangent_basis must have shape [B, P, H, T, Dh]")
    if output_cotangent_basis.shape[0] != q.shape[0] or output_cotangent_basis.shape[2:] != q.shape[1:]:
        raise ValueError("output_cotangent_basis must have shape [B, P, H, T, Dh] matching q/k/v")


def attention_input_pullback_basis(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    output_cotangent_basis: torch.Tensor,
    *,
    softmax_scale: float,
    causal: bool = True,
    use_cuda: bool = True,
    kernel_mode: str = "fa2_mma_pblock4",
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """dQ, dK, dV for every basis direction (signature of reference cuda/transformer/__init__.py:279-289)."""
    _validate(q, k, v, output_cotangent_basis)
    if kernel_mode not in _MODE_BASIS_LIMIT:
        raise ValueError(f"unknown attention pullback kernel_mode: {kernel_mode}")
    basis = output_cotangent_basis.shape[1]
    limit = _MODE_BASIS_LIMIT[kernel_mode]
    if limit == 1 and basis != 1:
        raise ValueError(f"kernel_mode='{kernel_mode}' requires output_cotangent_basis.shape[1] == 1")
    if limit == 4 and not 1 <= basis <= 4:
        raise ValueError("kernel_mode='fa2_mma_pblock4' requires 1 <= output_cotangent_basis.shape[1] <= 4")
    if not use_cuda:
        raise RuntimeError(
            "use_cuda=False selects the reference's dense torch formula, which this build does not ship; "
            "only the HIP kernels are available"
        )
    if not q.is_cuda:
        raise RuntimeError("q, k, v must be CUDA tensors (this build has no CPU execution path)")
    if not (k.device == q.device and v.device == q.device and output_cotangent_basis.device == q.device):
        raise RuntimeError("q, k, v and output_cotangent_basis must be on the same device")
    if not (k.dtype == q.dtype and v.dtype == q.dtype and output_cotangent_basis.dtype == q.dtype):
        raise RuntimeError("q, k, v and output_cotangent_basis must have the same dtype")
    dtype = _lib.dtype_code(q.dtype)

    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    d_out = output_cotangent_basis.contiguous()
    bsz, heads, seqlen, head_dim = q.shape
    wide_dim = next((w for w in _MFMA_HEAD_DIMS if w >= head_dim), head_dim)
    single_launch = seqlen <= _SINGLE_LAUNCH_MAX_SEQ.get(wide_dim, 0)
    if q.dtype in (torch.float16, torch.bfloat16) and d_out.numel() and (single_launch or seqlen > _MFMA_SEQ_MULTIPLE // 2):
        # The matrix-core kernels take head dims 64 and 128 and sequence lengths that are multiples of 64 (short
        # sequences, which run as a single launch, any length); everything else runs on the generic kernels, at a
        # small fraction of their speed.  Two paddings are exact:
        # * zero columns appended to the head dim add nothing to any dot product (the scale is passed explicitly)
        #   and receive zero cotangents;
        # * under the causal mask, zero rows appended after the sequence are invisible to every real query, and as
        #   queries they carry a zero cotangent, so they add nothing to dK or dV.
        multiple = 1 if single_launch else _MFMA_SEQ_MULTIPLE
        ragged = seqlen % multiple != 0
        long_seq = seqlen + (multiple - seqlen % multiple) if (ragged and causal) else seqlen
        if (wide_dim != head_dim or long_seq != seqlen) and long_seq % multiple == 0 \
                and wide_dim in _MFMA_HEAD_DIMS:
            pads = (0, wide_dim - head_dim, 0, long_seq - seqlen)
            padded = [torch.nn.functional.pad(t, pads) for t in (q, k, v, d_out)]
            outs = attention_input_pullback_basis(*padded, softmax_scale=softmax_scale, causal=causal,
                                                  use_cuda=use_cuda, kernel_mode="hip")
            return tuple(o[..., :seqlen, :head_dim].contiguous() for o in outs)
    dq = torch.empty_like(d_out)
    dk = torch.empty_like(d_out)
    dv = torch.empty_like(d_out)
    if d_out.numel() == 0:
        return dq, dk, dv
    lib = _lib.load()
    with torch.cuda.device(q.device):
        need = int(lib.lbi_attn_pullback_workspace_bytes(bsz, heads, seqlen, head_dim, basis, dtype))
        # short sequences run as one launch that needs none
        workspace = torch.empty(need, device=q.device, dtype=torch.uint8) if need > 0 else None
        status = lib.lbi_attn_pullback(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), d_out.data_ptr(),
            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
            workspace.data_ptr() if need > 0 else None, need,
            bsz, heads, seqlen, head_dim, basis,
            float(softmax_scale), int(bool(causal)), dtype, _lib.current_stream_ptr(q.device),
        )
    _lib.check(status, "lbi_attn_pullback")
    # The workspace is only used by kernels already queued on this stream; torch's
    # caching allocator reuses it in stream order, so releasing it here is safe.
    return dq, dk, dv


def attention_input_pullback_basis_static(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    output_cotangent_basis: torch.Tensor,
    out: tuple[torch.Tensor, torch.Tensor, torch.Tensor],
    *,
    softmax_scale: float,
    causal: bool = True,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """The same pullback written into caller-provided ``out = (dq, dk, dv)`` with no allocation at all (no
    workspace, no padding, no copies): ``lbi_attn_pullback_static``, whose scratch memory is a static device
    array of ``_lib.ATTN_STATIC_SCRATCH_BYTES`` per GPU.  For callers that cannot allocate (graph capture, serving
    loops).  Every tensor must already be contiguous, on one device and of one dtype; a call whose scratch need
    exceeds the static array raises.  Calls on one GPU share the array and must not overlap in time."""
    _validate(q, k, v, output_cotangent_basis)
    tensors = (q, k, v, output_cotangent_basis, *out)
    if len(out) != 3 or any(o.shape != output_cotangent_basis.shape for o in out):
        raise ValueError("out must be three tensors shaped like output_cotangent_basis")
    if not all(t.is_cuda and t.device == q.device and t.dtype == q.dtype and t.is_contiguous() for t in tensors):
        raise RuntimeError("all tensors must be contiguous CUDA tensors of one dtype on one device")
    if output_cotangent_basis.numel() == 0:
        return out
    bsz, heads, seqlen, head_dim = q.shape
    lib = _lib.load()
    with torch.cuda.device(q.device):
        status = lib.lbi_attn_pullback_static(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), output_cotangent_basis.data_ptr(),
            out[0].data_ptr(), out[1].data_ptr(), out[2].data_ptr(),
            bsz, heads, seqlen, head_dim, output_cotangent_basis.shape[1],
            float(softmax_scale), int(bool(causal)), _lib.dtype_code(q.dtype), _lib.current_stream_ptr(q.device),
        )
    _lib.check(status, "lbi_attn_pullback_static")
    return out


__all__ = ["attention_input_pullback_basis", "attention_input_pullback_basis_static"]
