"""Suffix scan of interface pullback matrices on the GPU.

Counterpart of reference cuda/interface/__init__.py: same function name, argument
and result (``[B, K, d, d] -> [B, K+1, d, d]``, fp32 result as the native
reference extension returns, cuda/interface/suffix_scan.cu:76,110).  The work is
done by ``lbi_suffix_scan`` / ``lbi_suffix_cotangents`` of liblbi_hip.so.
"""
from __future__ import annotations

import torch

from ... import _lib


def _validate(mats: torch.Tensor) -> tuple[int, int, int]:
    # Same contract and messages as reference cuda/interface/__init__.py:12-16 and
    # cuda/interface/suffix_scan.cu:8-17.
    if not isinstance(mats, torch.Tensor):
        raise TypeError("mats must be a torch.Tensor")
    if mats.dim() != 4:
        raise ValueError("mats must have shape [B, K, R, R]")
    bsz, count, rank, rank2 = mats.shape
    if rank != rank2:
        raise ValueError("mats must be square in the last two dimensions")
    if not mats.is_cuda:
        raise RuntimeError("mats must be a CUDA tensor (this build has no CPU execution path)")
    if mats.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        raise RuntimeError("mats must have float, half, or bfloat16 dtype")
    return bsz, count, rank


#: interface widths the matrix-core scan kernels are built for
_MFMA_WIDTHS = (32, 64, 128, 256, 512)


def _padded_width(rank: int) -> int:
    """The matrix-core width a scan of ``rank x rank`` matrices is padded to, or ``rank`` itself when it is one
    already, too small to matter (<= 16) or beyond the largest."""
    if rank <= 16 or rank in _MFMA_WIDTHS:
        return rank
    return next((w for w in _MFMA_WIDTHS if w > rank), rank)


def suffix_scan_pullbacks(mats: torch.Tensor, *, exact_suffix: bool = False) -> torch.Tensor:
    """``out[:, r] = mats[:, r] @ ... @ mats[:, K-1]``, ``out[:, K] = I``; fp32, input untouched.

    ``exact_suffix`` matters for bf16 storage at d = 256 only, whose products run on the 16-bit matrix cores with the
    running suffix as a sum of bf16 planes: by default two planes (the suffix operand rounded to 16 significand bits,
    error <= 2e-4 where 16-bit storage is asked 2e-2), with ``exact_suffix=True`` three (its exact fp32 value: only
    the rounding of fp32 accumulation is left, ~1e-5 at K = 128; half again as many products)."""
    bsz, count, rank = _validate(mats)
    width = _padded_width(rank)
    if width != rank and mats.numel():
        # Products of zero-padded matrices are the zero-padded products, and the identity tail cuts to the
        # identity: run the matrix-core kernel of the next width instead of the scalar kernel (several times
        # faster even with the extra bytes).
        pad = width - rank
        wide = suffix_scan_pullbacks(torch.nn.functional.pad(mats, (0, pad, 0, pad)), exact_suffix=exact_suffix)
        return wide[:, :, :rank, :rank].contiguous()
    mats = mats.contiguous()
    out = torch.empty((bsz, count + 1, rank, rank), device=mats.device, dtype=torch.float32)
    if out.numel() == 0:
        return out
    lib = _lib.load()
    with torch.cuda.device(mats.device):
        status = lib.lbi_suffix_scan_ex(
            mats.data_ptr(), None, out.data_ptr(), None, bsz, count, rank, _lib.dtype_code(mats.dtype), _lib.LBI_F32,
            _lib.LBI_SCAN_EXACT_SUFFIX if exact_suffix else 0, _lib.current_stream_ptr(mats.device),
        )
    _lib.check(status, "lbi_suffix_scan_ex")
    return out


def suffix_scan_cotangents(mats: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """Cotangent-only chain: ``out[:, K] = g``, ``out[:, r] = mats[:, r] @ out[:, r+1]``.

    Returns ``[B, K+1, d]`` fp32 without forming any ``d x d`` product.  Equals
    ``suffix_scan_pullbacks(mats) @ g`` (reference backward/suffix_scan.py:41-56).
    """
    bsz, count, rank = _validate(mats)
    if g.dim() != 2 or g.shape[0] != bsz or g.shape[1] != rank:
        raise ValueError("g must have shape [B, R]")
    mats = mats.contiguous()
    g32 = g.to(device=mats.device, dtype=torch.float32).contiguous()
    out = torch.empty((bsz, count + 1, rank), device=mats.device, dtype=torch.float32)
    if out.numel() == 0:
        return out
    lib = _lib.load()
    with torch.cuda.device(mats.device):
        status = lib.lbi_suffix_cotangents(
            mats.data_ptr(), g32.data_ptr(), out.data_ptr(), bsz, count, rank,
            _lib.dtype_code(mats.dtype), _lib.current_stream_ptr(mats.device),
        )
    _lib.check(status, "lbi_suffix_cotangents")
    return out


def suffix_scan_pullbacks_and_cotangents(mats: torch.Tensor, g: torch.Tensor, *,
                                         exact_suffix: bool = False) -> tuple[torch.Tensor, torch.Tensor]:
    """Both results of the two functions above from one pass over ``mats`` (one kernel
    for d in {32, 64, 128, 256}): ``(suffix [B, K+1, d, d], cotangents [B, K+1, d])``, fp32.
    ``exact_suffix``: see :func:`suffix_scan_pullbacks`."""
    bsz, count, rank = _validate(mats)
    if g.dim() != 2 or g.shape[0] != bsz or g.shape[1] != rank:
        raise ValueError("g must have shape [B, R]")
    width = _padded_width(rank)
    if width != rank and mats.numel():
        pad = width - rank  # see suffix_scan_pullbacks; a zero-padded g leaves the first `rank` cotangents unchanged
        wide, wide_cot = suffix_scan_pullbacks_and_cotangents(torch.nn.functional.pad(mats, (0, pad, 0, pad)),
                                                              torch.nn.functional.pad(g, (0, pad)),
                                                              exact_suffix=exact_suffix)
        return wide[:, :, :rank, :rank].contiguous(), wide_cot[:, :, :rank].contiguous()
    mats = mats.contiguous()
    g32 = g.to(device=mats.device, dtype=torch.float32).contiguous()
    out = torch.empty((bsz, count + 1, rank, rank), device=mats.device, dtype=torch.float32)
    cot = torch.empty((bsz, count + 1, rank), device=mats.device, dtype=torch.float32)
    if out.numel() == 0:
        return out, cot
    lib = _lib.load()
    with torch.cuda.device(mats.device):
        status = lib.lbi_suffix_scan_ex(
            mats.data_ptr(), g32.data_ptr(), out.data_ptr(), cot.data_ptr(), bsz, count, rank,
            _lib.dtype_code(mats.dtype), _lib.LBI_F32, _lib.LBI_SCAN_EXACT_SUFFIX if exact_suffix else 0,
            _lib.current_stream_ptr(mats.device),
        )
    _lib.check(status, "lbi_suffix_scan_ex")
    return out, cot


def suffix_apply(suffix: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """``out[b, r] = suffix[b, r] @ g[b]`` for every matrix of ``suffix [B, M, d, d]`` (fp32, as the scan returns
    it; other float types are converted) in one launch: the mat-vecs of reference backward/suffix_scan.py:49-53."""
    if not isinstance(suffix, torch.Tensor) or suffix.dim() != 4 or suffix.shape[-1] != suffix.shape[-2]:
        raise ValueError("suffix must have shape [B, M, R, R]")
    bsz, count, rank, _ = suffix.shape
    if g.dim() != 2 or g.shape[0] != bsz or g.shape[1] != rank:
        raise ValueError("g must have shape [B, R]")
    if not suffix.is_cuda:
        raise RuntimeError("suffix must be a CUDA tensor (this build has no CPU execution path)")
    suffix = suffix.to(torch.float32).contiguous()
    g32 = g.to(device=suffix.device, dtype=torch.float32).contiguous()
    out = torch.empty((bsz, count, rank), device=suffix.device, dtype=torch.float32)
    if out.numel() == 0:
        return out
    lib = _lib.load()
    with torch.cuda.device(suffix.device):
        status = lib.lbi_suffix_apply(suffix.data_ptr(), g32.data_ptr(), out.data_ptr(), bsz, count, rank,
                                      _lib.current_stream_ptr(suffix.device))
    _lib.check(status, "lbi_suffix_apply")
    return out


def matrix_norms(mats: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``(spectral, frobenius)`` norms, fp32, of every square matrix of ``mats [..., d, d]``.

    What reference backward/suffix_scan.py:117-118 and :126 get from ``torch.linalg.matrix_norm``
    (``ord=2`` runs a singular value decomposition per matrix); here one ``lbi_matrix_norms`` launch
    (repeated squaring of ``A^T A``, no decomposition).
    """
    if not isinstance(mats, torch.Tensor):
        raise TypeError("mats must be a torch.Tensor")
    if mats.dim() < 2 or mats.shape[-1] != mats.shape[-2]:
        raise ValueError("mats must be square in the last two dimensions")
    if not mats.is_cuda:
        raise RuntimeError("mats must be a CUDA tensor (this build has no CPU execution path)")
    if mats.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        raise RuntimeError("mats must have float, half, or bfloat16 dtype")
    batch_shape = mats.shape[:-2]
    rank = int(mats.shape[-1])
    mats = mats.contiguous()
    count = mats.numel() // (rank * rank) if rank else 0
    spectral = torch.empty(batch_shape, device=mats.device, dtype=torch.float32)
    frobenius = torch.empty(batch_shape, device=mats.device, dtype=torch.float32)
    if count == 0:
        return spectral, frobenius
    lib = _lib.load()
    need = int(lib.lbi_matrix_norms_workspace_bytes(count, rank))
    workspace = torch.empty(max(need, 16), device=mats.device, dtype=torch.uint8)
    with torch.cuda.device(mats.device):
        status = lib.lbi_matrix_norms(
            mats.data_ptr(), spectral.data_ptr(), frobenius.data_ptr(), workspace.data_ptr(), workspace.numel(),
            count, rank, _lib.dtype_code(mats.dtype), _lib.current_stream_ptr(mats.device),
        )
    _lib.check(status, "lbi_matrix_norms")
    return spectral, frobenius


__all__ = ["matrix_norms", "suffix_apply", "suffix_scan_pullbacks", "suffix_scan_cotangents",
           "suffix_scan_pullbacks_and_cotangents"]
