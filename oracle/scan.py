"""CPU oracle for the interface suffix scan (test infrastructure, not product code).

Convention (reference backward/pullbacks.py:53-64): ``Jt[b, i, j] = d s_out[j] / d s_in[i]``;
cotangents are column vectors and ``g_in = Jt @ g_out``.  The scan returns, for
``mats`` of shape ``[B, K, d, d]``, the tensor ``out`` of shape ``[B, K+1, d, d]`` with
``out[:, r] = mats[:, r] @ mats[:, r+1] @ ... @ mats[:, K-1]`` and ``out[:, K] = I``.
"""
from __future__ import annotations

import numpy as np
import torch


def _check(mats: torch.Tensor) -> tuple[int, int, int]:
    # Contract of reference cuda/interface/__init__.py:12-16.
    if mats.dim() != 4:
        raise ValueError("mats must have shape [B, K, R, R]")
    bsz, count, rank, rank2 = mats.shape
    if rank != rank2:
        raise ValueError("mats must be square in the last two dimensions")
    return bsz, count, rank


def suffix_scan_levels(mats: torch.Tensor) -> torch.Tensor:
    """Log-depth (Hillis-Steele) inclusive suffix scan, the reference's CPU path.

    Restates reference cuda/interface/__init__.py:11-30: at level ``off = 1, 2, 4...``
    every position ``r < K - off`` is replaced by ``prev[r] @ prev[r + off]`` using a
    snapshot of the previous level; the identity is appended last.  Keeps the
    input dtype (reference :27) and does not modify ``mats``.
    """
    bsz, count, rank = _check(mats)
    eye = torch.eye(rank, dtype=mats.dtype)
    if count == 0:
        return eye.expand(bsz, 1, rank, rank).clone()
    cur = mats.clone()
    off = 1
    while off < count:
        snap = cur.clone()
        cur[:, : count - off] = torch.matmul(snap[:, : count - off], snap[:, off:])
        off *= 2
    out = torch.empty((bsz, count + 1, rank, rank), dtype=mats.dtype)
    out[:, :count] = cur
    out[:, count] = eye
    return out


def suffix_scan_sequential(mats: torch.Tensor, dtype: torch.dtype | None = None) -> torch.Tensor:
    """Right-to-left running product, the oracle the reference tests themselves use.

    Restates reference tests/test_interface_scan.py:12-21 (``_manual_suffix``);
    ``dtype`` selects the arithmetic type (fp64 for ground truth).
    """
    bsz, count, rank = _check(mats)
    work = mats if dtype is None else mats.to(dtype)
    out = torch.empty((bsz, count + 1, rank, rank), dtype=work.dtype, device=work.device)
    run = torch.eye(rank, dtype=work.dtype, device=work.device).expand(bsz, rank, rank).clone()
    out[:, count] = run
    for r in range(count - 1, -1, -1):
        run = torch.matmul(work[:, r], run)
        out[:, r] = run
    return out


def suffix_scan_loops(mats) -> np.ndarray:
    """Pure-Python triple loop in exact Python floats (fp64); tiny shapes only.

    Independent of any BLAS / matmul routine: used to pin the two torch
    restatements above.  Follows the definition in reference
    tests/test_interface_scan.py:12-21.
    """
    arr = np.asarray(mats, dtype=np.float64)
    bsz, count, rank, _ = arr.shape
    out = np.zeros((bsz, count + 1, rank, rank), dtype=np.float64)
    for b in range(bsz):
        run = [[1.0 if i == j else 0.0 for j in range(rank)] for i in range(rank)]
        for i in range(rank):
            for j in range(rank):
                out[b, count, i, j] = run[i][j]
        for r in range(count - 1, -1, -1):
            nxt = [[0.0] * rank for _ in range(rank)]
            for i in range(rank):
                for j in range(rank):
                    acc = 0.0
                    for k in range(rank):
                        acc += float(arr[b, r, i, k]) * run[k][j]
                    nxt[i][j] = acc
            run = nxt
            for i in range(rank):
                for j in range(rank):
                    out[b, r, i, j] = run[i][j]
    return out


def suffix_cotangents_sequential(
    mats: torch.Tensor, g: torch.Tensor, dtype: torch.dtype | None = None
) -> torch.Tensor:
    """Cotangent chain ``g_r = Jt_r @ g_{r+1}``, ``g_K = g``; returns ``[B, K+1, d]``.

    Restates the sequential re-check of reference backward/scan.py:63-72, with the
    mat-vec of reference backward/suffix_scan.py:24-38 (``einsum("bij,bj->bi")``).
    """
    bsz, count, rank = _check(mats)
    if g.shape != (bsz, rank):
        raise ValueError("g must have shape [B, d]")
    dt = dtype or torch.promote_types(mats.dtype, g.dtype)
    work = mats.to(dt)
    out = torch.empty((bsz, count + 1, rank), dtype=dt)
    cur = g.to(dt)
    out[:, count] = cur
    for r in range(count - 1, -1, -1):
        cur = torch.einsum("bij,bj->bi", work[:, r], cur)
        out[:, r] = cur
    return out


def suffix_cotangents_from_matrices(suffix: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """Apply every suffix matrix to the terminal cotangent.

    Restates reference backward/suffix_scan.py:41-56: ``g_r = suffix[r] @ g`` for
    ``r < K`` and ``g_K = g``.
    """
    dt = torch.promote_types(suffix.dtype, g.dtype)
    return torch.einsum("bkij,bj->bki", suffix.to(dt), g.to(dt))


# --------------------------------------------------------------------------- inputs

def make_scan_inputs(bsz: int, count: int, rank: int, *, kind: str, seed: int = 0):
    """Synthetic scan inputs on the CPU generator.

    ``kind="randn"``  : ``randn * d^-1/2`` (reference tests/test_interface_scan.py:28-30).
    ``kind="near_identity"`` : ``I + randn * sqrt(0.01/d)``, bounded products (benchmark config).
    Returns ``(mats fp32 [B,K,d,d], g fp32 [B,d])``.
    """
    gen = torch.Generator(device="cpu").manual_seed(seed)
    noise = torch.randn(bsz, count, rank, rank, generator=gen, dtype=torch.float32)
    if kind == "randn":
        mats = noise * (1.0 / max(rank, 1) ** 0.5)
    elif kind == "near_identity":
        mats = torch.eye(rank, dtype=torch.float32) + noise * (0.01 / rank) ** 0.5
    else:
        raise ValueError(f"unknown kind {kind!r}")
    g = torch.randn(bsz, rank, generator=gen, dtype=torch.float32)
    return mats, g
