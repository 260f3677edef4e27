"""CPU oracle for the Transformer attention input-pullback (test infrastructure only).

Shapes: ``q, k, v [B, H, T, Dh]``; ``d_out [B, P, H, T, Dh]`` holds P output
cotangent basis directions; the result is ``(dq, dk, dv)`` each ``[B, P, H, T, Dh]``
where slice ``p`` is the ordinary attention backward for cotangent ``d_out[:, p]``.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def _check(q, k, v, d_out) -> None:
    # Contract of reference cuda/transformer/__init__.py:21-26.
    if q.dim() != 4 or k.shape != q.shape or v.shape != q.shape:
        raise ValueError("q, k, and v must have matching shape [B, H, T, Dh]")
    if d_out.dim() != 5:
        raise ValueError("output_cotangent_basis must have shape [B, P, H, T, Dh]")
    if d_out.shape[0] != q.shape[0] or d_out.shape[2:] != q.shape[1:]:
        raise ValueError("output_cotangent_basis must have shape [B, P, H, T, Dh] matching q/k/v")


def attention_pullback_dense(q, k, v, d_out, *, softmax_scale: float, causal: bool = True,
                             dtype: torch.dtype | None = None):
    """Defining dense formula; materialises ``[B, P, H, T, T]`` so small shapes only.

    Restates reference cuda/transformer/__init__.py:12-41:
    ``P = softmax(scale * Q K^T + mask)``, ``dV = P^T dO``, ``dP = dO V^T``,
    ``delta = sum_j dP * P``, ``dS = P * (dP - delta)``, ``dQ = scale * dS K``,
    ``dK = scale * dS^T Q``.  ``dtype`` selects the arithmetic type.
    """
    _check(q, k, v, d_out)
    if dtype is not None:
        q, k, v, d_out = (t.to(dtype) for t in (q, k, v, d_out))
    seqlen = q.shape[2]
    scores = torch.matmul(q, k.transpose(-1, -2)) * float(softmax_scale)
    if causal:
        keep = torch.ones((seqlen, seqlen), dtype=torch.bool).tril()
        scores = scores.masked_fill(~keep.view(1, 1, seqlen, seqlen), float("-inf"))
    probs = torch.softmax(scores, dim=-1)
    dv = torch.einsum("bhij,bphid->bphjd", probs, d_out)
    d_probs = torch.einsum("bphid,bhjd->bphij", d_out, v)
    row_dot = (d_probs * probs.unsqueeze(1)).sum(dim=-1, keepdim=True)
    d_scores = probs.unsqueeze(1) * (d_probs - row_dot)
    dq = torch.einsum("bphij,bhjd->bphid", d_scores, k) * float(softmax_scale)
    dk = torch.einsum("bphij,bhid->bphjd", d_scores, q) * float(softmax_scale)
    return dq, dk, dv


def attention_pullback_sdpa_loop(q, k, v, d_out, *, softmax_scale: float, causal: bool = True):
    """P independent SDPA forward + autograd backward passes.

    Restates reference cuda/transformer/__init__.py:44-90 and the oracle of the
    reference tests (tests/test_cuda_attention_pullback.py:28-56).  This is what
    the reference runs on the CPU, and for shapes its fused kernels reject.
    """
    _check(q, k, v, d_out)
    dq_cols, dk_cols, dv_cols = [], [], []
    for p in range(d_out.shape[1]):
        q_r = q.detach().clone().requires_grad_(True)
        k_r = k.detach().clone().requires_grad_(True)
        v_r = v.detach().clone().requires_grad_(True)
        out = F.scaled_dot_product_attention(
            q_r, k_r, v_r, attn_mask=None, dropout_p=0.0, is_causal=causal, scale=float(softmax_scale)
        )
        dq, dk, dv = torch.autograd.grad(out, (q_r, k_r, v_r), grad_outputs=d_out[:, p])
        dq_cols.append(dq.unsqueeze(1))
        dk_cols.append(dk.unsqueeze(1))
        dv_cols.append(dv.unsqueeze(1))
    return torch.cat(dq_cols, 1), torch.cat(dk_cols, 1), torch.cat(dv_cols, 1)


def attention_forward_dense(q, k, v, *, softmax_scale: float, causal: bool = True):
    """Plain attention forward, returning ``(out, logsumexp)``; used by finite-difference checks."""
    seqlen = q.shape[2]
    scores = torch.matmul(q, k.transpose(-1, -2)) * float(softmax_scale)
    if causal:
        keep = torch.ones((seqlen, seqlen), dtype=torch.bool).tril()
        scores = scores.masked_fill(~keep.view(1, 1, seqlen, seqlen), float("-inf"))
    lse = torch.logsumexp(scores, dim=-1)
    return torch.matmul(torch.softmax(scores, dim=-1), v), lse


def attention_pullback_blocked(q, k, v, d_out, *, softmax_scale: float, causal: bool = True,
                               block: int = 256, dtype: torch.dtype = torch.float32):
    """Dense formula evaluated one query block at a time (bounded memory, any T).

    Same arithmetic as ``attention_pullback_dense`` (reference
    cuda/transformer/__init__.py:12-41) in ``dtype``; rows of the softmax are
    independent, so processing ``block`` queries at once changes nothing but the
    peak memory (``B*P*H*block*T`` instead of ``B*P*H*T*T``).
    """
    _check(q, k, v, d_out)
    qf, kf, vf, gf = (t.to(dtype) for t in (q, k, v, d_out))
    seqlen = q.shape[2]
    dq = torch.zeros_like(gf)
    dk = torch.zeros_like(gf)
    dv = torch.zeros_like(gf)
    for start in range(0, seqlen, block):
        stop = min(seqlen, start + block)
        hi = stop if causal else seqlen
        scores = torch.matmul(qf[:, :, start:stop], kf[:, :, :hi].transpose(-1, -2)) * float(softmax_scale)
        if causal:
            rows = torch.arange(start, stop).view(-1, 1)
            cols = torch.arange(hi).view(1, -1)
            scores = scores.masked_fill((cols > rows).view(1, 1, stop - start, hi), float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        g_blk = gf[:, :, :, start:stop]
        dv[:, :, :, :hi] += torch.einsum("bhij,bphid->bphjd", probs, g_blk)
        d_probs = torch.einsum("bphid,bhjd->bphij", g_blk, vf[:, :, :hi])
        row_dot = (d_probs * probs.unsqueeze(1)).sum(dim=-1, keepdim=True)
        d_scores = probs.unsqueeze(1) * (d_probs - row_dot)
        dq[:, :, :, start:stop] = torch.einsum("bphij,bhjd->bphid", d_scores, kf[:, :, :hi]) * float(softmax_scale)
        dk[:, :, :, :hi] += torch.einsum("bphij,bhid->bphjd", d_scores, qf[:, :, start:stop]) * float(softmax_scale)
    return dq, dk, dv


def make_attention_inputs(bsz: int, heads: int, seqlen: int, head_dim: int, basis: int, *,
                          dtype: torch.dtype = torch.float32, seed: int = 0):
    """``q, k, v, d_out ~ N(0, 1)`` on the CPU generator, rounded to ``dtype``.

    Same distribution as reference benchmarks/time_attention_pullback.py:270-284.
    """
    gen = torch.Generator(device="cpu").manual_seed(seed)
    shape = (bsz, heads, seqlen, head_dim)
    q = torch.randn(shape, generator=gen, dtype=torch.float32).to(dtype)
    k = torch.randn(shape, generator=gen, dtype=torch.float32).to(dtype)
    v = torch.randn(shape, generator=gen, dtype=torch.float32).to(dtype)
    d_out = torch.randn((bsz, basis, heads, seqlen, head_dim), generator=gen, dtype=torch.float32).to(dtype)
    return q, k, v, d_out
