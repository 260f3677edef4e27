"""Region-level input pullback of a Transformer layer range for P cotangent directions.

Implements ``TransformerLowering.input_pullback_basis`` of the reference
(backends/transformer.py:64-75; the CUDA class leaves it as a stub,
backends/transformer_cuda.py:45-64) for the block the reference's backend executes
(backends/transformer.py:118-246):

    res1 = hidden (+ residual);  a = out_proj(attention(rope(split(conv1d(in_proj(norm(res1)))))))
    res2 = a + res1;             m = fc2(up * silu(gate)),  [up | gate] = fc1(norm2(res2))
    region_output = m + res2 of the last layer

The cotangent basis [B, P, T, D] is pulled back through the layers in reverse.  Matrix
products are library GEMMs on the [B*P*T, *] cotangent rows; everything between them runs in
the kernels of liblbi_hip.so (RMSNorm, gated MLP, head split, rotary embedding + KV-group
sum, causal convolution, and the attention pullback itself).  The residual-stream cotangent
is kept in fp32, branch cotangents in the dtype of the weights.  Inputs are read from the
forward cache the backend recorded; nothing is recomputed except the softmax statistics
inside the attention kernel.  GPU only.
"""
from __future__ import annotations

import math
from typing import Any

import torch

from ... import _lib
from . import attention_input_pullback_basis


def _stream(t: torch.Tensor) -> int:
    return _lib.current_stream_ptr(t.device)


def _require_cuda(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("region pullback tensors must be CUDA tensors (this build has no CPU execution path)")


def rmsnorm_pullback(g_out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float,
                     g_residual: torch.Tensor | None, *, want_branch: bool,
                     keep_residual: bool = False) -> tuple[torch.Tensor, torch.Tensor | None]:
    """``g_out [B,P,T,D]`` through RMSNorm at input ``x [B,T,D]``, plus ``g_residual`` (fp32).

    Returns ``(sum fp32, sum in g_out.dtype or None)``.  ``g_residual [B,P,T,D]`` is overwritten with the
    sum unless ``keep_residual``; ``g_residual [B,P,1,D]`` (the same cotangent at every position) is read only.
    """
    _require_cuda(g_out, x, weight)
    bsz, basis, seqlen, dim = g_out.shape
    if x.shape != (bsz, seqlen, dim) or weight.shape != (dim,):
        raise ValueError("rmsnorm_pullback: x must be [B, T, D] and weight [D] matching g_out [B, P, T, D]")
    g_out, x, weight = g_out.contiguous(), x.contiguous(), weight.to(g_out.dtype).contiguous()
    shared = 0
    if g_residual is None:
        total = torch.empty(g_out.shape, device=g_out.device, dtype=torch.float32)
        res_ptr = None
    else:
        if g_residual.dtype != torch.float32 or not g_residual.is_contiguous():
            raise ValueError("rmsnorm_pullback: g_residual must be a contiguous fp32 tensor")
        if g_residual.shape == g_out.shape:
            total = torch.empty_like(g_residual) if keep_residual else g_residual
        elif g_residual.shape == (bsz, basis, 1, dim):
            total = torch.empty(g_out.shape, device=g_out.device, dtype=torch.float32)
            shared = 1
        else:
            raise ValueError("rmsnorm_pullback: g_residual must be shaped like g_out, or [B, P, 1, D]")
        res_ptr = g_residual.data_ptr()
    branch = torch.empty_like(g_out) if want_branch else None
    with torch.cuda.device(g_out.device):
        status = _lib.load().lbi_rmsnorm_pullback(
            g_out.data_ptr(), x.data_ptr(), weight.data_ptr(), res_ptr, total.data_ptr(),
            branch.data_ptr() if branch is not None else None, bsz, basis, seqlen, dim, float(eps), shared,
            _lib.dtype_code(g_out.dtype), _lib.dtype_code(x.dtype), _stream(g_out))
    _lib.check(status, "lbi_rmsnorm_pullback")
    return total, branch


def gated_mlp_pullback(g_down_input: torch.Tensor, fc1_output: torch.Tensor) -> torch.Tensor:
    """``g_down_input [B,P,T,Hd]`` (or ``[B,P,1,Hd]``: the same at every position), ``fc1_output [B,T,2Hd]``
    -> cotangent of fc1_output ``[B,P,T,2Hd]``."""
    _require_cuda(g_down_input, fc1_output)
    bsz, basis, g_len, hidden = g_down_input.shape
    if fc1_output.dim() != 3 or fc1_output.shape[0] != bsz or fc1_output.shape[2] != 2 * hidden \
            or fc1_output.dtype != g_down_input.dtype:
        raise ValueError("gated_mlp_pullback: fc1_output must be [B, T, 2*hidden] in the dtype of g_down_input")
    seqlen = int(fc1_output.shape[1])
    if g_len != seqlen and g_len != 1:
        raise ValueError("gated_mlp_pullback: g_down_input must be [B, P, T, hidden] or [B, P, 1, hidden]")
    shared = int(g_len == 1 and seqlen != 1)
    g_down_input, fc1_output = g_down_input.contiguous(), fc1_output.contiguous()
    out = torch.empty((bsz, basis, seqlen, 2 * hidden), device=g_down_input.device, dtype=g_down_input.dtype)
    with torch.cuda.device(out.device):
        status = _lib.load().lbi_gated_mlp_pullback(
            g_down_input.data_ptr(), fc1_output.data_ptr(), out.data_ptr(), bsz, basis, seqlen, hidden, shared,
            _lib.dtype_code(out.dtype), _stream(out))
    _lib.check(status, "lbi_gated_mlp_pullback")
    return out


def attn_heads_split(g_merged: torch.Tensor, n_heads: int, head_dim: int) -> torch.Tensor:
    """``[B,P,T,H*Dh]`` -> ``[B,P,H,T,Dh]``."""
    _require_cuda(g_merged)
    bsz, basis, seqlen, width = g_merged.shape
    if width != n_heads * head_dim:
        raise ValueError("attn_heads_split: last dimension must be n_heads * head_dim")
    g_merged = g_merged.contiguous()
    out = torch.empty((bsz, basis, n_heads, seqlen, head_dim), device=g_merged.device, dtype=g_merged.dtype)
    with torch.cuda.device(out.device):
        status = _lib.load().lbi_attn_heads_split(g_merged.data_ptr(), out.data_ptr(), bsz, basis, seqlen, n_heads,
                                                  head_dim, _lib.dtype_code(out.dtype), _stream(out))
    _lib.check(status, "lbi_attn_heads_split")
    return out


_ROPE_TABLES: dict[tuple, tuple[torch.Tensor, torch.Tensor]] = {}


def rope_tables(seq_len: int, head_dim: int, base: float, device: torch.device) -> tuple[torch.Tensor, torch.Tensor]:
    """cos, sin ``[T, Dh/2]`` fp32 of the rotary angles, built as the reference's apply_rope does
    (backbones/transformer/rope.py:14-20) and cached per (T, Dh, base, device)."""
    key = (seq_len, head_dim, float(base), str(device))
    hit = _ROPE_TABLES.get(key)
    if hit is None:
        half = head_dim // 2
        positions = torch.arange(seq_len, device=device, dtype=torch.float32)
        freq_seq = torch.arange(half, device=device, dtype=torch.float32)
        freqs = torch.outer(positions, base ** (-2.0 * freq_seq / float(head_dim)))
        hit = (freqs.cos().contiguous(), freqs.sin().contiguous())
        if len(_ROPE_TABLES) > 32:
            _ROPE_TABLES.clear()
        _ROPE_TABLES[key] = hit
    return hit


def attn_qkv_pullback(dq: torch.Tensor, dk: torch.Tensor, dv: torch.Tensor, *, n_kv_heads: int, rope_base: float,
                      rope_interleaved: bool) -> torch.Tensor:
    """``dq, dk, dv [B,P,H,T,Dh]`` -> cotangent of the packed projection ``[B,P,T,(H+2Hkv)*Dh]``."""
    _require_cuda(dq, dk, dv)
    bsz, basis, heads, seqlen, head_dim = dq.shape
    if dk.shape != dq.shape or dv.shape != dq.shape or dk.dtype != dq.dtype or dv.dtype != dq.dtype:
        raise ValueError("attn_qkv_pullback: dq, dk, dv must share shape [B, P, H, T, Dh] and dtype")
    if heads % n_kv_heads:
        raise ValueError("n_heads must be divisible by n_kv_heads")
    if head_dim % 2:
        raise ValueError("RoPE requires an even head dimension.")
    dq, dk, dv = dq.contiguous(), dk.contiguous(), dv.contiguous()
    cos, sin = rope_tables(seqlen, head_dim, rope_base, dq.device)
    out = torch.empty((bsz, basis, seqlen, (heads + 2 * n_kv_heads) * head_dim), device=dq.device, dtype=dq.dtype)
    with torch.cuda.device(out.device):
        status = _lib.load().lbi_attn_qkv_pullback(
            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), cos.data_ptr(), sin.data_ptr(), out.data_ptr(), bsz, basis,
            seqlen, heads, n_kv_heads, head_dim, int(bool(rope_interleaved)), _lib.dtype_code(out.dtype), _stream(out))
    _lib.check(status, "lbi_attn_qkv_pullback")
    return out


def causal_conv1d_pullback(g_out: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``g_out [B,P,T,C]`` through the depthwise causal convolution with ``weight [C,1,k]``."""
    _require_cuda(g_out, weight)
    bsz, basis, seqlen, channels = g_out.shape
    if weight.dim() != 3 or weight.shape[0] != channels or weight.shape[1] != 1:
        raise ValueError("causal_conv1d_pullback: weight must be [C, 1, k] (depthwise)")
    g_out = g_out.contiguous()
    weight = weight.to(g_out.dtype).contiguous()
    out = torch.empty_like(g_out)
    with torch.cuda.device(out.device):
        status = _lib.load().lbi_causal_conv1d_pullback(g_out.data_ptr(), weight.data_ptr(), out.data_ptr(),
                                                        bsz * basis, seqlen, channels, weight.shape[-1],
                                                        _lib.dtype_code(out.dtype), _stream(out))
    _lib.check(status, "lbi_causal_conv1d_pullback")
    return out


#: longest convolution filter the one-pass projection + convolution pullback takes
FUSED_CONV_MAX_TAPS = 8


def attn_qkv_conv_pullback(dq: torch.Tensor, dk: torch.Tensor, dv: torch.Tensor, conv_weight: torch.Tensor, *,
                           n_kv_heads: int, rope_base: float, rope_interleaved: bool) -> torch.Tensor:
    """:func:`attn_qkv_pullback` then :func:`causal_conv1d_pullback` in one pass over ``dq, dk, dv``
    (same arithmetic as the two calls, bit-identical in fp32; filters of at most ``FUSED_CONV_MAX_TAPS`` taps)."""
    _require_cuda(dq, dk, dv, conv_weight)
    bsz, basis, heads, seqlen, head_dim = dq.shape
    if dk.shape != dq.shape or dv.shape != dq.shape or dk.dtype != dq.dtype or dv.dtype != dq.dtype:
        raise ValueError("attn_qkv_conv_pullback: dq, dk, dv must share shape [B, P, H, T, Dh] and dtype")
    if heads % n_kv_heads:
        raise ValueError("n_heads must be divisible by n_kv_heads")
    if head_dim % 2:
        raise ValueError("RoPE requires an even head dimension.")
    channels = (heads + 2 * n_kv_heads) * head_dim
    if conv_weight.dim() != 3 or conv_weight.shape[0] != channels or conv_weight.shape[1] != 1:
        raise ValueError("attn_qkv_conv_pullback: weight must be [C, 1, k] (depthwise) with C = (H + 2 Hkv) Dh")
    dq, dk, dv = dq.contiguous(), dk.contiguous(), dv.contiguous()
    weight = conv_weight.to(dq.dtype).contiguous()
    cos, sin = rope_tables(seqlen, head_dim, rope_base, dq.device)
    out = torch.empty((bsz, basis, seqlen, channels), device=dq.device, dtype=dq.dtype)
    with torch.cuda.device(out.device):
        status = _lib.load().lbi_attn_qkv_conv_pullback(
            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), cos.data_ptr(), sin.data_ptr(), weight.data_ptr(),
            out.data_ptr(), bsz, basis, seqlen, heads, n_kv_heads, head_dim, int(bool(rope_interleaved)),
            weight.shape[-1], _lib.dtype_code(out.dtype), _stream(out))
    _lib.check(status, "lbi_attn_qkv_conv_pullback")
    return out


#: widest RMSNorm and longest convolution filter the parameter-gradient kernels take
NORM_GRAD_MAX_WIDTH = 2048
CONV_GRAD_MAX_TAPS = 8


def rmsnorm_weight_grad(g_out: torch.Tensor, x: torch.Tensor, eps: float) -> torch.Tensor:
    """Gradient of an RMSNorm weight, fp32 ``[D]``: ``g_out [..., D]`` (in the weight dtype) summed over all rows
    against the normalised input, with ``x [..., D]`` (weight dtype or fp32) rounded to the weight dtype first and
    the normalised value rounded again, as the forward does (reference backbones/transformer/block.py:18-23)."""
    _require_cuda(g_out, x)
    width = g_out.shape[-1]
    if x.shape[-1] != width or x.numel() != g_out.numel():
        raise ValueError("rmsnorm_weight_grad: g_out and x must hold the same rows of the same width")
    if x.dtype not in (g_out.dtype, torch.float32):
        raise ValueError("rmsnorm_weight_grad: x must be in the dtype of g_out or fp32")
    g_out, x = g_out.contiguous(), x.contiguous()
    rows = g_out.numel() // width
    out = torch.empty(width, device=g_out.device, dtype=torch.float32)
    lib = _lib.load()
    with torch.cuda.device(out.device):
        need = int(lib.lbi_rmsnorm_weight_grad_workspace_bytes(rows, width))
        workspace = torch.empty(max(need, 16), device=out.device, dtype=torch.uint8)
        status = lib.lbi_rmsnorm_weight_grad(g_out.data_ptr(), x.data_ptr(), out.data_ptr(), workspace.data_ptr(),
                                             workspace.numel(), rows, width, float(eps), _lib.dtype_code(g_out.dtype),
                                             _lib.dtype_code(x.dtype), _stream(out))
    _lib.check(status, "lbi_rmsnorm_weight_grad")
    return out


def causal_conv1d_weight_grad(g_out: torch.Tensor, x: torch.Tensor, ksize: int) -> tuple[torch.Tensor, torch.Tensor]:
    """Weight ``[C, 1, k]`` and bias ``[C]`` gradients (fp32) of the depthwise causal convolution for
    ``g_out, x [B, T, C]``: ``g_w[c, 0, j] = sum_{b, t} g_out[b, t, c] x[b, t - (k-1-j), c]``."""
    _require_cuda(g_out, x)
    if g_out.dim() != 3 or x.shape != g_out.shape or x.dtype != g_out.dtype:
        raise ValueError("causal_conv1d_weight_grad: g_out and x must share shape [B, T, C] and dtype")
    bsz, seqlen, channels = g_out.shape
    g_out, x = g_out.contiguous(), x.contiguous()
    out = torch.empty(channels * ksize + channels, device=g_out.device, dtype=torch.float32)
    lib = _lib.load()
    with torch.cuda.device(out.device):
        need = int(lib.lbi_causal_conv1d_weight_grad_workspace_bytes(bsz, seqlen, channels, ksize))
        workspace = torch.empty(max(need, 16), device=out.device, dtype=torch.uint8)
        status = lib.lbi_causal_conv1d_weight_grad(g_out.data_ptr(), x.data_ptr(), out.data_ptr(), workspace.data_ptr(),
                                                   workspace.numel(), bsz, seqlen, channels, ksize,
                                                   _lib.dtype_code(g_out.dtype), _stream(out))
    _lib.check(status, "lbi_causal_conv1d_weight_grad")
    return out[:channels * ksize].view(channels, 1, ksize), out[channels * ksize:]


#: rows below which the transposed copy of the weight costs more than the faster product form gains
_TRANSPOSED_COPY_MIN_ROWS = 65536


def _apply_transposed(g: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``g @ weight`` for ``weight [out, in]``: the pullback of ``y = x weight^T``.  For tall ``g`` it is issued as
    the library's ``A B^T`` form on a transposed copy of the (small) weight, which is its faster path for these
    products; for few rows (the single direction of a parameter VJP) the copy is not worth it."""
    if weight.dtype != g.dtype:
        # a forward run under autocast multiplied by the weight cast to the compute dtype; so does its pullback
        weight = weight.to(g.dtype)
    if g.numel() // g.shape[-1] < _TRANSPOSED_COPY_MIN_ROWS:
        return torch.matmul(g, weight)
    return torch.nn.functional.linear(g, weight.t().contiguous())


def _rows(t: torch.Tensor) -> torch.Tensor:
    return t.reshape(-1, t.shape[-1])


def _linear_grads(sink: dict, linear: Any, g_out: torch.Tensor, x: torch.Tensor) -> None:
    """Weight (and bias) gradient of ``y = x W^T + b`` for the single direction in ``g_out [B,1,T,O]``."""
    g2 = _rows(g_out)
    sink[id(linear.weight)] = torch.matmul(g2.t(), _rows(x).to(g2.dtype)).to(linear.weight.dtype)
    bias = getattr(linear, "bias", None)
    if bias is not None:
        sink[id(bias)] = g2.float().sum(dim=0).to(bias.dtype)


def _norm_weight_grad(sink: dict, norm: Any, g_out: torch.Tensor, x: torch.Tensor) -> None:
    """Gradient of the RMSNorm weight: sum over rows of g_out o normalised(x), with x rounded to
    the weight dtype first and the normalised value rounded again, as the forward does
    (reference backbones/transformer/block.py:18-23)."""
    wdtype = norm.weight.dtype
    width = x.shape[-1]
    if g_out.dtype == wdtype and x.dtype in (wdtype, torch.float32) and width % 4 == 0 and width <= NORM_GRAD_MAX_WIDTH:
        sink[id(norm.weight)] = rmsnorm_weight_grad(g_out, x, norm.eps).to(wdtype)
        return
    # widths the kernel does not take: the same sum with torch operations on the device
    xf = x.to(wdtype).float()
    normed = (xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + norm.eps)).to(wdtype).float()
    sink[id(norm.weight)] = (_rows(g_out).float() * _rows(normed)).sum(dim=0).to(wdtype)


def _conv_grads(sink: dict, conv: Any, g_out: torch.Tensor, x_pre: torch.Tensor) -> None:
    """Depthwise causal convolution: g_w[c, j] = sum_{b,t} g_out[b,t,c] x_pre[b, t + j - (k-1), c]."""
    ksize = conv.weight.shape[-1]
    if ksize <= CONV_GRAD_MAX_TAPS and x_pre.dtype == g_out.dtype:
        g_weight, g_bias = causal_conv1d_weight_grad(g_out[:, 0], x_pre, ksize)
        sink[id(conv.weight)] = g_weight.to(conv.weight.dtype)
        if getattr(conv, "bias", None) is not None:
            sink[id(conv.bias)] = g_bias.to(conv.bias.dtype)
        return
    # longer filters: the same sums with torch operations on the device
    g = g_out[:, 0].float()
    x = x_pre.float()
    seqlen = g.shape[1]
    cols = []
    for j in range(ksize):
        shift = ksize - 1 - j
        if shift >= seqlen:
            cols.append(torch.zeros(g.shape[-1], device=g.device))
        else:
            cols.append((g[:, shift:] * x[:, :seqlen - shift]).sum(dim=(0, 1)))
    sink[id(conv.weight)] = torch.stack(cols, dim=-1).unsqueeze(1).to(conv.weight.dtype)
    if getattr(conv, "bias", None) is not None:
        sink[id(conv.bias)] = g.sum(dim=(0, 1)).to(conv.bias.dtype)


def _layer_input_pullback(block: Any, layer_cache: Any, g_hidden: torch.Tensor | None, g_residual: torch.Tensor,
                          kernel_mode: str, want_branch: bool, param_grads: dict | None = None,
                          keep_residual: bool = False) -> tuple[torch.Tensor, torch.Tensor | None]:
    """One block, backwards.  ``g_residual`` (fp32, [B,P,T,D]) is the cotangent of the block's
    residual output and is updated in place (``[B,P,1,D]``: the same at every position, read only; with
    ``keep_residual`` a full-size one is left untouched too);
    ``g_hidden`` is the cotangent of its hidden output
    in the weight dtype (``None``: equal to ``g_residual``).  Returns the cotangent of
    ``hidden (+ residual)`` at the block input in fp32 and, if ``want_branch``, also rounded to
    the weight dtype (the ``g_hidden`` of the block before).

    With ``param_grads`` (a dict filled as ``id(parameter) -> gradient``; P must be 1) the
    parameter gradients of the block are formed on the way, each from the cotangent at the
    output of its module and the cached input of that module."""
    attn, mlp = block.attn, block.mlp
    a_cache, m_cache = layer_cache.attention, layer_cache.mlp
    # Branch cotangents live in the dtype the forward's matrix products ran in, which is what the cached
    # attention operands have: the weights' own dtype, or the autocast dtype of a mixed-precision forward
    # (fp32 master weights, 16-bit products; reference train/runners.py:361), whose weights are cast per use.
    wdtype = a_cache.q_rope.dtype
    if g_hidden is None:
        g_hidden = g_residual.to(wdtype)

    # gated MLP: hidden_out = fc2(up * silu(gate)), [up | gate] = fc1(norm2(res2))
    if param_grads is not None:
        _linear_grads(param_grads, mlp.fc2, g_hidden, m_cache.down_input)
    g_down_input = _apply_transposed(g_hidden, mlp.fc2.weight)
    g_fc1 = gated_mlp_pullback(g_down_input, m_cache.fc1_output)
    del g_down_input
    if param_grads is not None:
        _linear_grads(param_grads, mlp.fc1, g_fc1, m_cache.norm_output)
    g_norm2 = _apply_transposed(g_fc1, mlp.fc1.weight)
    del g_fc1
    if param_grads is not None:
        _norm_weight_grad(param_grads, block.norm2, g_norm2, m_cache.norm_input)
    # res2 feeds norm2 and the residual output
    g_res2, g_attn_out = rmsnorm_pullback(g_norm2, m_cache.norm_input, block.norm2.weight, block.norm2.eps,
                                          g_residual, want_branch=True, keep_residual=keep_residual)
    del g_norm2

    # attention: res2 = out_proj(heads) + res1
    if param_grads is not None:
        _linear_grads(param_grads, attn.out_proj, g_attn_out, a_cache.out_proj_input)
    g_merged = _apply_transposed(g_attn_out, attn.out_proj.weight)
    del g_attn_out
    g_heads = attn_heads_split(g_merged, attn.n_heads, attn.head_dim)
    del g_merged
    scale = attn.softmax_scale if attn.softmax_scale is not None else 1.0 / math.sqrt(attn.head_dim)
    dq, dk, dv = attention_input_pullback_basis(a_cache.q_rope, a_cache.k_expanded, a_cache.v_expanded, g_heads,
                                                softmax_scale=float(scale), causal=True, kernel_mode=kernel_mode)
    del g_heads
    if attn.d_conv > 0 and param_grads is None and attn.conv1d.weight.shape[-1] <= FUSED_CONV_MAX_TAPS:
        # nothing needs the cotangent of the convolved projection itself: one pass
        g_qkv = attn_qkv_conv_pullback(dq, dk, dv, attn.conv1d.weight, n_kv_heads=attn.n_kv_heads,
                                       rope_base=attn.rope_base, rope_interleaved=attn.rope_interleaved)
        del dq, dk, dv
    else:
        g_qkv = attn_qkv_pullback(dq, dk, dv, n_kv_heads=attn.n_kv_heads, rope_base=attn.rope_base,
                                  rope_interleaved=attn.rope_interleaved)
        del dq, dk, dv
        if attn.d_conv > 0:
            if param_grads is not None:
                # the cache keeps the projection after the convolution only: redo the projection
                bias = getattr(attn.in_proj, "bias", None)
                x_pre = torch.nn.functional.linear(a_cache.norm_output.to(wdtype), attn.in_proj.weight.to(wdtype),
                                                   None if bias is None else bias.to(wdtype))
                _conv_grads(param_grads, attn.conv1d, g_qkv, x_pre)
                del x_pre
            g_qkv = causal_conv1d_pullback(g_qkv, attn.conv1d.weight)
    if param_grads is not None:
        _linear_grads(param_grads, attn.in_proj, g_qkv, a_cache.norm_output)
    g_norm1 = _apply_transposed(g_qkv, attn.in_proj.weight)
    del g_qkv
    if param_grads is not None:
        _norm_weight_grad(param_grads, block.norm, g_norm1, a_cache.norm_input)
    return rmsnorm_pullback(g_norm1, a_cache.norm_input, block.norm.weight, block.norm.eps, g_res2,
                            want_branch=want_branch)


def _pull_back_region(backend: Any, cache: Any, cotangent: torch.Tensor, kernel_mode: str,
                      param_grads: dict | None) -> torch.Tensor:
    start, end = cache.layer_range
    device = cache.region_input.device
    # region_output = hidden + residual of the last block: both receive the cotangent
    if param_grads is None and cotangent.shape[2] > 1 and cotangent.stride(2) == 0:
        # an expanded view: the same cotangent at every position (what mean pooling sends back).  The last
        # block's down-projection product then runs on one row per (b, p) and the kernels read [B,P,1,*].
        g = cotangent[:, :, :1].to(device=device, dtype=torch.float32, copy=True).contiguous()
    else:
        g = cotangent.to(device=device, dtype=torch.float32).contiguous()
    # the caller's tensor itself when it already is fp32, contiguous and on the device: the last block then
    # writes its residual sum to a new tensor instead of updating in place
    borrowed = g.data_ptr() == cotangent.data_ptr()
    g_branch = None
    for offset in range(end - start - 1, -1, -1):
        layer_cache = cache.layer_caches[offset]
        block = backend.backbone.blocks[layer_cache.layer_index]
        # hidden and residual at a block input enter only through their sum, so one cotangent
        # (fp32, and its rounded copy for the first product of the block before) is carried
        g, g_branch = _layer_input_pullback(block, layer_cache, g_branch, g, kernel_mode, want_branch=offset > 0,
                                            param_grads=param_grads, keep_residual=borrowed)
        borrowed = False
    return g


def region_input_pullback_basis(backend: Any, cache: Any, output_cotangent_basis: torch.Tensor, *,
                                kernel_mode: str = "hip") -> torch.Tensor:
    """``output_cotangent_basis [B, P, T, D]`` -> region-input cotangents ``[B, P, T, D]``.

    ``backend.backbone.blocks`` and ``cache.layer_caches`` use the attribute names of the
    reference's ``TransformerRegionBackend`` / ``TransformerRegionCache``.
    """
    if output_cotangent_basis.dim() != 4:
        raise ValueError("output_cotangent_basis must have shape [B, P, T, D]")
    if not output_cotangent_basis.is_cuda:
        raise RuntimeError("output_cotangent_basis must be a CUDA tensor (this build has no CPU execution path)")
    start, end = cache.layer_range
    if len(cache.layer_caches) != end - start:
        raise ValueError("cache.layer_caches does not match cache.layer_range")
    if end == start:
        return output_cotangent_basis.detach().clone()
    # the result carries no autograd graph (weights and cache are constants here, as in the reference's extension)
    with torch.no_grad():
        g = _pull_back_region(backend, cache, output_cotangent_basis, kernel_mode, None)
        return g.to(device=output_cotangent_basis.device, dtype=output_cotangent_basis.dtype)


def region_parameter_vjp_with_input_cotangent(backend: Any, cache: Any, output_cotangent: torch.Tensor, *,
                                              kernel_mode: str = "hip") -> tuple[dict[str, torch.Tensor], torch.Tensor]:
    """:func:`region_parameter_vjp` together with the cotangent of the region input ``[B, T, D]`` (fp32) that the
    same backward sweep ends with: what a local-VJP provider needs to carry a region's seed on to the decoder of
    the interface and to the canvas, at no extra cost."""
    if output_cotangent.dim() != 3:
        raise ValueError("output_cotangent must have shape [B, T, D]")
    if not output_cotangent.is_cuda:
        raise RuntimeError("output_cotangent must be a CUDA tensor (this build has no CPU execution path)")
    start, end = cache.layer_range
    if len(cache.layer_caches) != end - start:
        raise ValueError("cache.layer_caches does not match cache.layer_range")
    by_id: dict[int, torch.Tensor] = {}
    if end > start:
        with torch.no_grad():
            g_input = _pull_back_region(backend, cache, output_cotangent.unsqueeze(1), kernel_mode, by_id)[:, 0]
    else:
        g_input = output_cotangent.detach().float()
    wanted = {id(p) for layer_cache in cache.layer_caches
              for p in backend.backbone.blocks[layer_cache.layer_index].parameters() if p.requires_grad}
    out: dict[str, torch.Tensor] = {}
    for name, param in backend.named_parameters():
        if id(param) in wanted and id(param) in by_id:
            out[name] = by_id[id(param)].detach()
    return out, g_input


def region_parameter_vjp(backend: Any, cache: Any, output_cotangent: torch.Tensor, *,
                         kernel_mode: str = "hip") -> dict[str, torch.Tensor]:
    """Parameter gradients of one region for ``output_cotangent [B, T, D]``, keyed by the
    parameter names of ``backend.named_parameters()``.

    ``TransformerLowering.parameter_vjp`` of the reference (backends/transformer.py:76-85;
    autograd version :332-355).  One backward sweep over the cached activations with a single
    direction; every weight gradient is a plain GEMM of the cotangent at a module's output
    with the module's cached input.
    """
    return region_parameter_vjp_with_input_cotangent(backend, cache, output_cotangent, kernel_mode=kernel_mode)[0]


__all__ = [
    "attn_heads_split", "attn_qkv_conv_pullback", "attn_qkv_pullback", "causal_conv1d_pullback",
    "causal_conv1d_weight_grad", "gated_mlp_pullback", "rmsnorm_pullback", "rmsnorm_weight_grad", "region_input_pullback_basis", "region_parameter_vjp", "region_parameter_vjp_with_input_cotangent", "rope_tables",
]
