"""CPU restatement of the reference's Transformer region forward and of its autograd
region-level input pullback.  TEST INFRASTRUCTURE ONLY: nothing under the product package
imports this module; tests, the smoke check and the CPU-baseline leg of the benchmark do.

What is restated (reference file:line):

* ``RMSNorm``                       backbones/transformer/block.py:12-23
* pre-norm residual handling        backbones/transformer/block.py:66-76
* rotary embedding                  backbones/transformer/rope.py:6-34
* attention forward with cache      backends/transformer.py:118-171
                                    (module layout backbones/transformer/attention.py:20-60)
* gated MLP forward with cache      backends/transformer.py:172-188
                                    (module layout backbones/transformer/mlp.py:11-32)
* block / region forward            backends/transformer.py:190-246
* cache field names                 backends/transformer.py:17-61
* autograd input pullback           backends/transformer.py:284-330 (one direction at a time)

The stand-in modules use the reference's attribute names (``norm``, ``attn.in_proj``,
``attn.conv1d``, ``attn.out_proj``, ``norm2``, ``mlp.fc1``, ``mlp.fc2``, ``residual_in_fp32``
...) and the caches its field names, so a lowering written against the reference's backend
objects runs unchanged on these.

Pinned by tests/test_oracle_region.py: RMSNorm against ``torch.nn.functional.rms_norm``;
the rotary embedding against complex multiplication and against its own inverse; the
attention branch against a dense softmax; the causal convolution against an explicit loop;
the block against a second, independently written formulation; the autograd pullback against
central finite differences in fp64.
"""
from __future__ import annotations

import math
from types import SimpleNamespace

import torch
import torch.nn.functional as F
from torch import nn


class OracleRMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float = 1e-5) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.eps = eps

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        xf = x.float()
        inv = torch.rsqrt((xf * xf).mean(dim=-1, keepdim=True) + self.eps)
        return (xf * inv).to(x.dtype) * self.weight.to(x.dtype)


def rope_tables(seq_len: int, head_dim: int, base: float, device=None) -> tuple[torch.Tensor, torch.Tensor]:
    """cos / sin of position * base^(-2i/head_dim), each [seq_len, head_dim/2] fp32."""
    half = head_dim // 2
    pos = torch.arange(seq_len, device=device, dtype=torch.float32)
    idx = torch.arange(half, device=device, dtype=torch.float32)
    angles = torch.outer(pos, base ** (-2.0 * idx / float(head_dim)))
    return angles.cos(), angles.sin()


def rope(x: torch.Tensor, base: float = 10000.0, interleaved: bool = False) -> torch.Tensor:
    """Rotary embedding of x [B, H, T, Dh]: pairs (j, j+Dh/2), or (2j, 2j+1) when interleaved."""
    if x.dim() != 4:
        raise ValueError("RoPE expects x shaped [B, H, L, D].")
    dh = x.shape[-1]
    if dh % 2:
        raise ValueError("RoPE requires an even head dimension.")
    cos, sin = rope_tables(x.shape[-2], dh, base, device=x.device)
    xf = x.float()
    if interleaved:
        a, b = xf[..., 0::2], xf[..., 1::2]
        out = torch.stack((a * cos - b * sin, a * sin + b * cos), dim=-1).flatten(-2)
    else:
        a, b = xf[..., : dh // 2], xf[..., dh // 2:]
        out = torch.cat((a * cos - b * sin, a * sin + b * cos), dim=-1)
    return out.to(x.dtype)


class OracleAttention(nn.Module):
    def __init__(self, dim, *, n_heads, n_kv_heads, head_dim, rope_base=10000.0, rope_interleaved=False,
                 softmax_scale=None, d_conv=0, bias=False) -> None:
        super().__init__()
        if n_heads % n_kv_heads:
            raise ValueError("n_heads must be divisible by n_kv_heads")
        self.dim, self.n_heads, self.n_kv_heads, self.head_dim = dim, n_heads, n_kv_heads, head_dim
        self.rope_base, self.rope_interleaved, self.softmax_scale, self.d_conv = rope_base, rope_interleaved, softmax_scale, d_conv
        self.qkv_dim = head_dim * (n_heads + 2 * n_kv_heads)
        self.out_dim = head_dim * n_heads
        self.in_proj = nn.Linear(dim, self.qkv_dim, bias=bias)
        if d_conv > 0:
            self.conv1d = nn.Conv1d(self.qkv_dim, self.qkv_dim, kernel_size=d_conv, padding=d_conv - 1,
                                    groups=self.qkv_dim, bias=bias)
        self.out_proj = nn.Linear(self.out_dim, dim, bias=bias)

    def _expand_kv(self, x: torch.Tensor) -> torch.Tensor:
        rep = self.n_heads // self.n_kv_heads
        return x if rep == 1 else x.repeat_interleave(rep, dim=1)


class OracleGatedMLP(nn.Module):
    def __init__(self, dim, hidden, bias=False) -> None:
        super().__init__()
        self.fc1 = nn.Linear(dim, 2 * hidden, bias=bias)
        self.fc2 = nn.Linear(hidden, dim, bias=bias)


class OracleBlock(nn.Module):
    def __init__(self, dim, *, n_heads, n_kv_heads, head_dim, hidden, rope_base=10000.0, rope_interleaved=False,
                 softmax_scale=None, d_conv=0, residual_in_fp32=True, bias=False) -> None:
        super().__init__()
        self.residual_in_fp32 = residual_in_fp32
        self.norm = OracleRMSNorm(dim)
        self.attn = OracleAttention(dim, n_heads=n_heads, n_kv_heads=n_kv_heads, head_dim=head_dim,
                                    rope_base=rope_base, rope_interleaved=rope_interleaved,
                                    softmax_scale=softmax_scale, d_conv=d_conv, bias=bias)
        self.norm2 = OracleRMSNorm(dim)
        self.mlp = OracleGatedMLP(dim, hidden, bias=bias)

    def _prenorm(self, hidden_states, residual, norm):
        residual = hidden_states if residual is None else hidden_states + residual
        normed = norm(residual.to(norm.weight.dtype))
        if self.residual_in_fp32:
            residual = residual.float()
        return normed, residual


def attention_forward(attn: OracleAttention, x: torch.Tensor):
    """x [B, T, D] (normed) -> (out_proj output, cache namespace)."""
    bsz, seqlen, _ = x.shape
    qkv = attn.in_proj(x)
    if attn.d_conv > 0:
        qkv = attn.conv1d(qkv.transpose(1, 2))[..., :seqlen].transpose(1, 2).contiguous()
    qd, kd = attn.n_heads * attn.head_dim, attn.n_kv_heads * attn.head_dim
    q, k, v = qkv.split((qd, kd, kd), dim=-1)
    q = q.view(bsz, seqlen, attn.n_heads, attn.head_dim).transpose(1, 2)
    k = k.view(bsz, seqlen, attn.n_kv_heads, attn.head_dim).transpose(1, 2)
    v = v.view(bsz, seqlen, attn.n_kv_heads, attn.head_dim).transpose(1, 2)
    q_rope = rope(q, attn.rope_base, attn.rope_interleaved)
    k_rope = rope(k, attn.rope_base, attn.rope_interleaved)
    k_exp, v_exp = attn._expand_kv(k_rope), attn._expand_kv(v)
    scale = attn.softmax_scale if attn.softmax_scale is not None else 1.0 / math.sqrt(attn.head_dim)
    heads = F.scaled_dot_product_attention(q_rope, k_exp, v_exp, attn_mask=None, dropout_p=0.0, is_causal=True,
                                           scale=scale).transpose(1, 2)
    merged = heads.contiguous().view(bsz, seqlen, attn.out_dim)
    out = attn.out_proj(merged)
    cache = SimpleNamespace(norm_input=x, norm_output=x, qkv=qkv, q=q, k=k, v=v, q_rope=q_rope, k_rope=k_rope,
                            k_expanded=k_exp, v_expanded=v_exp, attn_output=heads, out_proj_input=merged,
                            out_proj_output=out)
    return out, cache


def mlp_forward(mlp: OracleGatedMLP, x: torch.Tensor):
    fc1 = mlp.fc1(x)
    up, gate = fc1.chunk(2, dim=-1)
    act = F.silu(gate)
    down_in = up * act
    out = mlp.fc2(down_in)
    cache = SimpleNamespace(norm_input=x, norm_output=x, fc1_output=fc1, up=up, gate=gate, activation=act,
                            down_input=down_in, down_output=out)
    return out, cache


def block_forward(block: OracleBlock, hidden, residual):
    norm1_in = hidden if residual is None else hidden + residual
    n1, res1 = block._prenorm(hidden, residual, block.norm)
    a, a_cache = attention_forward(block.attn, n1)
    a_cache.norm_input = norm1_in
    norm2_in = a + res1
    n2, res2 = block._prenorm(a, res1, block.norm2)
    m, m_cache = mlp_forward(block.mlp, n2)
    m_cache.norm_input = norm2_in
    return m, res2, a_cache, m_cache


class OracleRegionBackend(nn.Module):
    """Stand-in for the reference's TransformerRegionBackend: ``backbone.blocks`` plus
    ``region_ranges`` and ``forward_region`` (backends/transformer.py:88-116, 217-246)."""

    name = "transformer"

    def __init__(self, blocks, region_ranges) -> None:
        super().__init__()
        self.backbone = nn.Module()
        self.backbone.blocks = nn.ModuleList(blocks)
        self.region_ranges = list(region_ranges)

    def forward_region(self, *, region_input: torch.Tensor, region_index: int):
        start, end = self.region_ranges[region_index]
        hidden, residual, layer_caches = region_input, None, []
        for layer_index in range(start, end):
            h_in, r_in = hidden, residual
            hidden, residual, a_cache, m_cache = block_forward(self.backbone.blocks[layer_index], hidden, residual)
            layer_caches.append(SimpleNamespace(layer_index=layer_index, hidden_input=h_in, residual_input=r_in,
                                                attention=a_cache, mlp=m_cache, hidden_output=hidden,
                                                residual_output=residual))
        out = hidden if residual is None else hidden + residual
        cache = SimpleNamespace(region_index=region_index, layer_range=(start, end), layer_caches=layer_caches,
                                region_input=region_input, region_output=out)
        return out, cache

    def parameters_for_region(self, region_index: int):
        start, end = self.region_ranges[region_index]
        return [p for i in range(start, end) for p in self.backbone.blocks[i].parameters() if p.requires_grad]


def make_backend(*, dim, n_heads, n_kv_heads=None, head_dim=None, hidden=None, layers=2, region_ranges=None,
                 rope_base=10000.0, rope_interleaved=False, softmax_scale=None, d_conv=0, residual_in_fp32=True,
                 bias=False, dtype=torch.float32, seed=0, weight_std=None) -> OracleRegionBackend:
    """Random-init region backend.  Weights ~ N(0, weight_std^2) (default dim^-1/2 so that
    activations stay O(1)), norm weights 1 + 0.1 N(0,1), from a CPU generator seeded with `seed`."""
    n_kv_heads = n_kv_heads or n_heads
    head_dim = head_dim or dim // n_heads
    hidden = hidden or 4 * dim
    blocks = [OracleBlock(dim, n_heads=n_heads, n_kv_heads=n_kv_heads, head_dim=head_dim, hidden=hidden,
                          rope_base=rope_base, rope_interleaved=rope_interleaved, softmax_scale=softmax_scale,
                          d_conv=d_conv, residual_in_fp32=residual_in_fp32, bias=bias) for _ in range(layers)]
    gen = torch.Generator(device="cpu").manual_seed(seed)
    with torch.no_grad():
        for block in blocks:
            for name, p in block.named_parameters():
                if name.endswith("norm.weight") or name.endswith("norm2.weight"):
                    p.copy_(1.0 + 0.1 * torch.randn(p.shape, generator=gen))
                elif "conv1d.weight" in name:
                    p.copy_(torch.randn(p.shape, generator=gen) * (1.0 / p.shape[-1]) ** 0.5)
                elif p.dim() >= 2:
                    std = weight_std if weight_std is not None else p.shape[-1] ** -0.5
                    p.copy_(torch.randn(p.shape, generator=gen) * std)
                else:
                    p.copy_(0.1 * torch.randn(p.shape, generator=gen))
    backend = OracleRegionBackend(blocks, region_ranges or [(0, layers)])
    return backend.to(dtype)


def input_pullback_basis_autograd(backend, cache, output_cotangent_basis: torch.Tensor) -> torch.Tensor:
    """Region input pullback [B, P, T, D] by autograd, one basis direction at a time."""
    if output_cotangent_basis.dim() != 4:
        raise ValueError("output_cotangent_basis must have shape [B, P, T, D]")
    grads = []
    for p in range(output_cotangent_basis.shape[1]):
        x = cache.region_input.detach().requires_grad_(True)
        y, _ = backend.forward_region(region_input=x, region_index=cache.region_index)
        (gx,) = torch.autograd.grad(y, x, grad_outputs=output_cotangent_basis[:, p].to(y.dtype))
        grads.append(gx.unsqueeze(1))
    return torch.cat(grads, dim=1).to(output_cotangent_basis.dtype)


def parameter_vjp_autograd(backend, cache, output_cotangent: torch.Tensor) -> dict[str, torch.Tensor]:
    """Parameter VJP of one region by autograd (reference backends/transformer.py:332-355)."""
    params = backend.parameters_for_region(cache.region_index)
    y, _ = backend.forward_region(region_input=cache.region_input.detach(), region_index=cache.region_index)
    grads = torch.autograd.grad(y, params, grad_outputs=output_cotangent.to(y.dtype), allow_unused=True)
    names = {id(p): n for n, p in backend.named_parameters()}
    return {names[id(p)]: g.detach().clone() for p, g in zip(params, grads) if g is not None}
