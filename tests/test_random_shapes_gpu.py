"""Seeded random shapes through the kernels with the most shape-dependent dispatch (needs the GPU): the single-launch
attention pullback, the parameter-gradient sums and the 16-bit cotangent chain, each against its fp64 / fp32 truth."""
from __future__ import annotations

import random

import pytest
import torch
import torch.nn.functional as F

from oracle import attention as oattn
from oracle import scan as oscan

pytestmark = pytest.mark.gpu


def _rel(a, b):
    return float((a.double() - b.double()).abs().max() / b.double().abs().max().clamp_min(1e-30))


def test_short_sequence_attention_random_shapes(device):
    from latent_bounded_interfaces_amd.hip.transformer import attention_input_pullback_basis

    rng = random.Random(1)
    for case in range(20):
        head_dim = rng.choice([64, 64, 128])
        seqlen = rng.randint(1, 256 if head_dim == 64 else 128)
        seqlen = 32 * ((seqlen + 31) // 32) if rng.random() < 0.3 else seqlen
        bsz, heads, basis = rng.randint(1, 3), rng.randint(1, 4), rng.randint(1, 6)
        causal = rng.random() < 0.7
        dtype = rng.choice([torch.float16, torch.bfloat16])
        scale = head_dim ** -0.5 * rng.choice([0.5, 1.0, 2.0])
        q, k, v, g = oattn.make_attention_inputs(bsz, heads, seqlen, head_dim, basis, dtype=dtype, seed=100 + case)
        got = attention_input_pullback_basis(q.to(device), k.to(device), v.to(device), g.to(device),
                                             softmax_scale=scale, causal=causal, kernel_mode="hip")
        want = oattn.attention_pullback_blocked(q, k, v, g, softmax_scale=scale, causal=causal, dtype=torch.float32)
        for name, a, c in zip(("dq", "dk", "dv"), got, want):
            assert _rel(a.cpu(), c) <= 2e-2, (case, (bsz, heads, seqlen, head_dim, basis), causal, dtype, name)


def test_parameter_gradient_sums_random_shapes(device):
    from latent_bounded_interfaces_amd.hip.transformer import region

    rng = random.Random(2)
    for case in range(12):
        dtype = rng.choice([torch.float32, torch.float16, torch.bfloat16])
        width, rows = 4 * rng.randint(1, 512), rng.randint(1, 700)
        gen = torch.Generator().manual_seed(case)
        g = torch.randn(rows, width, generator=gen).to(dtype)
        x = torch.randn(rows, width, generator=gen) * rng.choice([0.1, 1.0, 30.0])
        x = x.to(dtype) if rng.random() < 0.5 else x
        got = region.rmsnorm_weight_grad(g.to(device), x.to(device), 1e-5).cpu()
        xr = x.to(dtype).float()
        normed = (xr * torch.rsqrt(xr.pow(2).mean(-1, keepdim=True) + 1e-5)).to(dtype)
        want = (g.double() * normed.double()).sum(0)
        assert _rel(got, want) <= (2e-5 if dtype == torch.float32 else 3e-3), (case, rows, width, dtype)
    for case in range(12):
        dtype = rng.choice([torch.float32, torch.float16, torch.bfloat16])
        channels = rng.choice([1, 3, 4, 12, 100, 2304, 4 * rng.randint(1, 300), rng.randint(1, 50)])
        ksize, bsz, seqlen = rng.randint(1, 8), rng.randint(1, 3), rng.randint(1, 200)
        gen = torch.Generator().manual_seed(50 + case)
        g = torch.randn(bsz, seqlen, channels, generator=gen).to(dtype)
        x = torch.randn(bsz, seqlen, channels, generator=gen).to(dtype)
        g_w, g_b = region.causal_conv1d_weight_grad(g.to(device), x.to(device), ksize)
        w = torch.zeros(channels, 1, ksize, dtype=torch.float64, requires_grad=True)
        b = torch.zeros(channels, dtype=torch.float64, requires_grad=True)
        y = F.conv1d(x.double().transpose(1, 2), w, b, padding=ksize - 1, groups=channels)[..., :seqlen].transpose(1, 2)
        want_w, want_b = torch.autograd.grad(y, (w, b), grad_outputs=g.double())
        assert _rel(g_w.cpu(), want_w) <= 3e-5 and _rel(g_b.cpu(), want_b) <= 3e-5, (case, (bsz, seqlen, channels, ksize))


def test_16bit_cotangent_chain_random_lengths(device):
    from latent_bounded_interfaces_amd.hip.interface import suffix_scan_cotangents

    rng = random.Random(3)
    for case in range(6):
        bsz, count = rng.randint(1, 9), rng.randint(0, 20)
        dtype = rng.choice([torch.float16, torch.bfloat16])
        mats, g = oscan.make_scan_inputs(bsz, count, 256, kind="randn", seed=case)
        mats = mats.to(dtype)
        out = suffix_scan_cotangents(mats.to(device), g.to(device)).cpu()
        truth = oscan.suffix_cotangents_sequential(mats.double(), g.double())
        scale = truth.abs().amax(dim=2, keepdim=True).clamp_min(1e-30)
        assert float(((out.double() - truth).abs() / scale).max()) <= 1e-5, (case, bsz, count, dtype)


def test_suffix_scan_random_shapes(device):
    """The scan entries over random batch sizes, chain lengths and widths (matrix-core widths, padded widths,
    scalar widths; chains short and long enough for the K-parallel form; every storage type): matrices against the
    fp64 sequential product at the fp32 bar, cotangents at the bars of their two forms, fused == separate."""
    from latent_bounded_interfaces_amd.hip.interface import (suffix_scan_cotangents, suffix_scan_pullbacks,
                                                             suffix_scan_pullbacks_and_cotangents)

    rng = random.Random(3)
    for case in range(28):
        rank = rng.choice([32, 64, 128, 256, 256, 64, rng.randint(1, 40), rng.randint(41, 200)])
        count = rng.choice([0, 1, 2, rng.randint(3, 11), rng.randint(12, 40), rng.randint(41, 90)])
        bsz = rng.choice([1, 1, 2, 3, rng.randint(4, 9), rng.randint(10, 20)])
        if rank > 128:
            count, bsz = min(count, 48), min(bsz, 6)
        dtype = rng.choice([torch.float32, torch.float32, torch.bfloat16, torch.float16])
        kind = rng.choice(["randn", "near_identity"])
        mats, g = oscan.make_scan_inputs(bsz, count, rank, kind=kind, seed=300 + case)
        mats = mats.to(dtype)
        tag = (case, bsz, count, rank, dtype, kind)
        out, cot = suffix_scan_pullbacks_and_cotangents(mats.to(device), g.to(device))
        assert torch.equal(out, suffix_scan_pullbacks(mats.to(device))), tag
        truth = oscan.suffix_scan_sequential(mats.float(), dtype=torch.float64)
        err = (out.cpu().double() - truth).abs().flatten(2).amax(2) / truth.abs().flatten(2).amax(2).clamp_min(1e-30)
        assert float(err.max()) <= 1e-5, tag
        assert torch.equal(out[:, count].cpu(), torch.eye(rank).expand(bsz, rank, rank)), tag
        want = oscan.suffix_cotangents_sequential(mats.double(), g.double())
        scale = want.abs().amax(dim=2, keepdim=True).clamp_min(1e-30)
        # the fused entry's cotangents are the chain, or in its K-parallel form the products applied to g (3e-5)
        assert float(((cot.cpu().double() - want).abs() / scale).max()) <= 3e-5, tag
        chain = suffix_scan_cotangents(mats.to(device), g.to(device)).cpu()
        assert float(((chain.double() - want).abs() / scale).max()) <= 1e-5, tag
