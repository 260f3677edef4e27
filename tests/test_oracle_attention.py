"""Pins the CPU attention-pullback oracle: closed forms, library autograd, finite differences (no GPU)."""
from __future__ import annotations

import json
import math
from pathlib import Path

import pytest
import torch

from oracle import attention as oattn

GOLDEN = json.loads((Path(__file__).parent / "golden" / "attention_known_answers.json").read_text())


@pytest.mark.parametrize("case", ["two_keys_equal", "single_token"])
@pytest.mark.parametrize("fn", ["dense", "sdpa", "blocked"])
def test_known_answers(case, fn):
    c = GOLDEN[case]
    q, k, v, g = (torch.tensor(c[n], dtype=torch.float64) for n in ("q", "k", "v", "d_out"))
    kw = dict(softmax_scale=c["softmax_scale"], causal=c["causal"])
    if fn == "dense":
        got = oattn.attention_pullback_dense(q, k, v, g, **kw)
    elif fn == "sdpa":
        got = oattn.attention_pullback_sdpa_loop(q, k, v, g, **kw)
    else:
        got = oattn.attention_pullback_blocked(q, k, v, g, block=1, dtype=torch.float64, **kw)
    for name, t in zip(("dq", "dk", "dv"), got):
        assert torch.allclose(t, torch.tensor(c[name], dtype=torch.float64), atol=1e-12), name


# Shapes and seeds of the reference's own tests (tests/test_cuda_attention_pullback.py:62-66,
# 86-90, 115-119, 178-182).
REFERENCE_CASES = [(101, (2, 3, 5, 4), 2), (103, (1, 2, 4, 3), 3), (117, (1, 2, 4, 16), 3), (121, (1, 2, 16, 64), 1)]


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("seed,shape,basis", REFERENCE_CASES)
def test_dense_formula_matches_library_autograd(seed, shape, basis, causal):
    torch.manual_seed(seed)
    q = torch.randn(*shape)
    k = torch.randn_like(q)
    v = torch.randn_like(q)
    g = torch.randn(shape[0], basis, *shape[1:])
    scale = 1.0 / math.sqrt(shape[-1])
    dense = oattn.attention_pullback_dense(q, k, v, g, softmax_scale=scale, causal=causal)
    sdpa = oattn.attention_pullback_sdpa_loop(q, k, v, g, softmax_scale=scale, causal=causal)
    blocked = oattn.attention_pullback_blocked(q, k, v, g, softmax_scale=scale, causal=causal, block=3)
    for a, b, c in zip(dense, sdpa, blocked):
        assert a.shape == g.shape
        assert torch.allclose(a, b, atol=2e-5, rtol=2e-5)  # the reference's fp32 tolerance
        assert torch.allclose(a, c, atol=2e-5, rtol=2e-5)


@pytest.mark.parametrize("causal", [True, False])
def test_finite_differences_fp64(causal):
    torch.manual_seed(7)
    shape, basis, scale, eps = (1, 2, 5, 3), 2, 0.6, 1e-6
    q, k, v = (torch.randn(*shape, dtype=torch.float64) for _ in range(3))
    g = torch.randn(shape[0], basis, *shape[1:], dtype=torch.float64)
    dq, dk, dv = oattn.attention_pullback_dense(q, k, v, g, softmax_scale=scale, causal=causal)

    def scalar(qq, kk, vv, p):
        out, _ = oattn.attention_forward_dense(qq, kk, vv, softmax_scale=scale, causal=causal)
        return (out * g[:, p]).sum()

    for p in range(basis):
        for tensor, grad, which in ((q, dq, 0), (k, dk, 1), (v, dv, 2)):
            flat = tensor.reshape(-1)
            for idx in range(0, flat.numel(), 4):
                plus, minus = tensor.clone().reshape(-1), tensor.clone().reshape(-1)
                plus[idx] += eps
                minus[idx] -= eps
                args_p = [q, k, v]
                args_m = [q, k, v]
                args_p[which] = plus.reshape(shape)
                args_m[which] = minus.reshape(shape)
                fd = (scalar(*args_p, p) - scalar(*args_m, p)) / (2 * eps)
                assert abs(fd - grad[:, p].reshape(-1)[idx]) < 1e-7


def test_invariants():
    q, k, v, g = oattn.make_attention_inputs(2, 2, 6, 4, 3, dtype=torch.float64, seed=3)
    scale = 0.5
    dq, dk, dv = oattn.attention_pullback_dense(q, k, v, g, softmax_scale=scale, causal=True)
    # linear in the cotangent, and direction p only depends on d_out[:, p]
    g2 = g.clone()
    g2[:, 1] = 2.0 * g[:, 1] - g[:, 0]
    dq2, dk2, dv2 = oattn.attention_pullback_dense(q, k, v, g2, softmax_scale=scale, causal=True)
    for a, b in ((dq, dq2), (dk, dk2), (dv, dv2)):
        assert torch.allclose(b[:, 0], a[:, 0], atol=1e-13)
        assert torch.allclose(b[:, 2], a[:, 2], atol=1e-13)
        assert torch.allclose(b[:, 1], 2.0 * a[:, 1] - a[:, 0], atol=1e-12)
    # causal: the first query sees one key, so its dQ vanishes; the last key only hears from the last query
    assert torch.allclose(dq[:, :, :, 0], torch.zeros_like(dq[:, :, :, 0]), atol=1e-14)
    _, lse = oattn.attention_forward_dense(q, k, v, softmax_scale=scale, causal=True)
    p_last = torch.exp((q[:, :, -1] * k[:, :, -1]).sum(-1) * scale - lse[:, :, -1])
    assert torch.allclose(dv[:, :, :, -1], p_last[:, None, :, None] * g[:, :, :, -1], atol=1e-13)
    # a swapped scale (applied to dV, or missing from dQ) must be told apart
    assert not torch.allclose(dq, dq / scale, atol=1e-3)


def test_contract_errors():
    q = torch.zeros(1, 2, 3, 4)
    with pytest.raises(ValueError):
        oattn.attention_pullback_dense(q, q[:, :1], q, torch.zeros(1, 1, 2, 3, 4), softmax_scale=1.0)
    with pytest.raises(ValueError):
        oattn.attention_pullback_dense(q, q, q, torch.zeros(1, 2, 3, 4), softmax_scale=1.0)
    with pytest.raises(ValueError):
        oattn.attention_pullback_dense(q, q, q, torch.zeros(1, 1, 2, 5, 4), softmax_scale=1.0)
