"""Pins the CPU scan oracle: known answers, brute force, closed forms, invariants (no GPU)."""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import scan as oscan

GOLDEN = json.loads((Path(__file__).parent / "golden" / "scan_known_answers.json").read_text())

# Shapes of the reference's own CPU test (tests/test_interface_scan.py:45-53).
REFERENCE_CPU_SHAPES = [(1, 0, 1), (1, 1, 1), (1, 1, 4), (2, 3, 5), (2, 4, 8), (4, 8, 16), (1, 16, 64)]


def _reference_tolerances(count: int, rank: int) -> tuple[float, float]:
    # reference tests/test_interface_scan.py:33-40
    if rank >= 256:
        return 7e-1, 1e-5
    if rank >= 128:
        return 2.5e-1, 1e-5
    if count >= 8 or rank >= 16:
        return 3e-2, 1e-5
    return 2e-5, 1e-5


@pytest.mark.parametrize("fn", [oscan.suffix_scan_levels, oscan.suffix_scan_sequential])
def test_known_answer_2x2(fn):
    case = GOLDEN["order_case_2x2"]
    mats = torch.tensor(case["mats"], dtype=torch.float32)
    expected = torch.tensor(case["suffix"], dtype=torch.float32)
    assert torch.equal(fn(mats), expected)  # small integers: exact in fp32


def test_known_answer_cotangents():
    case = GOLDEN["order_case_2x2"]
    mats = torch.tensor(case["mats"], dtype=torch.float32)
    g = torch.tensor(case["g"], dtype=torch.float32)
    expected = torch.tensor(case["cotangents"], dtype=torch.float32)
    assert torch.equal(oscan.suffix_cotangents_sequential(mats, g), expected)
    assert torch.equal(oscan.suffix_cotangents_from_matrices(oscan.suffix_scan_sequential(mats), g), expected)


def test_loops_known_answer():
    case = GOLDEN["order_case_2x2"]
    assert np.array_equal(oscan.suffix_scan_loops(case["mats"]), np.array(case["suffix"]))


@pytest.mark.parametrize("shape", [(1, 1, 1), (2, 3, 5), (2, 4, 8), (1, 7, 3)])
def test_torch_restatements_match_python_loops(shape):
    bsz, count, rank = shape
    mats, _ = oscan.make_scan_inputs(bsz, count, rank, kind="randn", seed=3)
    brute = torch.from_numpy(oscan.suffix_scan_loops(mats.numpy()))
    for fn in (oscan.suffix_scan_levels, oscan.suffix_scan_sequential):
        got = fn(mats.double())
        assert torch.allclose(got, brute, atol=1e-13, rtol=1e-12)


@pytest.mark.parametrize("shape", REFERENCE_CPU_SHAPES)
def test_levels_match_sequential_on_reference_shapes(shape):
    bsz, count, rank = shape
    torch.manual_seed(0)
    mats = torch.randn(bsz, count, rank, rank) * (1.0 / max(rank, 1) ** 0.5)
    original = mats.clone()
    actual = oscan.suffix_scan_levels(mats)
    expected = oscan.suffix_scan_sequential(mats)
    atol, rtol = _reference_tolerances(count, rank)
    assert actual.shape == (bsz, count + 1, rank, rank)
    assert actual.dtype == mats.dtype
    assert torch.allclose(actual, expected, atol=atol, rtol=rtol)
    assert torch.equal(mats, original)
    truth = oscan.suffix_scan_sequential(mats, dtype=torch.float64)
    assert (actual.double() - truth).abs().max() <= 1e-5 * max(1.0, truth.abs().max().item())


def test_empty_chain_is_identity():
    mats = torch.empty(3, 0, 4, 4)
    for fn in (oscan.suffix_scan_levels, oscan.suffix_scan_sequential):
        out = fn(mats)
        assert out.shape == (3, 1, 4, 4)
        assert torch.equal(out, torch.eye(4).expand(3, 1, 4, 4))


def test_permutation_matrices_compose_exactly():
    gen = torch.Generator().manual_seed(5)
    rank, count = 7, 6
    perms = [torch.randperm(rank, generator=gen) for _ in range(count)]
    mats = torch.stack([torch.eye(rank)[p] for p in perms]).unsqueeze(0)  # row i of mats[r] is e_{p[i]}
    out = oscan.suffix_scan_levels(mats)
    # (A_r @ S)[i, :] = S[p_r[i], :], so the composed permutation is index composition.
    idx = torch.arange(rank)
    for r in range(count - 1, -1, -1):
        idx = idx[perms[r]]
        assert torch.equal(out[0, r], torch.eye(rank)[idx])


def test_diagonal_and_scalar_closed_forms():
    gen = torch.Generator().manual_seed(7)
    diag = torch.rand(2, 5, 6, generator=gen, dtype=torch.float64) + 0.5
    mats = torch.diag_embed(diag)
    expected = torch.flip(torch.cumprod(torch.flip(diag, dims=[1]), dim=1), dims=[1])
    for fn in (oscan.suffix_scan_levels, oscan.suffix_scan_sequential):
        out = fn(mats)
        assert torch.allclose(torch.diagonal(out[:, :5], dim1=-2, dim2=-1), expected, rtol=1e-13, atol=0)
        assert torch.equal(out[:, :5] * (1 - torch.eye(6, dtype=torch.float64)), torch.zeros(2, 5, 6, 6, dtype=torch.float64))
    scal = torch.rand(3, 9, 1, 1, generator=gen, dtype=torch.float64) + 0.5
    expected1 = torch.flip(torch.cumprod(torch.flip(scal[:, :, 0, 0], dims=[1]), dim=1), dims=[1])
    assert torch.allclose(oscan.suffix_scan_levels(scal)[:, :9, 0, 0], expected1, rtol=1e-13, atol=0)
    g = torch.rand(3, 1, generator=gen, dtype=torch.float64)
    cot = oscan.suffix_cotangents_sequential(scal, g)
    assert torch.allclose(cot[:, :9, 0], expected1 * g, rtol=1e-13, atol=0)
    assert torch.equal(cot[:, 9], g)


def test_recurrence_and_order_of_multiplication():
    mats, g = oscan.make_scan_inputs(2, 6, 5, kind="randn", seed=11)
    mats = mats.double()
    out = oscan.suffix_scan_levels(mats)
    for r in range(6):
        assert torch.allclose(out[:, r], mats[:, r] @ out[:, r + 1], atol=1e-13)
    # A wrong operand order (S @ A instead of A @ S) must be told apart.
    wrong = mats[:, 5] @ mats[:, 4]
    assert not torch.allclose(out[:, 4], wrong, atol=1e-3)
    cot = oscan.suffix_cotangents_sequential(mats, g.double())
    assert torch.allclose(cot, oscan.suffix_cotangents_from_matrices(out, g.double()), atol=1e-12)


def test_contract_errors():
    with pytest.raises(ValueError):
        oscan.suffix_scan_levels(torch.zeros(2, 3, 4))
    with pytest.raises(ValueError):
        oscan.suffix_scan_levels(torch.zeros(2, 3, 4, 5))
    with pytest.raises(ValueError):
        oscan.suffix_cotangents_sequential(torch.zeros(2, 3, 4, 4), torch.zeros(2, 5))
