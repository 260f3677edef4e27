"""lbi_matrix_norms against a singular value decomposition in fp64 (what the reference's diagnostics call,
backward/suffix_scan.py:117-126), through the C ABI."""
from __future__ import annotations

import pytest
import torch

pytestmark = pytest.mark.gpu


def _truth(mats: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    wide = mats.double().cpu()
    return (torch.linalg.matrix_norm(wide, ord=2, dim=(-2, -1)), torch.linalg.matrix_norm(wide, ord="fro", dim=(-2, -1)))


def _check(mats: torch.Tensor, device, tol: float = 1e-5) -> None:
    from latent_bounded_interfaces_amd.hip.interface import matrix_norms

    before = mats.clone()
    spec, frob = matrix_norms(mats.to(device))
    want_spec, want_frob = _truth(mats)
    assert spec.dtype == torch.float32 and spec.shape == mats.shape[:-2] and frob.shape == mats.shape[:-2]
    assert torch.equal(mats, before)
    scale = want_spec.abs().clamp_min(1e-30)
    assert float(((spec.cpu().double() - want_spec).abs() / scale).max()) <= tol
    assert float(((frob.cpu().double() - want_frob).abs() / want_frob.abs().clamp_min(1e-30)).max()) <= tol


@pytest.mark.parametrize("rank", [1, 2, 5, 32, 64, 88, 90, 100, 256])
def test_random_matrices(rank, device):
    """d <= 88 keeps its buffers in LDS, larger d in the workspace; d not a multiple of 4 is zero padded."""
    gen = torch.Generator().manual_seed(rank)
    _check(torch.randn(3, 4, rank, rank, generator=gen) * rank ** -0.5, device)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_16bit_storage(dtype, device):
    gen = torch.Generator().manual_seed(7)
    _check((torch.randn(5, 64, 64, generator=gen) / 8).to(dtype), device)


def test_near_identity_and_special_spectra(device):
    gen = torch.Generator().manual_seed(11)
    rank = 64
    near = torch.eye(rank) + torch.randn(6, rank, rank, generator=gen) * (0.01 / rank) ** 0.5
    orth = torch.linalg.qr(torch.randn(rank, rank, generator=gen))[0]
    rank1 = torch.outer(torch.randn(rank, generator=gen), torch.randn(rank, generator=gen))
    cluster = torch.diag(torch.cat((torch.tensor([1.0, 1.0 - 1e-4, 1.0 - 2e-4]), torch.full((rank - 3,), 0.5))))
    nilpotent = torch.diag(torch.ones(rank - 1), 1) * 3.0      # every eigenvalue 0, largest singular value 3
    special = torch.stack((torch.eye(rank), orth, rank1, cluster, nilpotent, 1e-12 * orth, 1e12 * rank1))
    _check(torch.cat((near, special)), device)


def test_zero_matrix_and_empty_batch(device):
    from latent_bounded_interfaces_amd.hip.interface import matrix_norms

    spec, frob = matrix_norms(torch.zeros(2, 8, 8, device=device))
    assert torch.equal(spec.cpu(), torch.zeros(2)) and torch.equal(frob.cpu(), torch.zeros(2))
    spec, frob = matrix_norms(torch.zeros(0, 8, 8, device=device))
    assert spec.shape == (0,) and frob.shape == (0,)


def test_many_matrices_at_the_benchmark_width(device):
    """More matrices than workgroups (grid-stride loop), d=256 (workspace path), near-identity as the scan
    benchmark's inputs; a sample is checked against the decomposition, all against the bounds that hold for
    every matrix: max column norm <= spectral <= Frobenius."""
    from latent_bounded_interfaces_amd.hip.interface import matrix_norms

    gen = torch.Generator().manual_seed(5)
    count, rank = 1300, 256
    mats = torch.eye(rank) + torch.randn(count, rank, rank, generator=gen) * (0.01 / rank) ** 0.5
    spec, frob = matrix_norms(mats.to(device))
    spec, frob = spec.cpu(), frob.cpu()
    col = mats.norm(dim=-2).amax(-1)
    assert bool((spec >= col * (1 - 1e-5)).all()) and bool((spec <= frob * (1 + 1e-6)).all())
    sample = torch.arange(0, count, 97)
    want, _ = _truth(mats[sample])
    assert float(((spec[sample].double() - want).abs() / want).max()) <= 1e-5
    again, _ = matrix_norms(mats.to(device))
    assert torch.equal(again.cpu(), spec)


def test_contract(device):
    from latent_bounded_interfaces_amd.hip.interface import matrix_norms

    with pytest.raises(ValueError, match="square"):
        matrix_norms(torch.zeros(2, 3, 4, device=device))
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        matrix_norms(torch.zeros(2, 4, 4))
    with pytest.raises(RuntimeError, match="dtype"):
        matrix_norms(torch.zeros(2, 4, 4, device=device, dtype=torch.float64))


def test_jacobian_stats_match_the_decomposition(device):
    """interface_state_jacobian_t_stats: the reference's keys, values from an fp64 decomposition on the host."""
    from latent_bounded_interfaces_amd.backward import suffix_scan as bs
    from oracle import scan as oscan

    mats, _ = oscan.make_scan_inputs(3, 5, 32, kind="randn", seed=2)
    jts = [mats[:, i].to(device) for i in range(5)]
    stats = bs.interface_state_jacobian_t_stats(jts, include_suffix=True)
    spec, frob = _truth(mats)
    suffix_spec, _ = _truth(oscan.suffix_scan_sequential(mats, dtype=torch.float64))
    want = {
        "jac_local_spec_mean": spec.mean(), "jac_local_spec_max": spec.max(), "jac_local_frob_mean": frob.mean(),
        "jac_local_frob_max": frob.max(), "jac_local_frob_normed_mean": (frob / 32 ** 0.5).mean(),
        "jac_suffix_spec_mean": suffix_spec.mean(), "jac_suffix_spec_max": suffix_spec.max(),
    }
    assert set(stats) == set(want)
    for key, value in want.items():
        assert stats[key] == pytest.approx(float(value), rel=2e-5), key
    local_only = bs.interface_state_jacobian_t_stats(jts, include_suffix=False)
    assert set(local_only) == {k for k in want if "suffix" not in k}
    assert bs.interface_state_jacobian_t_stats([], include_suffix=True) == {}
