"""Parity of the HIP suffix scan against the CPU oracle, through the C ABI (needs the GPU)."""
from __future__ import annotations

import json
from pathlib import Path

import pytest
import torch

from oracle import scan as oscan

pytestmark = pytest.mark.gpu

GOLDEN = json.loads((Path(__file__).parent / "golden" / "scan_known_answers.json").read_text())

# Every shape of the reference's tests (tests/test_interface_scan.py:45-53 and :78-86)
# plus ragged / non-power-of-two cases and each MFMA width with K not a power of two.
SHAPES = [
    (1, 0, 1), (1, 1, 1), (1, 1, 4), (2, 3, 5), (2, 4, 8), (4, 8, 16), (1, 16, 64),
    (1, 2, 16), (2, 4, 32), (2, 8, 64), (1, 16, 128), (1, 8, 256),
    (4, 8, 32), (3, 5, 32), (9, 7, 64), (5, 3, 128), (3, 5, 256), (2, 6, 48), (2, 3, 33), (1, 4, 100),
    (1, 3, 300), (2, 3, 512), (1, 2, 384),  # the widest matrix-core kernel, directly and through padding
    (1, 2, 520), (2, 5, 12),  # widths the scalar kernel still runs: past the largest matrix-core width, and tiny
    (17, 2, 256), (1, 1, 256), (2, 0, 32),
    (24, 14, 256), (33, 3, 256),  # d=256: 32-wide column blocks up to 32 batch elements, 64-wide beyond
]


# bf16 storage at d=256 runs on the 16-bit matrix cores.  By default the running suffix enters the products rounded to
# 16 significand bits (two bf16 planes): error against fp64 a hundred times inside the 2e-2 asked of 16-bit storage.
# exact_suffix=True (LBI_SCAN_EXACT_SUFFIX) keeps the fp32 value (three planes) and meets the fp32 bar.
BF16_D256_BAR = 2e-4
BF16_D256_EXACT_BAR = 1e-5


def _rel_err(actual: torch.Tensor, truth: torch.Tensor) -> float:
    """max over suffix matrices of max|diff| / max|truth| (fp64 truth)."""
    diff = (actual.double() - truth).abs().flatten(2).max(dim=2).values
    ref = truth.abs().flatten(2).max(dim=2).values.clamp_min(1e-30)
    return float((diff / ref).max())


def _scan(mats_cpu: torch.Tensor, device) -> torch.Tensor:
    from latent_bounded_interfaces_amd.hip.interface import suffix_scan_pullbacks

    mats = mats_cpu.to(device)
    keep = mats.clone()
    out = suffix_scan_pullbacks(mats)
    torch.cuda.synchronize()
    assert torch.equal(mats, keep), "input was modified"
    return out.cpu()


def test_known_answer_2x2(device):
    case = GOLDEN["order_case_2x2"]
    out = _scan(torch.tensor(case["mats"], dtype=torch.float32), device)
    assert torch.equal(out, torch.tensor(case["suffix"], dtype=torch.float32))


@pytest.mark.parametrize("shape", SHAPES)
def test_fp32_matches_oracle(shape, device):
    bsz, count, rank = shape
    mats, _ = oscan.make_scan_inputs(bsz, count, rank, kind="randn", seed=0)
    out = _scan(mats, device)
    assert out.shape == (bsz, count + 1, rank, rank)
    assert out.dtype == torch.float32
    assert torch.equal(out[:, count], torch.eye(rank).expand(bsz, rank, rank))
    truth = oscan.suffix_scan_sequential(mats, dtype=torch.float64)
    assert _rel_err(out, truth) <= 1e-5  # bar for the fp32 scan
    # The reference's CPU algorithm (log-depth order) agrees to the same bar.
    levels = oscan.suffix_scan_levels(mats)
    assert _rel_err(out, levels.double()) <= 1e-5
    # Sequential fp32 product has the SAME association order as the kernel.
    seq = oscan.suffix_scan_sequential(mats)
    assert torch.allclose(out, seq, atol=2e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 8, 64), (2, 5, 256), (3, 4, 24), (2, 6, 128), (2, 9, 32)])
def test_low_precision_storage_promotes_to_fp32(shape, dtype, device):
    # reference tests/test_interface_scan.py:104-115
    bsz, count, rank = shape
    mats, _ = oscan.make_scan_inputs(bsz, count, rank, kind="randn", seed=0)
    mats = mats.to(dtype)
    out = _scan(mats, device)
    assert out.dtype == torch.float32
    truth = oscan.suffix_scan_sequential(mats.float(), dtype=torch.float64)
    # Inputs are rounded before both sides see them, so only fp32 accumulation differs.
    bar = BF16_D256_BAR if (dtype == torch.bfloat16 and rank == 256) else 1e-5
    assert _rel_err(out, truth) <= bar
    assert torch.allclose(out, oscan.suffix_scan_sequential(mats.float()), atol=2e-1, rtol=5e-3)
    from latent_bounded_interfaces_amd.hip.interface import suffix_scan_pullbacks

    exact = suffix_scan_pullbacks(mats.to(device), exact_suffix=True).cpu()
    assert _rel_err(exact, truth) <= 1e-5


def test_permutations_are_exact(device):
    gen = torch.Generator().manual_seed(5)
    rank, count = 64, 9
    perms = [torch.randperm(rank, generator=gen) for _ in range(count)]
    mats = torch.stack([torch.eye(rank)[p] for p in perms]).unsqueeze(0).repeat(3, 1, 1, 1)
    out = _scan(mats, device)
    idx = torch.arange(rank)
    for r in range(count - 1, -1, -1):
        idx = idx[perms[r]]
        assert torch.equal(out[1, r], torch.eye(rank)[idx])


@pytest.mark.parametrize("shape", [(1, 0, 3), (2, 1, 8), (3, 5, 7), (4, 8, 32), (2, 6, 64), (3, 9, 128),
                                   (5, 12, 256), (2, 3, 100), (2, 4, 260), (2, 0, 256), (3, 1, 256), (1, 2, 256)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_cotangent_chain_matches_oracle(shape, dtype, device):
    from latent_bounded_interfaces_amd.hip.interface import suffix_scan_cotangents

    bsz, count, rank = shape
    mats, g = oscan.make_scan_inputs(bsz, count, rank, kind="randn", seed=1)
    mats = mats.to(dtype)
    out = suffix_scan_cotangents(mats.to(device), g.to(device)).cpu()
    assert out.shape == (bsz, count + 1, rank) and out.dtype == torch.float32
    assert torch.equal(out[:, count], g)
    truth = oscan.suffix_cotangents_sequential(mats.double(), g.double())
    scale = truth.abs().amax(dim=2, keepdim=True).clamp_min(1e-30)
    assert float(((out.double() - truth).abs() / scale).max()) <= 1e-5
    case = GOLDEN["order_case_2x2"]
    got = suffix_scan_cotangents(torch.tensor(case["mats"]).to(device), torch.tensor(case["g"]).to(device))
    assert torch.equal(got.cpu(), torch.tensor(case["cotangents"]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("bsz,count", [(1, 2), (3, 5), (13, 128), (64, 128), (64, 9), (65, 11)])
def test_cotangent_chain_on_four_workgroups_per_element(bsz, count, dtype, device):
    """d = 256 with at most a quarter as many chains as CUs: four workgroups share a chain and exchange each step's
    vector through the result array (marker words).  Against the fp64 chain, terminal cotangent in place, no marker
    left behind, reruns bit-identical; 65 chains take the one-workgroup kernel and must agree to rounding."""
    from latent_bounded_interfaces_amd.hip.interface import suffix_scan_cotangents

    mats, g = oscan.make_scan_inputs(bsz, count, 256, kind="near_identity", seed=21)
    mats_d, g_d = mats.to(device).to(dtype), g.to(device)
    out = suffix_scan_cotangents(mats_d, g_d)
    assert torch.equal(out, suffix_scan_cotangents(mats_d, g_d)), "reruns differ"
    assert bool(torch.isfinite(out).all()) and torch.equal(out[:, count], g_d)
    truth = oscan.suffix_cotangents_sequential(mats_d.double().cpu(), g.double())
    scale = truth.abs().amax(dim=2, keepdim=True).clamp_min(1e-30)
    assert float(((out.cpu().double() - truth).abs() / scale).max()) <= 1e-5


def test_cotangent_chain_partner_timeout_path_in_subprocess(device):
    """A reader that gives up on its partners (forced from the host: LBI_COT_SPIN_LIMIT=0, no poll ever succeeds in
    time) forms every missing entry itself: every wave still reaches every barrier and the chain is still right, in
    the cotangent-only kernel and in the chain waves of the fused bf16 scan."""
    import os
    import subprocess
    import sys

    code = (
        "import torch, sys; sys.path.insert(0, %r);"
        "from oracle import scan as o;"
        "from latent_bounded_interfaces_amd.hip.interface import suffix_scan_cotangents as f;"
        "worst = 0.0\n"
        "from latent_bounded_interfaces_amd.hip.interface import suffix_scan_pullbacks_and_cotangents as fused\n"
        "for dt in (torch.float32, torch.bfloat16):\n"
        "    m, g = o.make_scan_inputs(5, 23, 256, kind='near_identity', seed=3); m = m.to(dt)\n"
        "    out = f(m.cuda(), g.cuda()).cpu().double()\n"
        "    t = o.suffix_cotangents_sequential(m.double(), g.double())\n"
        "    worst = max(worst, float(((out - t).abs() / t.abs().amax(2, keepdim=True)).max()))\n"
        "m, g = o.make_scan_inputs(20, 7, 256, kind='near_identity', seed=4); m = m.to(torch.bfloat16)\n"
        "mats, cot = fused(m.cuda(), g.cuda())\n"
        "t = o.suffix_cotangents_sequential(m.double(), g.double())\n"
        "worst = max(worst, float(((cot.cpu().double() - t).abs() / t.abs().amax(2, keepdim=True)).max()))\n"
        "tm = o.suffix_scan_sequential(m.float(), dtype=torch.float64)\n"
        "assert float(((mats.cpu().double() - tm).abs().flatten(2).amax(2) / tm.abs().flatten(2).amax(2)).max()) <= 2e-4\n"
        "print(worst); sys.exit(0 if worst <= 1e-5 else 1)"
    ) % str(Path(__file__).resolve().parents[1])
    env = dict(os.environ, LBI_COT_SPIN_LIMIT="0")
    res = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=110)
    assert res.returncode == 0, res.stdout + res.stderr


@pytest.mark.parametrize("shape", [(1, 0, 3), (2, 1, 8), (3, 5, 7), (4, 8, 32), (2, 6, 64), (3, 9, 128), (5, 12, 256),
                                   (9, 1, 256), (2, 2, 32), (2, 3, 100), (1, 1, 64), (2, 3, 512), (1, 2, 300)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_fused_scan_and_cotangents(shape, dtype, device):
    """One pass giving both results equals the two separate entry points (bit-exact for the
    matrices) and the oracle for the cotangents."""
    from latent_bounded_interfaces_amd.hip.interface import (
        suffix_scan_pullbacks,
        suffix_scan_pullbacks_and_cotangents,
    )

    bsz, count, rank = shape
    mats, g = oscan.make_scan_inputs(bsz, count, rank, kind="randn", seed=4)
    mats = mats.to(dtype)
    mats_d, g_d = mats.to(device), g.to(device)
    out, cot = suffix_scan_pullbacks_and_cotangents(mats_d, g_d)
    assert torch.equal(out, suffix_scan_pullbacks(mats_d))
    assert cot.shape == (bsz, count + 1, rank) and cot.dtype == torch.float32
    assert torch.equal(cot[:, count].cpu(), g)
    truth = oscan.suffix_cotangents_sequential(mats.double(), g.double())
    scale = truth.abs().amax(dim=2, keepdim=True).clamp_min(1e-30)
    assert float(((cot.cpu().double() - truth).abs() / scale).max()) <= 1e-5


@pytest.mark.parametrize("shape", [(2, 5, 256), (9, 1, 256), (3, 12, 256), (2, 6, 64), (17, 9, 256), (64, 3, 256),
                                   (65, 3, 256)])
def test_fused_scan_and_cotangents_bf16_storage(shape, device):
    """bf16 storage at d=256: the matrices-only entry runs the column-owner kernel; the fused entry the same kernel
    with chain waves (up to 64 batch elements: the four workgroups of an element exchange the chain vector) or the
    row-owner split kernel (larger batches); with ``exact_suffix`` both are exact-split fp32 products in different
    summation orders, by default the suffix operand is rounded to 16 significand bits in both."""
    from latent_bounded_interfaces_amd.hip.interface import (
        suffix_scan_pullbacks,
        suffix_scan_pullbacks_and_cotangents,
    )

    bsz, count, rank = shape
    mats, g = oscan.make_scan_inputs(bsz, count, rank, kind="randn", seed=6)
    mats = mats.to(torch.bfloat16)
    mats_d, g_d = mats.to(device), g.to(device)
    out, cot = suffix_scan_pullbacks_and_cotangents(mats_d, g_d)
    truth = oscan.suffix_scan_sequential(mats.float(), dtype=torch.float64)
    bar = BF16_D256_BAR if rank == 256 else 1e-5
    assert _rel_err(out.cpu(), truth) <= bar
    assert _rel_err(suffix_scan_pullbacks(mats_d).cpu(), truth) <= bar
    want = oscan.suffix_cotangents_sequential(mats.double(), g.double())
    scale = want.abs().amax(dim=2, keepdim=True).clamp_min(1e-30)
    assert float(((cot.cpu().double() - want).abs() / scale).max()) <= 1e-5  # the chain itself is fp32 throughout
    out3, cot3 = suffix_scan_pullbacks_and_cotangents(mats_d, g_d, exact_suffix=True)
    assert _rel_err(out3.cpu(), truth) <= BF16_D256_EXACT_BAR
    assert _rel_err(suffix_scan_pullbacks(mats_d, exact_suffix=True).cpu(), truth) <= BF16_D256_EXACT_BAR
    assert torch.equal(cot3, cot)
    if shape == (2, 5, 256):                   # (short chains of few elements; long ones run the fp32 chunked form)
        assert not torch.equal(out3, out)      # the flag does select another kernel instantiation


def test_benchmark_shape_properties(device):
    """B=64, K=128, d=256: size-independent checks (recurrence, identity tail, reruns bit-stable)."""
    from latent_bounded_interfaces_amd.hip.interface import suffix_scan_cotangents, suffix_scan_pullbacks

    bsz, count, rank = 64, 128, 256
    mats, g = oscan.make_scan_inputs(bsz, count, rank, kind="near_identity", seed=0)
    mats_d = mats.to(device)
    out = suffix_scan_pullbacks(mats_d)
    again = suffix_scan_pullbacks(mats_d)
    assert torch.equal(out, again), "reruns differ"
    assert torch.equal(out[:, count], torch.eye(rank, device=device).expand(bsz, rank, rank))
    # out[r] == mats[r] @ out[r+1] for a sample of r, checked in fp64 on the device.
    for r in (0, 1, 63, 126, 127):
        want = torch.matmul(mats_d[:, r].double(), out[:, r + 1].double())
        err = (out[:, r].double() - want).abs().amax() / want.abs().amax()
        assert float(err) <= 2e-6, (r, float(err))
    # Full fp64 truth for two batch elements on the CPU.
    pick = [0, 37]
    truth = oscan.suffix_scan_sequential(mats[pick], dtype=torch.float64)
    assert _rel_err(out[pick].cpu(), truth) <= 1e-5
    # Cotangents: chain == suffix matrices applied to g (the reference's interface_scan_rms check,
    # backward/scan.py:63-72, bar 1e-5 RMS).
    from latent_bounded_interfaces_amd.hip.interface import suffix_scan_pullbacks_and_cotangents

    g_d = g.to(device)
    chain = suffix_scan_cotangents(mats_d, g_d)
    via_mats = torch.einsum("bkij,bj->bki", out.double(), g_d.double())
    rms = float(torch.sqrt(((chain.double() - via_mats) ** 2).mean()))
    assert rms < 1e-5
    fused_out, fused_cot = suffix_scan_pullbacks_and_cotangents(mats_d, g_d)
    assert torch.equal(fused_out, out)
    assert float(torch.sqrt(((fused_cot.double() - via_mats) ** 2).mean())) < 1e-5
    # bf16 storage, fp32 accumulate: inputs are rounded to bf16 before either path sees
    # them; bar 2e-2 against the fp32 path on the same (rounded) inputs.
    mats_bf16 = mats_d.to(torch.bfloat16)
    out_bf16 = suffix_scan_pullbacks(mats_bf16)
    out_ref = suffix_scan_pullbacks(mats_bf16.float())
    rel = (out_bf16 - out_ref).abs().flatten(2).amax(dim=2) / out_ref.abs().flatten(2).amax(dim=2)
    assert float(rel.max()) <= 2e-2
    truth_bf = oscan.suffix_scan_sequential(mats_bf16[pick].float().cpu(), dtype=torch.float64)
    assert _rel_err(out_bf16[pick].cpu(), truth_bf) <= BF16_D256_BAR


@pytest.mark.parametrize("bsz", [1, 2, 4, 8])
@pytest.mark.parametrize("kind", ["near_identity", "randn"])
def test_k_parallel_scan_at_small_batches(bsz, kind, device):
    """K=128, d=256 with so few batch elements that the chain is cut into chunks that run side by side
    (three launches): same results as the sequential product to the fp32 bar, identity tail, cotangents,
    reruns bit-identical, fused entry == matrices-only entry."""
    from latent_bounded_interfaces_amd.hip.interface import (suffix_scan_pullbacks,
                                                             suffix_scan_pullbacks_and_cotangents)

    count, rank = 128, 256
    mats, g = oscan.make_scan_inputs(bsz, count, rank, kind=kind, seed=7)
    mats_d, g_d = mats.to(device), g.to(device)
    out = suffix_scan_pullbacks(mats_d)
    assert torch.equal(out, suffix_scan_pullbacks(mats_d)), "reruns differ"
    assert torch.equal(out[:, count], torch.eye(rank, device=device).expand(bsz, rank, rank))
    assert torch.equal(out[:, count - 1], mats_d[:, count - 1])
    truth = oscan.suffix_scan_sequential(mats, dtype=torch.float64)
    assert _rel_err(out.cpu(), truth) <= 1e-5
    fused, cot = suffix_scan_pullbacks_and_cotangents(mats_d, g_d)
    assert torch.equal(fused, out)
    assert torch.equal(cot[:, count].cpu(), g)
    want = oscan.suffix_cotangents_sequential(mats.double(), g.double())
    scale = want.abs().amax(dim=2, keepdim=True).clamp_min(1e-30)
    assert float(((cot.cpu().double() - want).abs() / scale).max()) <= 1e-5
    again = suffix_scan_pullbacks_and_cotangents(mats_d, g_d)
    assert torch.equal(again[0], fused) and torch.equal(again[1], cot)


# chains long enough to be cut, at every matrix-core width the chunked form runs, lengths that leave a ragged or
# one-matrix last chunk, batch sizes either side of the 8-chain launch mapping
K_PARALLEL_SHAPES = [(1, 13, 32), (1, 37, 64), (2, 100, 128), (3, 61, 256), (1, 12, 256), (1, 129, 256), (9, 33, 32),
                     (7, 50, 64), (2, 17, 100), (1, 40, 200),
                     # chunk boundaries sit at cL - 1: lengths that make the last chunk one matrix, a full chunk, and
                     # the shortest chains the planner cuts
                     (1, 15, 256), (1, 16, 256), (2, 47, 256), (1, 255, 128), (4, 128, 32), (1, 14, 64)]


@pytest.mark.parametrize("shape", K_PARALLEL_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_k_parallel_scan_shapes(shape, dtype, device):
    from latent_bounded_interfaces_amd.hip.interface import suffix_scan_pullbacks_and_cotangents

    bsz, count, rank = shape
    mats, g = oscan.make_scan_inputs(bsz, count, rank, kind="randn", seed=8)
    mats = mats.to(dtype)
    out, cot = suffix_scan_pullbacks_and_cotangents(mats.to(device), g.to(device))
    truth = oscan.suffix_scan_sequential(mats.float(), dtype=torch.float64)
    assert torch.equal(out[:, count].cpu(), torch.eye(rank).expand(bsz, rank, rank))
    assert _rel_err(out.cpu(), truth) <= 1e-5
    # The chunks share no chain, so these cotangents are the finished products applied to g, which is how the
    # reference gets them (backward/suffix_scan.py:49-53): the 1e-5 of a product can be amplified where the
    # mat-vec cancels, hence 3e-5 per vector here, and the reference's own bar for this quantity, an RMS
    # difference to the sequential chain below 1e-5 (backward/scan.py:63-72, tests/test_lbi_gradient_parity.py:44).
    want = oscan.suffix_cotangents_sequential(mats.double(), g.double())
    scale = want.abs().amax(dim=2, keepdim=True).clamp_min(1e-30)
    assert float(((cot.cpu().double() - want).abs() / scale).max()) <= 3e-5
    assert float(torch.sqrt((((cot.cpu().double() - want) / scale) ** 2).mean())) <= 1e-5


@pytest.mark.parametrize("shape", [(1, 1000, 64), (1, 520, 256), (3, 300, 128)])
def test_k_parallel_scan_long_chains(shape, device):
    """Chains of hundreds of matrices (many chunks: five or six levels over the chunk totals) on the benchmark's
    near-identity inputs: every product against the fp64 sequential product, the identity tail, reruns bit for
    bit, and the fused cotangents against the fp64 chain."""
    from latent_bounded_interfaces_amd.hip.interface import suffix_scan_pullbacks, suffix_scan_pullbacks_and_cotangents

    bsz, count, rank = shape
    mats, g = oscan.make_scan_inputs(bsz, count, rank, kind="near_identity", seed=9)
    out, cot = suffix_scan_pullbacks_and_cotangents(mats.to(device), g.to(device))
    truth = oscan.suffix_scan_sequential(mats, dtype=torch.float64)
    assert torch.equal(out[:, count].cpu(), torch.eye(rank).expand(bsz, rank, rank))
    assert _rel_err(out.cpu(), truth) <= 1e-5
    assert torch.equal(out, suffix_scan_pullbacks(mats.to(device)))
    want = oscan.suffix_cotangents_sequential(mats.double(), g.double())
    scale = want.abs().amax(dim=2, keepdim=True).clamp_min(1e-30)
    assert float(((cot.cpu().double() - want).abs() / scale).max()) <= 3e-5


@pytest.mark.parametrize("chunk,totals_chain", [(0, 0), (2, 0), (3, 0), (5, 0), (16, 0), (3, 1), (5, 1)])
def test_k_parallel_scan_forced_chunk_lengths_in_subprocess(chunk, totals_chain, device):
    """LBI_SCAN_CHUNK forces the chunk length (0: the plain chain): every cut of K=13 / 29 / 33 / 64, including a
    one-matrix last chunk, meets the bar, with and without the cotangent chain.  The products of the chunk totals
    are formed in log depth where there are eight chunks or more and chunks of three matrices or more (chunk
    lengths 3 and 5 at K = 33 / 64 here; length 3 uses the last free slot of a chunk), as one chain otherwise;
    LBI_SCAN_TOTALS_CHAIN=1 forces the chain."""
    import os
    import subprocess
    import sys

    code = (
        "import torch, sys; sys.path.insert(0, %r);"
        "from oracle import scan as o;"
        "from latent_bounded_interfaces_amd.hip.interface import suffix_scan_pullbacks as s, "
        "suffix_scan_pullbacks_and_cotangents as f;"
        "worst = 0.0\n"
        "for shape in ((1, 13, 64), (2, 33, 256), (1, 64, 32), (3, 21, 128), (1, 29, 256)):\n"
        "    m, g = o.make_scan_inputs(*shape, kind='randn', seed=5)\n"
        "    t = o.suffix_scan_sequential(m, dtype=torch.float64)\n"
        "    c = o.suffix_cotangents_sequential(m.double(), g.double())\n"
        "    out, cot = f(m.cuda(), g.cuda())\n"
        "    assert torch.equal(out, s(m.cuda()))\n"
        "    worst = max(worst, float(((out.cpu().double() - t).abs().flatten(2).amax(2) / t.abs().flatten(2).amax(2)).max()))\n"
        "    worst = max(worst, float(((cot.cpu().double() - c).abs() / c.abs().amax(2, keepdim=True)).max()))\n"
        "print(worst); sys.exit(0 if 0.0 < worst <= 1e-5 else 1)"
    ) % str(Path(__file__).resolve().parents[1])
    env = dict(os.environ, LBI_SCAN_CHUNK=str(chunk), LBI_SCAN_TOTALS_CHAIN=str(totals_chain))
    res = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=110)
    assert res.returncode == 0, res.stdout + res.stderr


@pytest.mark.parametrize("shape", [(1, 1, 1), (2, 4, 5), (3, 6, 16), (2, 9, 64), (1, 3, 100), (2, 5, 256), (1, 2, 300)])
def test_suffix_apply_matches_einsum(shape, device):
    """``lbi_suffix_apply``: every matrix of a stack applied to its batch element's vector, in fp64 on the CPU."""
    from latent_bounded_interfaces_amd.hip.interface import suffix_apply

    bsz, count, rank = shape
    gen = torch.Generator().manual_seed(rank)
    suffix = torch.randn(bsz, count, rank, rank, generator=gen)
    g = torch.randn(bsz, rank, generator=gen)
    got = suffix_apply(suffix.to(device), g.to(device)).cpu()
    want = torch.einsum("bkij,bj->bki", suffix.double(), g.double())
    assert got.shape == (bsz, count, rank) and got.dtype == torch.float32
    assert torch.allclose(got.double(), want, atol=1e-5 * float(want.abs().max()), rtol=1e-5)
    with pytest.raises(ValueError):
        suffix_apply(suffix.to(device), g[:, :-1].to(device)) if rank > 1 else suffix_apply(suffix[0].to(device), g.to(device))


def test_backward_module_contract(device):
    """Counterpart functions of reference backward/suffix_scan.py keep its edge cases."""
    from latent_bounded_interfaces_amd.backward import suffix_scan as bs

    mats, g = oscan.make_scan_inputs(3, 5, 16, kind="randn", seed=2)
    jts = [mats[:, r].to(device) for r in range(5)]
    g_d = g.to(device)
    suffix = bs.compose_suffix_jacobian_t(jts)
    assert len(suffix) == 6 and all(s.shape == (3, 16, 16) and s.is_contiguous() for s in suffix)
    truth = oscan.suffix_scan_sequential(mats, dtype=torch.float64)
    assert _rel_err(torch.stack([s.cpu() for s in suffix], 1), truth) <= 1e-5
    assert bs.compose_suffix_jacobian_t([]) == []
    with pytest.raises(ValueError):
        bs.compose_suffix_jacobian_t([torch.zeros(2, 3, 4, device=device)])
    want = oscan.suffix_cotangents_sequential(mats.double(), g.double())
    for flag in (False, True):
        got = bs.propagate_state_adjoint_with_jacobian_scan(jts, g_d, materialize_suffix=flag)
        assert len(got) == 6
        assert torch.allclose(torch.stack([x.cpu() for x in got], 1).double(), want, atol=1e-5, rtol=1e-5)
    # Drop-last rule and the 0 / 1 region cases.
    got = bs.propagate_state_adjoint_from_last_region_input(jts, g_d, num_regions=5)
    want4 = oscan.suffix_cotangents_sequential(mats[:, :4].double(), g.double())
    assert len(got) == 5
    assert torch.allclose(torch.stack([x.cpu() for x in got], 1).double(), want4, atol=1e-5, rtol=1e-5)
    assert bs.propagate_state_adjoint_from_last_region_input([], g_d, num_regions=0) == []
    assert bs.propagate_state_adjoint_from_last_region_input(jts[:1], g_d, num_regions=1)[0] is g_d
    with pytest.raises(ValueError):
        bs.propagate_state_adjoint_from_last_region_input(jts, g_d, num_regions=4)
    one = bs.apply_jacobian_t(jts[0], g_d)
    assert torch.allclose(one.cpu(), torch.einsum("bij,bj->bi", mats[:, 0], g), atol=1e-5, rtol=1e-5)
    stats = bs.interface_state_jacobian_t_stats(jts, include_suffix=True)
    assert {"jac_local_spec_mean", "jac_suffix_spec_max"} <= set(stats)


def test_split_fp32_variant_in_subprocess(device):
    """The opt-in bf16-split kernel for fp32 storage (LBI_SCAN_SPLIT_FP32=1) meets the same bar."""
    import os
    import subprocess
    import sys

    code = (
        "import torch, sys; sys.path.insert(0, %r);"
        "from oracle import scan as o;"
        "from latent_bounded_interfaces_amd.hip.interface import suffix_scan_pullbacks_and_cotangents as f;"
        "m, g = o.make_scan_inputs(3, 9, 256, kind='randn', seed=5);"
        "out, cot = f(m.cuda(), g.cuda());"
        "t = o.suffix_scan_sequential(m, dtype=torch.float64);"
        "e = float(((out.cpu().double() - t).abs().flatten(2).amax(2) / t.abs().flatten(2).amax(2)).max());"
        "c = o.suffix_cotangents_sequential(m.double(), g.double());"
        "ec = float(((cot.cpu().double() - c).abs() / c.abs().amax(2, keepdim=True)).max());"
        "print(e, ec); sys.exit(0 if e <= 1e-5 and ec <= 1e-5 else 1)"
    ) % str(Path(__file__).resolve().parents[1])
    env = dict(os.environ, LBI_SCAN_SPLIT_FP32="1")
    res = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=110)
    assert res.returncode == 0, res.stdout + res.stderr


@pytest.mark.parametrize("kind", ["near_identity", "randn"])
def test_bf16_storage_at_the_benchmark_shape_in_both_precisions(kind, device):
    """B=64, K=128, d=256 with bf16 storage, every suffix matrix of every batch element against the sequential
    product in fp64 (on the device) and against this library's fp32 path on the same rounded inputs.  Default (suffix
    operand rounded to 16 significand bits): <= 1e-3 against fp64 and <= 2e-2 against the fp32 path, the bar for
    16-bit storage; ``exact_suffix``: the rounding of fp32 accumulation alone (<= 2e-5 over all 8192 products of 128
    factors; 1e-5 on the shorter chains of the other tests).  Both entries (column-owner kernel for the matrices alone,
    row-owner kernel with the cotangent chain), reruns bit-identical."""
    from latent_bounded_interfaces_amd.hip.interface import (suffix_scan_pullbacks,
                                                             suffix_scan_pullbacks_and_cotangents)

    bsz, count, rank = 64, 128, 256
    mats, g = oscan.make_scan_inputs(bsz, count, rank, kind=kind, seed=11)
    mats_d, g_d = mats.to(device).to(torch.bfloat16), g.to(device)
    truth = oscan.suffix_scan_sequential(mats_d.double(), dtype=torch.float64)     # fp64 on the device
    scale = truth.abs().flatten(2).amax(dim=2).clamp_min(1e-300)

    def worst(out):
        return float(((out.double() - truth).abs().flatten(2).amax(dim=2) / scale).max())

    fp32_path = suffix_scan_pullbacks(mats_d.float())
    assert worst(fp32_path) <= 1e-5
    ref_scale = fp32_path.abs().flatten(2).amax(dim=2).clamp_min(1e-30)
    for exact, bar in ((False, 1e-3), (True, 2e-5)):
        only = suffix_scan_pullbacks(mats_d, exact_suffix=exact)
        fused, cot = suffix_scan_pullbacks_and_cotangents(mats_d, g_d, exact_suffix=exact)
        for out in (only, fused):
            err = worst(out)
            assert err <= bar, (kind, exact, err)
            assert float(((out - fp32_path).abs().flatten(2).amax(dim=2) / ref_scale).max()) <= 2e-2
            assert torch.equal(out[:, count], torch.eye(rank, device=device).expand(bsz, rank, rank))
        assert torch.equal(only, suffix_scan_pullbacks(mats_d, exact_suffix=exact)), "reruns differ"
        want = torch.einsum("bkij,bj->bki", truth, g_d.double())
        cscale = want.abs().amax(dim=2, keepdim=True).clamp_min(1e-300)
        assert float(((cot.double() - want).abs() / cscale).max()) <= 1e-5
        del only, fused, cot
