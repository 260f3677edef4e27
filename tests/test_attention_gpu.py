"""Parity of the HIP attention input-pullback against the CPU oracle, through the C ABI (needs the GPU)."""
from __future__ import annotations

import json
import math
from pathlib import Path

import pytest
import torch

from oracle import attention as oattn

pytestmark = pytest.mark.gpu

GOLDEN = json.loads((Path(__file__).parent / "golden" / "attention_known_answers.json").read_text())


def _run(q, k, v, g, device, *, scale, causal, mode="hip"):
    from latent_bounded_interfaces_amd.hip.transformer import attention_input_pullback_basis

    args = [t.to(device) for t in (q, k, v, g)]
    keep = [t.clone() for t in args]
    out = attention_input_pullback_basis(*args, softmax_scale=scale, causal=causal, kernel_mode=mode)
    torch.cuda.synchronize()
    for a, b in zip(args, keep):
        assert torch.equal(a, b), "input was modified"
    return tuple(t.cpu() for t in out)


def _max_rel(actual, truth):
    """max|diff| / max|truth| over a whole tensor."""
    return float((actual.double() - truth.double()).abs().max() / truth.double().abs().max().clamp_min(1e-30))


@pytest.mark.parametrize("case", ["two_keys_equal", "single_token"])
def test_known_answers(case, device):
    c = GOLDEN[case]
    q, k, v, g = (torch.tensor(c[n], dtype=torch.float32) for n in ("q", "k", "v", "d_out"))
    got = _run(q, k, v, g, device, scale=c["softmax_scale"], causal=c["causal"])
    for name, t in zip(("dq", "dk", "dv"), got):
        assert torch.allclose(t, torch.tensor(c[name]), atol=2e-5), name  # the fp32 bar of the reference tests


# fp32 cases of the reference's tests (tests/test_cuda_attention_pullback.py:62-66, 86-90, 115-119)
# plus ragged ones (T not a multiple of the 16-wide tile, odd head dims, T=1).
FP32_CASES = [
    (101, (2, 3, 5, 4), 2), (103, (1, 2, 4, 3), 3), (117, (1, 2, 4, 16), 3),
    (5, (1, 1, 1, 8), 2), (6, (2, 2, 17, 5), 1), (7, (1, 3, 33, 24), 2), (8, (1, 2, 40, 72), 3),
    (9, (1, 1, 64, 64), 2), (10, (1, 2, 19, 130), 1),
]


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("seed,shape,basis", FP32_CASES)
def test_fp32_matches_oracle(seed, shape, basis, causal, device):
    torch.manual_seed(seed)
    q = torch.randn(*shape)
    k = torch.randn_like(q)
    v = torch.randn_like(q)
    g = torch.randn(shape[0], basis, *shape[1:])
    scale = 1.0 / math.sqrt(shape[-1])
    got = _run(q, k, v, g, device, scale=scale, causal=causal)
    want = oattn.attention_pullback_sdpa_loop(q, k, v, g, softmax_scale=scale, causal=causal)
    truth = oattn.attention_pullback_dense(q, k, v, g, softmax_scale=scale, causal=causal, dtype=torch.float64)
    for a, b, c in zip(got, want, truth):
        assert a.shape == g.shape and a.dtype == torch.float32
        assert torch.allclose(a, b, atol=2e-5, rtol=2e-5)  # the reference's fp32 bar
        assert torch.allclose(a.double(), c, atol=2e-5, rtol=2e-5)


# 16-bit storage: the MFMA kernels (T % 64 == 0, Dh in {64, 128}; one fused launch for Dh = 64, T <= 128) and the
# generic ones otherwise.
# (121, (1, 2, 16, 64), P) are the reference's fp16 cases (tests/test_cuda_attention_pullback.py:178-243);
# (8, 8, 128, 64) with P=4 is the reference benchmark shape.
LOWP_CASES = [
    (121, (1, 2, 16, 64), 1), (129, (1, 2, 16, 64), 4), (11, (2, 2, 64, 64), 2), (12, (1, 3, 128, 128), 3),
    (13, (2, 1, 192, 64), 5), (14, (1, 2, 320, 128), 2), (15, (1, 1, 576, 128), 1), (16, (8, 8, 128, 64), 4),
    (17, (1, 2, 96, 64), 2), (18, (1, 1, 64, 32), 2), (19, (1, 2, 256, 64), 9), (20, (1, 1, 448, 64), 16),
    # lengths that are no multiple of 64: causal calls are padded onto the matrix-core kernels
    (21, (2, 2, 100, 64), 3), (22, (1, 1, 1000, 128), 2), (23, (1, 2, 33, 64), 2),
    # head dims below 128 that are not 64: zero-padded onto the matrix-core kernels (with the length, if causal)
    (24, (1, 2, 128, 32), 3), (25, (2, 1, 192, 96), 2), (26, (1, 2, 70, 80), 2), (27, (1, 1, 64, 8), 1),
    (28, (1, 1, 128, 160), 2),  # past 128: generic kernels
    # lengths up to 256 at head dim 64 and up to 128 at head dim 128: the single-launch kernel
    # (so are 11, 12, 13, 16, 17, 19 above and, once padded, the causal runs of 21, 23, 24, 27)
    (29, (1, 2, 32, 64), 3), (30, (3, 1, 128, 64), 1), (31, (2, 3, 96, 64), 5), (32, (1, 2, 160, 64), 2),
    (33, (2, 1, 64, 128), 3), (34, (1, 1, 96, 128), 2), (35, (1, 2, 224, 64), 1), (36, (2, 2, 256, 64), 4),
    # the same kernel at lengths that are no multiple of 32 (zero rows in the last tile, keys past the end masked)
    (37, (1, 2, 1, 64), 2), (38, (2, 1, 255, 64), 3), (39, (1, 2, 127, 128), 2), (40, (1, 1, 31, 64), 1),
    (41, (2, 2, 129, 64), 2), (42, (1, 1, 5, 128), 3),
    # past the single-launch limits with direction counts that leave the kernels a ragged tail: a last dQ group of
    # fewer than 8 (Dh = 64) or 4 (Dh = 128) directions, a last dK/dV group of fewer than 4 (Dh = 64, two directions
    # per wave) or an unpaired last direction (Dh = 128)
    (43, (1, 2, 320, 64), 5), (44, (1, 1, 320, 64), 9), (45, (1, 2, 192, 128), 3), (46, (1, 1, 320, 128), 5),
    (47, (1, 1, 384, 64), 11), (48, (2, 1, 192, 128), 7), (49, (1, 1, 512, 64), 3), (50, (1, 1, 256, 128), 9),
    (51, (1, 2, 320, 64), 6), (52, (2, 1, 384, 64), 7), (53, (1, 3, 576, 64), 4), (54, (1, 1, 320, 64), 2),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("seed,shape,basis", LOWP_CASES)
def test_low_precision_matches_oracle(seed, shape, basis, causal, dtype, device):
    q, k, v, g = oattn.make_attention_inputs(*shape, basis, dtype=dtype, seed=seed)
    scale = 1.0 / math.sqrt(shape[-1])
    got = _run(q, k, v, g, device, scale=scale, causal=causal)
    # fp32 path on the same (already rounded) inputs
    truth = oattn.attention_pullback_blocked(q, k, v, g, softmax_scale=scale, causal=causal, dtype=torch.float32)
    for name, a, c in zip(("dq", "dk", "dv"), got, truth):
        assert a.shape == g.shape and a.dtype == dtype
        assert _max_rel(a, c) <= 2e-2, (name, _max_rel(a, c))  # bar: <= 2e-2 against the fp32 path
        assert torch.allclose(a.float(), c, atol=3e-2 * float(c.abs().max()), rtol=3e-2), name


def test_four_kernel_path_at_short_lengths_in_subprocess(device):
    """LBI_ATTN_SMALL=0 sends short sequences through the four-kernel path; it meets the same bar."""
    import os
    import subprocess
    import sys

    code = (
        "import math, sys, torch; sys.path.insert(0, %r);"
        "from oracle import attention as o;"
        "from latent_bounded_interfaces_amd.hip.transformer import attention_input_pullback_basis as f;"
        "worst = 0.0\n"
        "for shape, basis, causal in (((2, 2, 64, 64), 2, True), ((8, 8, 128, 64), 4, True), ((1, 2, 128, 64), 3, False),"
        " ((1, 2, 256, 64), 2, True), ((1, 2, 128, 128), 2, True)):\n"
        "    q, k, v, g = o.make_attention_inputs(*shape, basis, dtype=torch.float16, seed=41)\n"
        "    got = f(q.cuda(), k.cuda(), v.cuda(), g.cuda(), softmax_scale=shape[-1] ** -0.5, causal=causal, kernel_mode='hip')\n"
        "    truth = o.attention_pullback_blocked(q, k, v, g, softmax_scale=shape[-1] ** -0.5, causal=causal, dtype=torch.float32)\n"
        "    for a, c in zip(got, truth):\n"
        "        worst = max(worst, float((a.cpu().double() - c.double()).abs().max() / c.double().abs().max()))\n"
        "print(worst); sys.exit(0 if 0.0 < worst <= 2e-2 else 1)"
    ) % str(Path(__file__).resolve().parents[1])
    env = dict(os.environ, LBI_ATTN_SMALL="0")
    res = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=110)
    assert res.returncode == 0, res.stdout + res.stderr


def test_modes_and_contract(device):
    from latent_bounded_interfaces_amd.backends import HipTransformerLowering
    from latent_bounded_interfaces_amd.hip.transformer import attention_input_pullback_basis

    q, k, v, g = (t.to(device) for t in oattn.make_attention_inputs(1, 2, 16, 64, 4, dtype=torch.float16, seed=131))
    scale = 0.125
    base = attention_input_pullback_basis(q, k, v, g, softmax_scale=scale, kernel_mode="hip")
    for mode in ("fa2_loop", "simple", "fa2_mma_pblock4"):
        out = attention_input_pullback_basis(q, k, v, g, softmax_scale=scale, kernel_mode=mode)
        assert all(torch.equal(a, b) for a, b in zip(out, base))
    # P limits of the reference's modes (tests/test_cuda_attention_pullback.py:163-173, 281-291)
    for mode in ("fa2_p1", "fa2_mma_p1"):
        with pytest.raises(ValueError, match="== 1"):
            attention_input_pullback_basis(q, k, v, g, softmax_scale=scale, kernel_mode=mode)
        one = attention_input_pullback_basis(q, k, v, g[:, :1], softmax_scale=scale, kernel_mode=mode)
        assert all(torch.equal(a, b[:, :1]) for a, b in zip(one, base))
    g5 = torch.cat([g, g[:, :1]], dim=1)
    with pytest.raises(ValueError, match="<= 4"):
        attention_input_pullback_basis(q, k, v, g5, softmax_scale=scale)
    with pytest.raises(ValueError, match="unknown attention pullback kernel_mode"):
        attention_input_pullback_basis(q, k, v, g, softmax_scale=scale, kernel_mode="nope")
    with pytest.raises(ValueError):
        attention_input_pullback_basis(q, k[:, :1], v, g, softmax_scale=scale)
    with pytest.raises(ValueError):
        attention_input_pullback_basis(q, k, v, g[:, 0], softmax_scale=scale)
    # lowering wrapper (reference tests/test_cuda_attention_pullback.py:294-315)
    low = HipTransformerLowering()
    assert low.name == "hip"
    out = low.attention_input_pullback_basis(q=q, k=k, v=v, output_cotangent_basis=g, softmax_scale=scale)
    assert all(torch.equal(a, b) for a, b in zip(out, base))
    # the default mode is the reference's (backends/transformer_cuda.py:31) with its limit of four directions;
    # "hip" is the mode without one
    with pytest.raises(ValueError, match="<= 4"):
        low.attention_input_pullback_basis(q=q, k=k, v=v, output_cotangent_basis=g5, softmax_scale=scale)
    out = low.attention_input_pullback_basis(q=q, k=k, v=v, output_cotangent_basis=g5, softmax_scale=scale,
                                             kernel_mode="hip")
    assert all(torch.equal(a[:, :4], b) for a, b in zip(out, base))
    with pytest.raises(RuntimeError, match="no CPU execution path"):
        low.input_pullback_basis(backend=None, cache=None, output_cotangent_basis=torch.zeros(1, 1, 2, 3))
    with pytest.raises(ValueError):
        low.input_pullback_basis(backend=None, cache=None, output_cotangent_basis=torch.zeros(1, 2, 3))
    with pytest.raises(RuntimeError, match="no CPU execution path"):
        low.parameter_vjp(backend=None, cache=None, output_cotangent=torch.zeros(1, 2, 3))
    with pytest.raises(ValueError):
        low.parameter_vjp(backend=None, cache=None, output_cotangent=torch.zeros(1, 2, 3, 4))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape,basis", [((2, 3, 384, 64), 11), ((1, 2, 320, 128), 7), ((1, 2, 1024, 64), 16)])
def test_results_do_not_depend_on_how_directions_are_grouped(shape, basis, dtype, device):
    """A direction's dQ, dK, dV are the same bits whether it is computed alone, in a pair, or among all directions:
    the kernels group directions (eight or four per dQ workgroup, two per dK/dV workgroup, four at head dim 64 with
    a second direction per wave) only to share the S / P tiles; every direction keeps its own products and sums."""
    from latent_bounded_interfaces_amd.hip.transformer import attention_input_pullback_basis

    q, k, v, g = (t.to(device) for t in oattn.make_attention_inputs(*shape, basis, dtype=dtype, seed=77))
    scale = 1.0 / math.sqrt(shape[-1])
    whole = attention_input_pullback_basis(q, k, v, g, softmax_scale=scale, kernel_mode="hip")
    for lo, hi in ((0, 2), (2, 3), (3, 6), (basis - 4, basis), (basis - 1, basis)):
        part = attention_input_pullback_basis(q, k, v, g[:, lo:hi].contiguous(), softmax_scale=scale, kernel_mode="hip")
        for name, a, b in zip(("dq", "dk", "dv"), part, whole):
            assert torch.equal(a, b[:, lo:hi]), (name, lo, hi)


def test_long_context_properties(device):
    """bf16, T=4096, Dh=128, P=16 on two (b, h) slices: size-independent checks."""
    from latent_bounded_interfaces_amd.hip.transformer import attention_input_pullback_basis

    q, k, v, g = (t.to(device) for t in oattn.make_attention_inputs(1, 2, 4096, 128, 16, dtype=torch.bfloat16, seed=0))
    scale = 1.0 / math.sqrt(128)
    dq, dk, dv = attention_input_pullback_basis(q, k, v, g, softmax_scale=scale, kernel_mode="hip")
    again = attention_input_pullback_basis(q, k, v, g, softmax_scale=scale, kernel_mode="hip")
    assert all(torch.equal(a, b) for a, b in zip((dq, dk, dv), again)), "reruns differ"
    # basis independence: direction p alone gives the same slice
    solo = attention_input_pullback_basis(q, k, v, g[:, 5:6].contiguous(), softmax_scale=scale, kernel_mode="hip")
    for a, b in zip(solo, (dq, dk, dv)):
        assert _max_rel(a[:, 0], b[:, 5].float()) <= 2e-2
    # first query row attends one key: dQ there is zero; P=1 slice equals torch's own attention backward
    assert float(dq[:, :, :, 0].abs().max()) <= 1e-5 * float(dq.abs().max())
    qr, kr, vr = (t.float().requires_grad_(True) for t in (q, k, v))
    out = torch.nn.functional.scaled_dot_product_attention(qr, kr, vr, is_causal=True, scale=scale)
    want = torch.autograd.grad(out, (qr, kr, vr), grad_outputs=g[:, 3].float())
    for name, a, b in zip(("dq", "dk", "dv"), (dq, dk, dv), want):
        assert _max_rel(a[:, 3], b) <= 2e-2, (name, _max_rel(a[:, 3], b))


def test_long_context_full_size_slices_match_oracle(device):
    """The whole long-context call (bf16, B=4, H=16, T=4096, Dh=128, P=16: 64 (b, h) pairs, 1 GiB of cotangents,
    3 GiB of results) run once; the first and the last (b, h) pair, two directions each, against per-direction
    SDPA + autograd of that slice in fp32 on the CPU."""
    from latent_bounded_interfaces_amd.hip.transformer import attention_input_pullback_basis

    bsz, heads, seq, hd, basis = 4, 16, 4096, 128, 16
    gen = torch.Generator(device=device).manual_seed(0)
    q, k, v = (torch.randn(bsz, heads, seq, hd, device=device, dtype=torch.bfloat16, generator=gen) for _ in range(3))
    g = torch.randn(bsz, basis, heads, seq, hd, device=device, dtype=torch.bfloat16, generator=gen)
    scale = 1.0 / math.sqrt(hd)
    out = attention_input_pullback_basis(q, k, v, g, softmax_scale=scale, causal=True, kernel_mode="hip")
    torch.cuda.synchronize()
    for (b, h), dirs in (((0, 0), (0, 7)), ((bsz - 1, heads - 1), (basis - 1, 6)), ((2, 5), (9, 12))):
        qs, ks, vs = (t[b:b + 1, h:h + 1].float().cpu() for t in (q, k, v))
        gs = g[b:b + 1, list(dirs), h:h + 1].float().cpu()
        want = oattn.attention_pullback_sdpa_loop(qs, ks, vs, gs, softmax_scale=scale, causal=True)
        for name, a, c in zip(("dq", "dk", "dv"), out, want):
            got = a[b:b + 1, list(dirs), h:h + 1].float().cpu()
            assert _max_rel(got, c) <= 2e-2, (name, b, h, _max_rel(got, c))
