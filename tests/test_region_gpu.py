"""Region-level input pullback on the GPU (through the C ABI) against autograd of the
CPU restatement of the reference's Transformer region."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import transformer_region as oreg

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]


def _tol(dtype):
    return 2e-5 if dtype == torch.float32 else 2e-2


def _max_rel(a, b):
    return float((a.double() - b.double()).abs().max() / b.double().abs().max().clamp_min(1e-30))


def _vjp(fn, inputs, cotangent):
    inputs = [t.detach().double().requires_grad_(True) for t in inputs]
    out = fn(*inputs)
    return torch.autograd.grad(out, inputs, grad_outputs=cotangent.double())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim", [32, 30, 768])
def test_rmsnorm_pullback(dtype, dim, device):
    from latent_bounded_interfaces_amd.hip.transformer import region

    torch.manual_seed(dim)
    b, p, t = 2, 3, 5
    g = torch.randn(b, p, t, dim).to(dtype)
    x = torch.randn(b, t, dim)  # fp32 residual stream
    w = (1 + 0.1 * torch.randn(dim)).to(dtype)
    res = torch.randn(b, p, t, dim)
    total, branch = region.rmsnorm_pullback(g.to(device), x.to(device), w.to(device), 1e-5, res.clone().to(device),
                                            want_branch=True)
    xr = x.to(dtype)  # the norm runs on the input rounded to the weight dtype

    def fwd(xx):
        return xx * torch.rsqrt(xx.pow(2).mean(-1, keepdim=True) + 1e-5) * w.double()

    want = torch.stack([_vjp(fwd, [xr], g[:, i])[0] for i in range(p)], dim=1) + res.double()
    assert total.dtype == torch.float32 and branch.dtype == dtype
    assert _max_rel(total.cpu(), want) <= 2e-5  # fp32 arithmetic on the given (rounded) inputs
    assert _max_rel(branch.cpu(), want) <= _tol(dtype)
    # no residual, fp32 output only
    only, none = region.rmsnorm_pullback(g.to(device), x.to(device), w.to(device), 1e-5, None, want_branch=False)
    assert none is None and _max_rel(only.cpu(), want - res.double()) <= 2e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [24, 27, 3072])
def test_gated_mlp_pullback(dtype, hidden, device):
    from latent_bounded_interfaces_amd.hip.transformer import region

    torch.manual_seed(hidden)
    b, p, t = 2, 2, 3
    g = torch.randn(b, p, t, hidden).to(dtype)
    fc1 = (2 * torch.randn(b, t, 2 * hidden)).to(dtype)
    got = region.gated_mlp_pullback(g.to(device), fc1.to(device)).cpu()

    def fwd(f):
        return f[..., :hidden] * F.silu(f[..., hidden:])

    want = torch.stack([_vjp(fwd, [fc1], g[:, i])[0] for i in range(p)], dim=1)
    assert got.dtype == dtype and got.shape == (b, p, t, 2 * hidden)
    assert _max_rel(got, want) <= _tol(dtype)
    assert torch.allclose(got.double(), want, atol=_tol(dtype) * 4, rtol=_tol(dtype) * 4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,head_dim", [(3, 4), (2, 64), (5, 6)])
def test_heads_split(dtype, heads, head_dim, device):
    from latent_bounded_interfaces_amd.hip.transformer import region

    x = torch.randn(2, 3, 7, heads * head_dim).to(dtype)
    got = region.attn_heads_split(x.to(device), heads, head_dim).cpu()
    assert torch.equal(got, x.view(2, 3, 7, heads, head_dim).permute(0, 1, 3, 2, 4).contiguous())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,head_dim,interleaved",
                         [(4, 4, 8, False), (4, 2, 8, True), (6, 2, 6, False), (3, 1, 2, True), (12, 4, 64, False),
                          (2, 1, 64, True)])
def test_qkv_pullback(dtype, heads, kv_heads, head_dim, interleaved, device):
    from latent_bounded_interfaces_amd.hip.transformer import region

    torch.manual_seed(heads * 100 + head_dim)
    b, p, t = 2, 3, 9
    dq, dk, dv = (torch.randn(b, p, heads, t, head_dim).to(dtype) for _ in range(3))
    got = region.attn_qkv_pullback(dq.to(device), dk.to(device), dv.to(device), n_kv_heads=kv_heads, rope_base=100.0,
                                   rope_interleaved=interleaved).cpu()
    rep = heads // kv_heads

    def fwd(qkv):  # [b, t, (H + 2 Hkv) Dh] -> concatenated (q_rope, k_expanded, v_expanded)
        q, k, v = qkv.split((heads * head_dim, kv_heads * head_dim, kv_heads * head_dim), dim=-1)
        q = q.view(b, t, heads, head_dim).transpose(1, 2)
        k = k.view(b, t, kv_heads, head_dim).transpose(1, 2)
        v = v.view(b, t, kv_heads, head_dim).transpose(1, 2)
        # float64 rotation from the same fp32 tables as the kernel
        cos, sin = (c.double() for c in oreg.rope_tables(t, head_dim, 100.0))

        def rot(x):
            if interleaved:
                a, c = x[..., 0::2], x[..., 1::2]
                return torch.stack((a * cos - c * sin, a * sin + c * cos), dim=-1).flatten(-2)
            a, c = x[..., : head_dim // 2], x[..., head_dim // 2:]
            return torch.cat((a * cos - c * sin, a * sin + c * cos), dim=-1)

        return torch.cat((rot(q), rot(k).repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)), dim=1)

    qkv0 = torch.zeros(b, t, (heads + 2 * kv_heads) * head_dim)
    want = torch.stack([_vjp(fwd, [qkv0], torch.cat((dq[:, i], dk[:, i], dv[:, i]), dim=1))[0] for i in range(p)], dim=1)
    assert got.dtype == dtype and got.shape == want.shape
    assert _max_rel(got, want) <= (1e-6 if dtype == torch.float32 else _tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("channels,ksize,seqlen", [(8, 4, 10), (6, 3, 2), (5, 1, 4), (2304, 4, 7)])
def test_causal_conv1d_pullback(dtype, channels, ksize, seqlen, device):
    from latent_bounded_interfaces_amd.hip.transformer import region

    torch.manual_seed(channels + ksize)
    b, p = 2, 2
    g = torch.randn(b, p, seqlen, channels).to(dtype)
    w = torch.randn(channels, 1, ksize).to(dtype)
    got = region.causal_conv1d_pullback(g.to(device), w.to(device)).cpu()

    def fwd(x):  # [b, T, C]
        return F.conv1d(x.transpose(1, 2), w.double(), padding=ksize - 1, groups=channels)[..., :seqlen].transpose(1, 2)

    want = torch.stack([_vjp(fwd, [torch.zeros(b, seqlen, channels)], g[:, i])[0] for i in range(p)], dim=1)
    assert _max_rel(got, want) <= (1e-6 if dtype == torch.float32 else _tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows_shape,dim,wide_x", [((2, 5), 32, True), ((3, 1, 7), 36, False), ((1, 300), 768, True),
                                                  ((4, 130), 2048, False), ((1, 1), 4, True)])
def test_rmsnorm_weight_grad(dtype, rows_shape, dim, wide_x, device):
    """Autograd of the norm's forward (input rounded to the weight dtype, normalised value rounded again, reference
    backbones/transformer/block.py:18-23) with respect to the weight, in fp64 on the rounded values."""
    from latent_bounded_interfaces_amd.hip.transformer import region

    torch.manual_seed(dim + len(rows_shape))
    g = torch.randn(*rows_shape, dim).to(dtype)
    x = torch.randn(*rows_shape, dim) * 1.7
    x = x if wide_x else x.to(dtype)
    got = region.rmsnorm_weight_grad(g.to(device), x.to(device), 1e-5)
    assert got.dtype == torch.float32 and got.shape == (dim,)
    xr = x.to(dtype).float()
    normed = (xr * torch.rsqrt(xr.pow(2).mean(-1, keepdim=True) + 1e-5)).to(dtype)
    want = (g.double() * normed.double()).reshape(-1, dim).sum(0)
    # the normalised value is rounded to the storage type before the sum: a last-place difference of the fp32
    # rsqrt can move single elements by one storage ulp
    assert _max_rel(got.cpu(), want) <= (2e-5 if dtype == torch.float32 else 2e-3)
    again = region.rmsnorm_weight_grad(g.to(device), x.to(device), 1e-5)
    assert torch.equal(got, again)


def test_rmsnorm_weight_grad_contract(device):
    from latent_bounded_interfaces_amd.hip.transformer import region

    g = torch.zeros(2, 3, 8, device=device)
    with pytest.raises(ValueError):
        region.rmsnorm_weight_grad(g, torch.zeros(2, 3, 4, device=device), 1e-5)
    with pytest.raises(ValueError):
        region.rmsnorm_weight_grad(g.half(), torch.zeros(2, 3, 8, device=device, dtype=torch.bfloat16), 1e-5)
    with pytest.raises(RuntimeError, match="multiple of 4"):
        region.rmsnorm_weight_grad(torch.zeros(2, 6, device=device), torch.zeros(2, 6, device=device), 1e-5)
    empty = region.rmsnorm_weight_grad(torch.zeros(0, 8, device=device), torch.zeros(0, 8, device=device), 1e-5)
    assert torch.equal(empty.cpu(), torch.zeros(8))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bsz,seqlen,channels,ksize", [(2, 10, 8, 4), (3, 2, 6, 3), (1, 4, 5, 1), (2, 130, 2304, 4),
                                                      (1, 70, 12, 8), (2, 3, 7, 5)])
def test_causal_conv1d_weight_grad(dtype, bsz, seqlen, channels, ksize, device):
    """Autograd of Conv1d(groups=C, padding=k-1) cut to the first T outputs (reference
    backends/transformer.py:121-122) with respect to weight and bias, in fp64 on the stored values."""
    from latent_bounded_interfaces_amd.hip.transformer import region

    torch.manual_seed(channels + ksize + seqlen)
    g = torch.randn(bsz, seqlen, channels).to(dtype)
    x = torch.randn(bsz, seqlen, channels).to(dtype)
    g_w, g_b = region.causal_conv1d_weight_grad(g.to(device), x.to(device), ksize)
    assert g_w.shape == (channels, 1, ksize) and g_b.shape == (channels,) and g_w.dtype == torch.float32
    w = torch.zeros(channels, 1, ksize, dtype=torch.float64, requires_grad=True)
    b = torch.zeros(channels, dtype=torch.float64, requires_grad=True)
    y = F.conv1d(x.double().transpose(1, 2), w, b, padding=ksize - 1, groups=channels)[..., :seqlen].transpose(1, 2)
    want_w, want_b = torch.autograd.grad(y, (w, b), grad_outputs=g.double())
    assert _max_rel(g_w.cpu(), want_w) <= 2e-5 and _max_rel(g_b.cpu(), want_b) <= 2e-5
    again = region.causal_conv1d_weight_grad(g.to(device), x.to(device), ksize)
    assert torch.equal(g_w, again[0]) and torch.equal(g_b, again[1])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,head_dim,interleaved,ksize,seqlen",
                         [(4, 2, 8, False, 4, 19), (4, 4, 8, True, 3, 8), (3, 1, 6, False, 4, 5), (3, 1, 2, True, 1, 9),
                          (12, 4, 64, False, 4, 33), (2, 1, 64, True, 7, 12), (2, 2, 16, False, 8, 3)])
def test_qkv_conv_pullback_equals_the_two_calls(dtype, heads, kv_heads, head_dim, interleaved, ksize, seqlen, device):
    """The one-pass projection + convolution pullback repeats the arithmetic of the two kernels it replaces (each
    of which is checked against autograd above), through run boundaries, sequence ends and grouped heads."""
    from latent_bounded_interfaces_amd.hip.transformer import region

    torch.manual_seed(heads * 1000 + head_dim * 10 + ksize)
    b, p = 2, 3
    channels = (heads + 2 * kv_heads) * head_dim
    dq, dk, dv = (torch.randn(b, p, heads, seqlen, head_dim).to(dtype).to(device) for _ in range(3))
    weight = torch.randn(channels, 1, ksize).to(dtype).to(device)
    kwargs = dict(n_kv_heads=kv_heads, rope_base=100.0, rope_interleaved=interleaved)
    want = region.causal_conv1d_pullback(region.attn_qkv_pullback(dq, dk, dv, **kwargs), weight)
    got = region.attn_qkv_conv_pullback(dq, dk, dv, weight, **kwargs)
    assert got.dtype == dtype and got.shape == want.shape
    differing = int((got != want).sum())
    if dtype == torch.float32:
        assert differing == 0, f"{differing} elements differ"
    else:
        # same arithmetic, but the compiler may fuse a final multiply-add with the narrowing conversion in one
        # kernel and not in the other: a last-place difference on a few elements in 10^5 is allowed, nothing more
        ulp = 2.0 ** (-10 if dtype == torch.float16 else -7)
        assert differing <= max(1, got.numel() // 2000), f"{differing} of {got.numel()} elements differ"
        assert float(((got.float() - want.float()).abs() / want.float().abs().clamp_min(1e-3)).max()) <= ulp


def test_qkv_conv_pullback_contract(device):
    from latent_bounded_interfaces_amd._lib import LbiLibraryError
    from latent_bounded_interfaces_amd.hip.transformer import region

    dq = torch.randn(1, 1, 2, 4, 8, device=device)
    with pytest.raises(ValueError, match="depthwise"):
        region.attn_qkv_conv_pullback(dq, dq, dq, torch.randn(5, 1, 4, device=device), n_kv_heads=2, rope_base=10.0,
                                      rope_interleaved=False)
    with pytest.raises(LbiLibraryError, match="above 8"):
        region.attn_qkv_conv_pullback(dq, dq, dq, torch.randn(48, 1, 9, device=device), n_kv_heads=2, rope_base=10.0,
                                      rope_interleaved=False)
    with pytest.raises(RuntimeError, match="no CPU execution path"):
        region.attn_qkv_conv_pullback(dq.cpu(), dq.cpu(), dq.cpu(), torch.randn(48, 1, 4), n_kv_heads=2,
                                      rope_base=10.0, rope_interleaved=False)


REGION_CASES = [
    # dim, heads, kv, head_dim, hidden, layers, d_conv, interleaved, B, P, T
    (32, 4, 2, 8, 48, 2, 4, False, 2, 3, 12),
    (24, 3, 3, 8, 40, 1, 0, True, 1, 2, 9),
    (16, 2, 1, 6, 20, 3, 2, False, 2, 2, 5),
]


@pytest.mark.parametrize("case", REGION_CASES)
def test_region_pullback_fp32_matches_autograd(case, device):
    from latent_bounded_interfaces_amd.backends import HipTransformerLowering

    dim, heads, kv, hd, hidden, layers, d_conv, inter, b, p, t = case
    backend = oreg.make_backend(dim=dim, n_heads=heads, n_kv_heads=kv, head_dim=hd, hidden=hidden, layers=layers,
                                d_conv=d_conv, rope_interleaved=inter, rope_base=1000.0, seed=dim)
    torch.manual_seed(t)
    x = torch.randn(b, t, dim)
    basis = torch.randn(b, p, t, dim)
    _, cpu_cache = backend.forward_region(region_input=x, region_index=0)
    want = oreg.input_pullback_basis_autograd(backend, cpu_cache, basis)

    gpu_backend = backend.to(device)
    with torch.no_grad():
        _, cache = gpu_backend.forward_region(region_input=x.to(device), region_index=0)
    basis_d = basis.to(device)
    got = HipTransformerLowering().input_pullback_basis(backend=gpu_backend, cache=cache,
                                                        output_cotangent_basis=basis_d)
    assert got.shape == basis.shape and got.dtype == basis.dtype and got.is_cuda
    assert _max_rel(got.cpu(), want) <= 2e-5, _max_rel(got.cpu(), want)
    assert torch.equal(basis_d.cpu(), basis) and got.data_ptr() != basis_d.data_ptr()  # the caller's tensor is read only
    assert not got.requires_grad and got.grad_fn is None  # no autograd graph although the weights require grad


@pytest.mark.parametrize("dtype", DTYPES)
def test_kernels_take_position_constant_cotangents(dtype, device):
    """[B,P,1,*] inputs (the same cotangent at every position) give exactly what their expanded copies give."""
    from latent_bounded_interfaces_amd.hip.transformer import region

    torch.manual_seed(5)
    b, p, t, dim, hidden = 2, 3, 7, 40, 24
    g = torch.randn(b, p, t, dim).to(dtype).to(device)
    x = torch.randn(b, t, dim, device=device)
    w = (1 + 0.1 * torch.randn(dim)).to(dtype).to(device)
    res1 = torch.randn(b, p, 1, dim, device=device)
    total, branch = region.rmsnorm_pullback(g, x, w, 1e-5, res1, want_branch=True)
    want_total, want_branch = region.rmsnorm_pullback(g, x, w, 1e-5, res1.expand(b, p, t, dim).contiguous(),
                                                      want_branch=True)
    assert torch.equal(total, want_total) and torch.equal(branch, want_branch)
    assert total.data_ptr() != res1.data_ptr()
    gd1 = torch.randn(b, p, 1, hidden).to(dtype).to(device)
    fc1 = (2 * torch.randn(b, t, 2 * hidden)).to(dtype).to(device)
    got = region.gated_mlp_pullback(gd1, fc1)
    assert torch.equal(got, region.gated_mlp_pullback(gd1.expand(b, p, t, hidden).contiguous(), fc1))
    with pytest.raises(ValueError, match=r"\[B, P, 1, hidden\]"):
        region.gated_mlp_pullback(gd1.expand(b, p, 2, hidden), fc1)
    with pytest.raises(ValueError, match=r"\[B, P, 1, D\]"):
        region.rmsnorm_pullback(g, x, w, 1e-5, torch.zeros(b, p, 2, dim, device=device), want_branch=False)


@pytest.mark.parametrize("case", REGION_CASES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_region_pullback_of_an_expanded_view(case, dtype, device):
    """A stride-0 basis over positions takes the shortened path through the last block; the result is that of
    the dense copy of the same basis (up to the rounding of a product run on fewer rows)."""
    from latent_bounded_interfaces_amd.backends import HipTransformerLowering

    dim, heads, kv, hd, hidden, layers, d_conv, inter, b, p, t = case
    backend = oreg.make_backend(dim=dim, n_heads=heads, n_kv_heads=kv, head_dim=hd, hidden=hidden, layers=layers,
                                d_conv=d_conv, rope_interleaved=inter, rope_base=1000.0, seed=dim, dtype=dtype).to(device)
    torch.manual_seed(t)
    x = torch.randn(b, t, dim, device=device)
    pooled = torch.randn(b, p, 1, dim, device=device)
    with torch.no_grad():
        _, cache = backend.forward_region(region_input=x, region_index=0)
    lowering = HipTransformerLowering()
    view = pooled.expand(b, p, t, dim)
    assert view.stride(2) == 0
    got = lowering.input_pullback_basis(backend=backend, cache=cache, output_cotangent_basis=view)
    want = lowering.input_pullback_basis(backend=backend, cache=cache, output_cotangent_basis=view.contiguous())
    assert got.shape == want.shape == (b, p, t, dim)
    assert _max_rel(got.cpu(), want.cpu()) <= (1e-6 if dtype == torch.float32 else _tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("residual_in_fp32", [True, False])
def test_region_pullback_16bit_matches_fp32_path(dtype, residual_in_fp32, device):
    """16-bit weights and activations (MFMA attention path: Dh=64, T=128) against fp32 autograd
    of the same (rounded) weights."""
    from latent_bounded_interfaces_amd.backends import HipTransformerLowering

    dim, heads, kv, hd, hidden, layers, b, p, t = 128, 2, 1, 64, 256, 2, 2, 5, 128
    backend = oreg.make_backend(dim=dim, n_heads=heads, n_kv_heads=kv, head_dim=hd, hidden=hidden, layers=layers,
                                d_conv=4, residual_in_fp32=residual_in_fp32, dtype=dtype, seed=11)
    torch.manual_seed(12)
    x = torch.randn(b, t, dim).to(dtype)
    basis = torch.randn(b, p, t, dim)
    import copy

    ref_backend = copy.deepcopy(backend).float()  # same rounded weights, fp32 arithmetic
    _, ref_cache = ref_backend.forward_region(region_input=x.float(), region_index=0)
    want = oreg.input_pullback_basis_autograd(ref_backend, ref_cache, basis)

    gpu_backend = backend.to(device)
    with torch.no_grad():
        _, cache = gpu_backend.forward_region(region_input=x.to(device), region_index=0)
    got = HipTransformerLowering().input_pullback_basis(backend=gpu_backend, cache=cache,
                                                        output_cotangent_basis=basis.to(device))
    assert got.dtype == basis.dtype
    assert _max_rel(got.cpu(), want) <= 2e-2, _max_rel(got.cpu(), want)


def test_region_pullback_contract(device):
    from latent_bounded_interfaces_amd.backends import HipTransformerLowering

    backend = oreg.make_backend(dim=16, n_heads=2, head_dim=8, hidden=16, layers=1, seed=1).to(device)
    x = torch.randn(1, 4, 16, device=device)
    with torch.no_grad():
        _, cache = backend.forward_region(region_input=x, region_index=0)
    low = HipTransformerLowering()
    with pytest.raises(ValueError, match=r"\[B, P, T, D\]"):
        low.input_pullback_basis(backend=backend, cache=cache, output_cotangent_basis=torch.zeros(1, 4, 16, device=device))
    # linear in the cotangent, and direction p depends on basis[:, p] only
    basis = torch.randn(1, 3, 4, 16, device=device)
    out = low.input_pullback_basis(backend=backend, cache=cache, output_cotangent_basis=basis)
    one = low.input_pullback_basis(backend=backend, cache=cache, output_cotangent_basis=basis[:, 1:2])
    assert torch.allclose(out[:, 1:2], one, atol=1e-6)
    twice = low.input_pullback_basis(backend=backend, cache=cache, output_cotangent_basis=2 * basis)
    assert torch.allclose(twice, 2 * out, atol=1e-5)
    # a zero-layer range is the identity
    cache.layer_range, cache.layer_caches = (0, 0), []
    assert torch.equal(low.input_pullback_basis(backend=backend, cache=cache, output_cotangent_basis=basis), basis)


@pytest.mark.parametrize("case", REGION_CASES)
@pytest.mark.parametrize("bias", [False, True])
def test_parameter_vjp_fp32_matches_autograd(case, bias, device):
    from latent_bounded_interfaces_amd.backends import HipTransformerLowering

    dim, heads, kv, hd, hidden, layers, d_conv, inter, b, p, t = case
    backend = oreg.make_backend(dim=dim, n_heads=heads, n_kv_heads=kv, head_dim=hd, hidden=hidden, layers=layers + 1,
                                region_ranges=[(0, 1), (1, layers + 1)], d_conv=d_conv, rope_interleaved=inter,
                                rope_base=1000.0, bias=bias, seed=dim + 1)
    torch.manual_seed(t)
    x = torch.randn(b, t, dim)
    cot = torch.randn(b, t, dim)
    _, cpu_cache = backend.forward_region(region_input=x, region_index=1)
    want = oreg.parameter_vjp_autograd(backend, cpu_cache, cot)

    gpu_backend = backend.to(device)
    with torch.no_grad():
        _, cache = gpu_backend.forward_region(region_input=x.to(device), region_index=1)
    got = HipTransformerLowering().parameter_vjp(backend=gpu_backend, cache=cache, output_cotangent=cot.to(device))
    assert set(got) == set(want) and all(n.startswith("backbone.blocks.") for n in got)
    assert not any(n.startswith("backbone.blocks.0.") for n in got)  # region 1 owns layers 1..
    for name, w in want.items():
        g = got[name].cpu()
        assert g.shape == w.shape and g.dtype == w.dtype
        assert _max_rel(g, w) <= 2e-5, (name, _max_rel(g, w))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_parameter_vjp_16bit_matches_fp32_path(dtype, device):
    import copy

    from latent_bounded_interfaces_amd.backends import HipTransformerLowering

    dim, heads, kv, hd, hidden, layers, b, t = 128, 2, 1, 64, 256, 2, 2, 128
    backend = oreg.make_backend(dim=dim, n_heads=heads, n_kv_heads=kv, head_dim=hd, hidden=hidden, layers=layers,
                                d_conv=4, dtype=dtype, seed=13)
    torch.manual_seed(14)
    x = torch.randn(b, t, dim).to(dtype)
    cot = torch.randn(b, t, dim)
    ref_backend = copy.deepcopy(backend).float()
    _, ref_cache = ref_backend.forward_region(region_input=x.float(), region_index=0)
    want = oreg.parameter_vjp_autograd(ref_backend, ref_cache, cot)
    gpu_backend = backend.to(device)
    with torch.no_grad():
        _, cache = gpu_backend.forward_region(region_input=x.to(device), region_index=0)
    got = HipTransformerLowering().parameter_vjp(backend=gpu_backend, cache=cache, output_cotangent=cot.to(device))
    assert set(got) == set(want)
    for name, w in want.items():
        assert got[name].dtype == dtype
        assert _max_rel(got[name].cpu(), w) <= 3e-2, (name, _max_rel(got[name].cpu(), w))


def test_kernels_at_the_end_to_end_scale(device):
    """B=8, P=64, T=1024, d_model 768 / hidden 3072 (up to 3.2e9 elements per tensor, past 2^31): the last batch
    element and direction of every kernel's output equal the same kernel run on that slice alone."""
    from latent_bounded_interfaces_amd.hip.transformer import region

    torch.manual_seed(0)
    b, p, t, heads, hd, dim, hidden = 8, 64, 1024, 12, 64, 768, 3072
    dt = torch.bfloat16
    gd = torch.randn(b, p, t, hidden, device=device, dtype=dt)
    fc1 = torch.randn(b, t, 2 * hidden, device=device, dtype=dt)
    full = region.gated_mlp_pullback(gd, fc1)
    assert torch.equal(full[-1, -1], region.gated_mlp_pullback(gd[-1:, -1:].contiguous(), fc1[-1:])[0, 0])
    del gd, fc1, full
    x = torch.randn(b, t, dim, device=device)
    wn = (1 + 0.1 * torch.randn(dim, device=device)).to(dt)
    gy = torch.randn(b, p, t, dim, device=device, dtype=dt)
    res = torch.randn(b, p, t, dim, device=device)
    tot, br = region.rmsnorm_pullback(gy, x, wn, 1e-5, res.clone(), want_branch=True)
    tot1, br1 = region.rmsnorm_pullback(gy[-1:, -1:].contiguous(), x[-1:], wn, 1e-5, res[-1:, -1:].contiguous(),
                                        want_branch=True)
    assert torch.equal(tot[-1, -1], tot1[0, 0]) and torch.equal(br[-1, -1], br1[0, 0])
    hs = region.attn_heads_split(gy, heads, hd)
    assert torch.equal(hs[-1, -1], gy[-1, -1].view(t, heads, hd).transpose(0, 1))
    del tot, br, res, hs, gy
    dq, dk, dv = (torch.randn(b, p, heads, t, hd, device=device, dtype=dt) for _ in range(3))
    w = torch.randn(3 * heads * hd, 1, 4, device=device, dtype=dt)
    kw = dict(n_kv_heads=heads, rope_base=10000.0, rope_interleaved=False)
    full = region.attn_qkv_conv_pullback(dq, dk, dv, w, **kw)
    part = region.attn_qkv_conv_pullback(*(z[-1:, -1:].contiguous() for z in (dq, dk, dv)), w, **kw)
    assert torch.equal(full[-1, -1], part[0, 0])
    two = region.causal_conv1d_pullback(region.attn_qkv_pullback(dq, dk, dv, **kw), w)
    assert int((two != full).sum()) <= full.numel() // 2000


def test_region_pullback_at_the_end_to_end_layer_shape_matches_oracle(device):
    """Two layers of the end-to-end configuration (d_model 768, 12 heads x 64, hidden 3072, conv 4, T=1024, bf16
    weights and activations, fp32 residual stream) with B=1 and P=4 against fp32 autograd of the CPU restatement
    on the same rounded weights: the values behind the full-size timings, not only their indexing."""
    import copy

    from latent_bounded_interfaces_amd.backends import HipTransformerLowering

    dim, heads, hd, hidden, layers, b, p, t = 768, 12, 64, 3072, 2, 1, 4, 1024
    dtype = torch.bfloat16
    backend = oreg.make_backend(dim=dim, n_heads=heads, n_kv_heads=heads, head_dim=hd, hidden=hidden, layers=layers,
                                d_conv=4, residual_in_fp32=True, dtype=dtype, seed=21)
    torch.manual_seed(22)
    x = torch.randn(b, t, dim).to(dtype)
    basis = torch.randn(b, p, t, dim)
    ref_backend = copy.deepcopy(backend).float()
    _, ref_cache = ref_backend.forward_region(region_input=x.float(), region_index=0)
    want = oreg.input_pullback_basis_autograd(ref_backend, ref_cache, basis)
    gpu_backend = backend.to(device)
    with torch.no_grad():
        _, cache = gpu_backend.forward_region(region_input=x.to(device), region_index=0)
    low = HipTransformerLowering()
    got = low.input_pullback_basis(backend=gpu_backend, cache=cache, output_cotangent_basis=basis.to(device))
    assert _max_rel(got.cpu(), want) <= 2e-2, _max_rel(got.cpu(), want)
    # the position-constant form a mean-pooling interface produces (stride-0 view over positions)
    const = torch.randn(b, p, 1, dim)
    want_c = oreg.input_pullback_basis_autograd(ref_backend, ref_cache, const.expand(b, p, t, dim).contiguous())
    got_c = low.input_pullback_basis(backend=gpu_backend, cache=cache,
                                     output_cotangent_basis=const.to(device).expand(b, p, t, dim))
    assert _max_rel(got_c.cpu(), want_c) <= 2e-2, _max_rel(got_c.cpu(), want_c)
    # parameter gradients of the same two layers
    cot = torch.randn(b, t, dim)
    want_p = oreg.parameter_vjp_autograd(ref_backend, ref_cache, cot)
    got_p = low.parameter_vjp(backend=gpu_backend, cache=cache, output_cotangent=cot.to(device))
    assert set(got_p) == set(want_p)
    for name, w in want_p.items():
        assert _max_rel(got_p[name].cpu(), w) <= 3e-2, (name, _max_rel(got_p[name].cpu(), w))
