"""Pins the CPU restatement of the Transformer region (oracle/transformer_region.py)
against library routines, independent formulations and finite differences."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import transformer_region as oreg


def test_rmsnorm_matches_library_routine():
    torch.manual_seed(0)
    norm = oreg.OracleRMSNorm(24, eps=1e-5)
    with torch.no_grad():
        norm.weight.copy_(torch.randn(24))
    x = torch.randn(3, 5, 24)
    want = F.rms_norm(x, (24,), norm.weight, eps=1e-5)
    assert torch.allclose(norm(x), want, atol=1e-6, rtol=1e-6)
    # 16-bit input: normalised in fp32, rounded, then scaled by the rounded weight
    xb = x.to(torch.bfloat16)
    got = norm.to(torch.bfloat16)(xb)
    inv = torch.rsqrt(xb.float().pow(2).mean(-1, keepdim=True) + 1e-5)
    assert torch.equal(got, (xb.float() * inv).to(torch.bfloat16) * norm.weight)


@pytest.mark.parametrize("interleaved", [False, True])
def test_rope_is_a_position_dependent_rotation(interleaved):
    torch.manual_seed(1)
    x = torch.randn(2, 3, 7, 8, dtype=torch.float64)
    got = oreg.rope(x.float(), base=100.0, interleaved=interleaved).double()
    # complex form: (a + ib) * exp(i * t * base^(-2j/Dh))
    half = 4
    if interleaved:
        a, b = x[..., 0::2], x[..., 1::2]
    else:
        a, b = x[..., :half], x[..., half:]
    theta = torch.arange(7, dtype=torch.float64)[:, None] * 100.0 ** (-2.0 * torch.arange(half, dtype=torch.float64) / 8)
    z = torch.complex(a, b) * torch.polar(torch.ones_like(theta), theta)
    if interleaved:
        want = torch.stack((z.real, z.imag), dim=-1).flatten(-2)
    else:
        want = torch.cat((z.real, z.imag), dim=-1)
    assert torch.allclose(got, want, atol=1e-5)
    # position 0 is the identity, and a rotation keeps pair norms
    assert torch.allclose(got[:, :, 0], x[:, :, 0], atol=1e-6)
    assert torch.allclose(got.pow(2).sum(-1), x.pow(2).sum(-1), atol=1e-4)


def _dense_attention(q, k, v, scale):
    s = torch.einsum("bhid,bhjd->bhij", q, k) * scale
    mask = torch.ones(s.shape[-2:], dtype=torch.bool).tril()
    return torch.softmax(s.masked_fill(~mask, float("-inf")), dim=-1) @ v


@pytest.mark.parametrize("d_conv,n_kv,interleaved", [(0, 4, False), (3, 2, False), (4, 1, True)])
def test_block_matches_second_formulation(d_conv, n_kv, interleaved):
    """The region forward against a straight-line rewrite that shares no helper with it."""
    backend = oreg.make_backend(dim=16, n_heads=4, n_kv_heads=n_kv, head_dim=4, hidden=24, layers=2, d_conv=d_conv,
                                rope_interleaved=interleaved, rope_base=50.0, seed=3)
    torch.manual_seed(4)
    x = torch.randn(2, 6, 16)
    got, cache = backend.forward_region(region_input=x, region_index=0)

    def rms(t, w):
        return t / torch.sqrt(t.pow(2).mean(-1, keepdim=True) + 1e-5) * w

    hidden, residual = x, None
    for block in backend.backbone.blocks:
        res1 = hidden if residual is None else hidden + residual
        a = block.attn
        qkv = rms(res1, block.norm.weight) @ a.in_proj.weight.T
        if d_conv > 0:
            w = a.conv1d.weight[:, 0]  # [C, k]
            padded = F.pad(qkv, (0, 0, d_conv - 1, 0))
            qkv = sum(w[:, j] * padded[:, j:j + 6] for j in range(d_conv))
        q, k, v = qkv.split((16, 4 * n_kv, 4 * n_kv), dim=-1)
        q = q.reshape(2, 6, 4, 4).permute(0, 2, 1, 3)
        k = k.reshape(2, 6, n_kv, 4).permute(0, 2, 1, 3)
        v = v.reshape(2, 6, n_kv, 4).permute(0, 2, 1, 3)
        q, k = oreg.rope(q, 50.0, interleaved), oreg.rope(k, 50.0, interleaved)
        rep = 4 // n_kv
        k = torch.stack([k[:, h // rep] for h in range(4)], dim=1)
        v = torch.stack([v[:, h // rep] for h in range(4)], dim=1)
        o = _dense_attention(q, k, v, 0.5).permute(0, 2, 1, 3).reshape(2, 6, 16)
        res2 = o @ a.out_proj.weight.T + res1
        f = rms(res2, block.norm2.weight) @ block.mlp.fc1.weight.T
        up, gate = f[..., :24], f[..., 24:]
        hidden = (up * gate * torch.sigmoid(gate)) @ block.mlp.fc2.weight.T
        residual = res2
    assert torch.allclose(got, hidden + residual, atol=2e-5, rtol=2e-5)
    assert len(cache.layer_caches) == 2 and cache.layer_range == (0, 2)
    lc = cache.layer_caches[1]
    assert lc.residual_input is not None and cache.layer_caches[0].residual_input is None
    assert torch.equal(lc.attention.norm_input, cache.layer_caches[0].hidden_output + cache.layer_caches[0].residual_output)


def test_autograd_pullback_matches_finite_differences():
    backend = oreg.make_backend(dim=8, n_heads=2, n_kv_heads=1, head_dim=4, hidden=12, layers=2, d_conv=2,
                                dtype=torch.float64, seed=5)
    torch.manual_seed(6)
    x = torch.randn(1, 3, 8, dtype=torch.float64)
    basis = torch.randn(1, 2, 3, 8, dtype=torch.float64)
    _, cache = backend.forward_region(region_input=x, region_index=0)
    got = oreg.input_pullback_basis_autograd(backend, cache, basis)
    # the norm and the rotary embedding compute in fp32 whatever the input type (as the reference's do),
    # so the step is sized for fp32 noise, not fp64
    eps = 1e-3
    want = torch.zeros_like(got)
    with torch.no_grad():
        for t in range(3):
            for d in range(8):
                e = torch.zeros_like(x)
                e[0, t, d] = eps
                yp, _ = backend.forward_region(region_input=x + e, region_index=0)
                ym, _ = backend.forward_region(region_input=x - e, region_index=0)
                jcol = (yp - ym) / (2 * eps)  # d out / d x[t, d]
                want[0, :, t, d] = (basis[0] * jcol[0]).sum(dim=(-1, -2))
    assert torch.allclose(got, want, atol=5e-3, rtol=5e-3)
    assert float((got - want).abs().max()) < 5e-3 < 0.01 * float(got.abs().max())


def test_mixed_precision_residual_stream_is_fp32():
    backend = oreg.make_backend(dim=16, n_heads=2, head_dim=8, hidden=16, layers=2, dtype=torch.bfloat16, seed=7)
    x = torch.randn(1, 4, 16).to(torch.bfloat16)
    out, cache = backend.forward_region(region_input=x, region_index=0)
    assert out.dtype == torch.float32
    assert cache.layer_caches[0].residual_output.dtype == torch.float32
    assert cache.layer_caches[0].attention.q_rope.dtype == torch.bfloat16
    assert cache.layer_caches[1].mlp.norm_input.dtype == torch.float32


def _tiny_model(dtype=torch.float32, **kw):
    from oracle import lbi_model as olbi

    args = dict(vocab_size=37, dim=16, n_heads=2, layers=6, layers_per_region=2, interface_width=6, hidden=24,
                d_conv=3, dtype=dtype, seed=21)
    args.update(kw)
    return olbi.OracleLBIModel(**args)


def test_lbi_model_state_jacobians_match_finite_differences():
    from oracle import lbi_model as olbi

    model = _tiny_model()
    ids = torch.randint(0, 37, (2, 5), generator=torch.Generator().manual_seed(1))
    _, cache = model.forward_with_cache(ids)
    jts = olbi.GraphInterfacePullbackProvider().materialize_state_jacobian_t(model=model, cache=cache)
    assert len(jts) == 3 and jts[0].shape == (2, 6, 6)
    r = 1
    rc = cache["region_caches"][r]

    def state_map(s):
        x = rc.canvas_features + model.interface.decode(s, r).unsqueeze(1)
        y, _ = model.region_backend.forward_region(region_input=x, region_index=r)
        return model.interface.update(s, y, r).state

    eps = 1e-2
    with torch.no_grad():
        for i in range(6):
            e = torch.zeros(2, 6)
            e[:, i] = eps
            col = (state_map(rc.state_in + e) - state_map(rc.state_in - e)) / (2 * eps)  # d s_out[:] / d s_in[i]
            assert torch.allclose(jts[r][:, i, :], col, atol=2e-3, rtol=2e-2)


@pytest.mark.parametrize("layers,per_region", [(6, 2), (2, 2), (4, 1)])
def test_lbi_model_scan_step_reproduces_dense_gradients(layers, per_region):
    from oracle import lbi_model as olbi

    model = _tiny_model(layers=layers, layers_per_region=per_region, interface_hidden=10)
    gen = torch.Generator().manual_seed(2)
    ids = torch.randint(0, 37, (2, 5), generator=gen)
    targets = torch.randint(0, 37, (2, 5), generator=gen)
    loss_dense, dense = olbi.dense_gradients(model, ids, targets)
    logits, cache = model.forward_with_cache(ids)
    loss = olbi.token_loss(logits, targets)
    assert abs(float(loss) - loss_dense) < 1e-7
    got = olbi.scan_backward_step_sequential(model, loss=loss, cache=cache,
                                             pullback_provider=olbi.GraphInterfacePullbackProvider(),
                                             local_vjp_provider=olbi.AutogradLocalVJPProvider())
    assert set(got) == set(dense)
    for name, want in dense.items():
        if want is None:  # the last region's state update never reaches the loss
            assert got[name] is None, name
            continue
        assert got[name] is not None, name
        assert torch.allclose(got[name], want, atol=1e-5, rtol=1e-4), name  # the reference's fp32 parity bar
