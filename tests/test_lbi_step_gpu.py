"""End-to-end LBI scan backward step on the GPU: state Jacobians from the structured
provider (region pullback on the HIP kernels), state adjoints from the HIP scan, parameter
gradients against the dense ``loss.backward()`` of the same model."""
import pytest
import torch

from oracle import lbi_model as olbi

pytestmark = pytest.mark.gpu


def _model(device, dtype=torch.float32, **kw):
    from latent_bounded_interfaces_amd.backends import HipTransformerLowering

    args = dict(vocab_size=61, dim=32, n_heads=4, n_kv_heads=2, layers=6, layers_per_region=2, interface_width=8,
                hidden=48, d_conv=4, interface_hidden=12, dtype=dtype, seed=31, lowering=HipTransformerLowering())
    args.update(kw)
    return olbi.OracleLBIModel(**args).to(device)


@pytest.mark.parametrize("basis_chunk", [0, 3])
def test_structured_jacobians_match_graph_provider(basis_chunk, device):
    from latent_bounded_interfaces_amd.backward import StructuredInterfacePullbackProvider

    model = _model(device)
    ids = torch.randint(0, 61, (2, 10), generator=torch.Generator().manual_seed(3)).to(device)
    _, cache = model.forward_with_cache(ids)
    want = olbi.GraphInterfacePullbackProvider().materialize_state_jacobian_t(model=model, cache=cache)
    got = StructuredInterfacePullbackProvider(basis_chunk=basis_chunk).materialize_state_jacobian_t(model=model, cache=cache)
    assert len(got) == len(want) == 3
    for a, b in zip(got, want):
        assert a.shape == b.shape == (2, 8, 8) and a.is_contiguous()
        assert float((a - b).abs().max()) <= 2e-5 * float(b.abs().max()), float((a - b).abs().max())


def test_position_constant_update_is_detected_and_optional(device):
    """The mean-pooling interface sends one cotangent to every position: the provider detects it on the
    device, hands the region a stride-0 view, and gives the same Jacobians as with the detection off."""
    from latent_bounded_interfaces_amd.backward import StructuredInterfacePullbackProvider

    model = _model(device)
    ids = torch.randint(0, 61, (2, 10), generator=torch.Generator().manual_seed(3)).to(device)
    _, cache = model.forward_with_cache(ids)
    seen = []
    inner = model.region_backend.input_pullback_basis

    def spy(*, cache, output_cotangent_basis):
        seen.append(output_cotangent_basis.stride(2))
        return inner(cache=cache, output_cotangent_basis=output_cotangent_basis)

    model.region_backend.input_pullback_basis = spy
    try:
        results = {}
        for mode in ("off", "verify", "verify_once"):
            seen.clear()
            provider = StructuredInterfacePullbackProvider(position_constant_update=mode)
            results[mode] = provider.materialize_state_jacobian_t(model=model, cache=cache)
            assert all(s != 0 for s in seen) if mode == "off" else all(s == 0 for s in seen), (mode, seen)
            if mode == "verify_once":
                assert provider._constant_over_positions == {type(model.interface): True}
    finally:
        del model.region_backend.input_pullback_basis
    for mode in ("verify", "verify_once"):
        for a, b in zip(results[mode], results["off"]):
            assert float((a - b).abs().max()) <= 2e-6 * float(b.abs().max())
    with pytest.raises(ValueError, match="position_constant_update"):
        StructuredInterfacePullbackProvider(position_constant_update="maybe")


@pytest.mark.parametrize("layers,per_region", [(6, 2), (4, 1), (2, 2)])
def test_scan_backward_step_reproduces_dense_gradients(layers, per_region, device):
    from latent_bounded_interfaces_amd.backward import StructuredInterfacePullbackProvider, lbi_scan_backward_step

    model = _model(device, layers=layers, layers_per_region=per_region)
    gen = torch.Generator().manual_seed(4)
    ids = torch.randint(0, 61, (2, 10), generator=gen).to(device)
    targets = torch.randint(0, 61, (2, 10), generator=gen).to(device)
    loss_dense, dense = olbi.dense_gradients(model, ids, targets)
    logits, cache = model.forward_with_cache(ids)
    loss = olbi.token_loss(logits, targets)
    result = lbi_scan_backward_step(model, ce_loss=loss, cache=cache,
                                    pullback_provider=StructuredInterfacePullbackProvider(),
                                    local_vjp_provider=olbi.AutogradLocalVJPProvider(),
                                    compute_interface_jacobian_stats=True, include_interface_jacobian_suffix=True,
                                    check_scan=True)
    assert abs(float(loss.detach()) - loss_dense) < 1e-6
    assert result.interface_scan_rms < 1e-5  # the reference's own bar for the scan cross-check
    if model.num_regions > 1:
        assert "jac_suffix_spec_max" in result.interface_jacobian_stats
    else:
        assert result.interface_jacobian_stats is None
    assert set(result.grad_map) == set(dense)
    for name, want in dense.items():
        got = result.grad_map[name]
        if want is None:
            assert got is None, name
            continue
        assert got is not None, name
        # gradient parity bar of the reference's fp32 cases (tests/test_lbi_gradient_parity.py:40)
        assert torch.allclose(got, want, atol=1e-5, rtol=1e-4), (name, float((got - want).abs().max()))


def test_step_contract(device):
    from latent_bounded_interfaces_amd.backward import (StructuredInterfacePullbackProvider,
                                                        build_interface_pullback_provider, lbi_scan_backward_step)

    assert build_interface_pullback_provider("structured", basis_chunk=2).basis_chunk == 2
    with pytest.raises(ValueError):
        build_interface_pullback_provider("graph")
    model = _model(device)
    ids = torch.randint(0, 61, (1, 4)).to(device)
    logits, cache = model.forward_with_cache(ids)
    cache_bad = dict(cache, region_caches=cache["region_caches"][:-1])
    with pytest.raises(ValueError, match="region_caches length"):
        StructuredInterfacePullbackProvider().materialize_state_jacobian_t(model=model, cache=cache_bad)
    with pytest.raises(RuntimeError, match="at least one region"):
        lbi_scan_backward_step(model, ce_loss=logits.sum(), cache=dict(cache, region_ranges=[]),
                               pullback_provider=StructuredInterfacePullbackProvider(),
                               local_vjp_provider=olbi.AutogradLocalVJPProvider())
