"""The autograd providers and gradient-map helpers of the backward package (CPU: they are plain torch.autograd;
the scan itself is replaced by the oracle's sequential chain, so no kernel is needed)."""
from __future__ import annotations

import pytest
import torch

from latent_bounded_interfaces_amd import backward
from oracle import lbi_model as olbi


def _model(**kw):
    args = dict(vocab_size=37, dim=16, n_heads=2, n_kv_heads=1, layers=3, layers_per_region=1, interface_width=5,
                hidden=24, d_conv=3, interface_hidden=7, dtype=torch.float64, seed=11)
    args.update(kw)
    return olbi.OracleLBIModel(**args).double()


def _batch(seed=5, shape=(2, 7)):
    gen = torch.Generator().manual_seed(seed)
    return torch.randint(0, 37, shape, generator=gen), torch.randint(0, 37, shape, generator=gen)


@pytest.mark.parametrize("mode,chunk", [("graph", 1), ("recompute", 1), ("recompute", 2), ("recompute", 5), ("recompute", 9)])
def test_autograd_pullback_providers_match_the_oracle_graph_provider(mode, chunk):
    model = _model()
    ids, _ = _batch()
    _, cache = model.forward_with_cache(ids)
    want = olbi.GraphInterfacePullbackProvider().materialize_state_jacobian_t(model=model, cache=cache)
    got = backward.build_interface_pullback_provider(mode, basis_chunk=chunk).materialize_state_jacobian_t(
        model=model, cache=cache)
    assert len(got) == len(want) == 3
    for a, b in zip(got, want):
        assert a.shape == (2, 5, 5)
        assert torch.allclose(a, b, atol=1e-12, rtol=1e-10)


@pytest.mark.parametrize("mode", ["graph", "recompute"])
def test_autograd_pullback_providers_can_leave_out_the_last_region(mode):
    """``skip_last=True`` (what the scan backward step of this package asks for when nothing reads the last
    region's Jacobian): the same matrices, ``None`` in the last place."""
    model = _model()
    ids, _ = _batch()
    _, cache = model.forward_with_cache(ids)
    provider = backward.build_interface_pullback_provider(mode)
    assert provider.can_skip_last_region
    full = provider.materialize_state_jacobian_t(model=model, cache=cache)
    short = provider.materialize_state_jacobian_t(model=model, cache=cache, skip_last=True)
    assert len(short) == len(full) == 3 and short[-1] is None
    assert all(torch.equal(a, b) for a, b in zip(short[:-1], full[:-1]))


def test_pullback_provider_errors():
    model = _model()
    ids, _ = _batch()
    _, cache = model.forward_with_cache(ids)
    with pytest.raises(ValueError, match="states length"):
        backward.TorchGraphInterfacePullbackProvider().materialize_state_jacobian_t(
            model=model, cache=dict(cache, states=cache["states"][:-1]))
    with pytest.raises(ValueError, match="basis_chunk must be > 0"):
        backward.TorchRecomputeInterfacePullbackProvider(basis_chunk=0).materialize_state_jacobian_t(model=model, cache=cache)
    with pytest.raises(ValueError, match="region_caches length"):
        backward.TorchRecomputeInterfacePullbackProvider().materialize_state_jacobian_t(
            model=model, cache=dict(cache, region_caches=[]))


@pytest.mark.parametrize("layers,per_region", [(3, 1), (4, 2), (2, 2)])
def test_default_local_vjp_provider_reproduces_dense_gradients(layers, per_region):
    """The reference's parity criterion (tests/test_lbi_gradient_parity.py): scan-step gradients == loss.backward()."""
    model = _model(layers=layers, layers_per_region=per_region)
    ids, targets = _batch()
    _, dense = olbi.dense_gradients(model, ids, targets)
    logits, cache = model.forward_with_cache(ids)
    grads = olbi.scan_backward_step_sequential(
        model, loss=olbi.token_loss(logits, targets), cache=cache,
        pullback_provider=backward.TorchGraphInterfacePullbackProvider(),
        local_vjp_provider=backward.TorchAutogradLocalVJPProvider())
    assert set(grads) == set(dense)
    for name, want in dense.items():
        if want is None:
            assert grads[name] is None
        else:
            assert torch.allclose(grads[name], want.to(grads[name].dtype), atol=1e-6, rtol=1e-4), (name, float((grads[name] - want).abs().max()))


@pytest.mark.parametrize("layers,per_region", [(3, 1), (4, 2), (2, 2)])
def test_structured_local_vjp_provider_reproduces_dense_gradients(layers, per_region):
    """The cache-based local-VJP provider, with the region sweeps answered by autograd of the oracle region (the
    two-call form of the lowering protocol) so that it runs without a GPU: the gradient map of the scan step equals
    ``loss.backward()`` of the same graph (fp64 apart from the norm, which the oracle block runs in fp32), name by name, ``None`` where the dense path leaves ``None``."""
    model = _model(layers=layers, layers_per_region=per_region)
    ids, targets = _batch()
    _, dense = olbi.dense_gradients(model, ids, targets)
    logits, cache = model.forward_with_cache(ids)
    provider = backward.StructuredLocalVJPProvider(cache=cache)
    assert isinstance(provider, backward.LocalVJPProvider) and provider.name == "structured"
    grads = olbi.scan_backward_step_sequential(
        model, loss=olbi.token_loss(logits, targets), cache=cache,
        pullback_provider=backward.TorchGraphInterfacePullbackProvider(), local_vjp_provider=provider)
    assert set(grads) == set(dense)
    for name, want in dense.items():
        if want is None:
            assert grads[name] is None, name
        else:
            assert grads[name] is not None, name
            assert torch.allclose(grads[name], want, atol=1e-7, rtol=1e-5), (name, float((grads[name] - want).abs().max()))


def test_structured_local_vjp_provider_contract():
    model = _model()
    ids, targets = _batch()
    logits, cache = model.forward_with_cache(ids)
    loss = olbi.token_loss(logits, targets)
    unbound = backward.StructuredLocalVJPProvider()
    with pytest.raises(RuntimeError, match="forward cache"):
        unbound.store_output_head_grads(model=model, loss=loss, grad_map={})
    unbound.bind_cache(cache)
    # a state other than the one the last region read is answered by the graph
    unbound.store_output_head_grads(model=model, loss=loss, grad_map=unbound.new_grad_map(model))
    want = torch.autograd.grad(loss, cache["states"][0], retain_graph=True)[0]
    assert torch.equal(unbound.state_adjoint_from_loss(loss=loss, state=cache["states"][0]), want)
    want = torch.autograd.grad(loss, cache["states"][-2], retain_graph=True)[0]
    got = unbound.state_adjoint_from_loss(loss=loss, state=cache["states"][-2])
    assert torch.allclose(got, want, atol=1e-12, rtol=1e-9)
    assert backward.build_local_vjp_provider("structured").name == "structured"
    assert backward.build_local_vjp_provider("torch-autograd").name == "torch_autograd"
    with pytest.raises(ValueError, match="must be one of"):
        backward.build_local_vjp_provider("dense")


def test_package_exports_every_name_of_the_reference_package():
    """reference backward/__init__.py:22-50."""
    reference_names = [
        "ADEngine", "ADResult", "AutogradEngine", "GradMap", "InterfacePullbackProvider", "LBIBackwardResult",
        "LocalVJPProvider", "ReferenceScanEngine", "ScanADEngine", "ScanBackpropModel", "TorchAutogradLocalVJPProvider",
        "TorchGraphInterfacePullbackProvider", "TorchRecomputeInterfacePullbackProvider", "assign_grad_map",
        "autograd_backward_step", "apply_jacobian_t", "build_interface_pullback_provider", "collect_named_grads",
        "compose_suffix_jacobian_t", "lbi_reference_scan_backward_step", "lbi_scan_backward_step",
        "materialize_interface_state_jacobian_t_graph", "materialize_interface_state_jacobian_t_recompute",
        "propagate_state_adjoint_by_autograd_chain", "propagate_state_adjoint_from_last_region_input",
        "propagate_state_adjoint_with_jacobian_scan", "store_named_grads"]
    assert [n for n in reference_names if n not in backward.__all__ or not hasattr(backward, n)] == []
    model = _model()
    ids, targets = _batch()
    _, dense = olbi.dense_gradients(model, ids, targets)
    logits, cache = model.forward_with_cache(ids)
    grads = backward.autograd_backward_step(model, ce_loss=olbi.token_loss(logits, targets))
    assert all((grads[n] is None) == (dense[n] is None) and (dense[n] is None or torch.equal(grads[n], dense[n]))
               for n in dense)
    assert backward.AutogradEngine.name == "autograd"
    _, cache = model.forward_with_cache(ids)          # the dense step released the graph of the first forward
    want = backward.TorchGraphInterfacePullbackProvider().materialize_state_jacobian_t(model=model, cache=cache)
    got = backward.materialize_interface_state_jacobian_t_graph(model=model, cache=cache)
    assert all(torch.equal(a, b) for a, b in zip(got, want))
    got = backward.materialize_interface_state_jacobian_t_recompute(model=model, cache=cache, basis_chunk=2)
    assert all(torch.allclose(a, b, atol=1e-12) for a, b in zip(got, want))


def test_autograd_chain_diagnostic_matches_the_jacobian_chain():
    model = _model()
    ids, targets = _batch()
    logits, cache = model.forward_with_cache(ids)
    states = cache["states"]
    top = torch.randn(2, 5, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    got = backward.propagate_state_adjoint_by_autograd_chain(states=states, top_state_adjoint=top)
    jts = olbi.GraphInterfacePullbackProvider().materialize_state_jacobian_t(model=model, cache=cache)
    want = top
    assert torch.equal(got[-1], top)
    for r in reversed(range(3)):
        want = torch.einsum("bij,bj->bi", jts[r], want)
        assert torch.allclose(got[r], want, atol=1e-12)
    with pytest.raises(ValueError, match="at least two"):
        backward.propagate_state_adjoint_by_autograd_chain(states=states[:1], top_state_adjoint=top)


def test_grad_map_helpers_round_trip():
    lin = torch.nn.Linear(3, 2)
    lin.bias.requires_grad_(False)
    assert backward.collect_named_grads(lin) == {"weight": None}
    lin(torch.ones(1, 3)).sum().backward()
    grads = backward.collect_named_grads(lin)
    assert set(grads) == {"weight"} and torch.equal(grads["weight"], torch.ones(2, 3))
    grads["weight"] = grads["weight"] * 2
    backward.assign_grad_map(lin, grads)
    assert torch.equal(lin.weight.grad, 2 * torch.ones(2, 3)) and lin.weight.grad is not grads["weight"]
    backward.assign_grad_map(lin, {})
    assert lin.weight.grad is None
    target: dict = {}
    backward.store_named_grads(target, {id(lin.weight): "w"}, [lin.weight], (None,))
    assert target == {"w": None}
    result = backward.ADResult(grad_map={})
    assert result.diagnostics == {}
    assert backward.LBIBackwardResult(grad_map={}, interface_scan_rms=0.5).interface_jacobian_stats is None


def test_slices_of_one_buffer_are_recognised_without_a_copy():
    """Lists whose members are, in order, the slices of one dense [B, K, d, d] buffer reach the kernels as that
    buffer; anything else (separate tensors, wrong order, a gap, other strides) takes the stacking copy."""
    from latent_bounded_interfaces_amd.backward.suffix_scan import _dense_stack_view

    buf = torch.randn(3, 4, 5, 5)
    views = [buf[:, r] for r in range(4)]
    dense = _dense_stack_view(views)
    assert dense is not None and dense.data_ptr() == buf.data_ptr() and dense.is_contiguous()
    assert torch.equal(dense, buf)
    assert _dense_stack_view([v.clone() for v in views]) is None
    assert _dense_stack_view(views[::-1]) is None
    assert _dense_stack_view(views[:3]) is None                      # a prefix has the wrong batch stride
    assert _dense_stack_view([views[0], views[2]]) is None
    assert _dense_stack_view([buf[:, r].transpose(1, 2) for r in range(4)]) is None
    inner = buf[:, 1:3]                                              # a window of a larger buffer is not dense
    assert _dense_stack_view([inner[:, 0], inner[:, 1]]) is None
    one = torch.randn(1, 2, 3, 3)                                    # B = 1: the batch stride is immaterial
    assert torch.equal(_dense_stack_view([one[:, 0], one[:, 1]]), one)
    offset = torch.randn(2 * 3 * 4 * 4 + 7)[7:].view(2, 3, 4, 4)     # a buffer that starts inside its storage
    assert torch.equal(_dense_stack_view([offset[:, r] for r in range(3)]), offset)
