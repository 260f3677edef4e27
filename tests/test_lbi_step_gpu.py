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
        assert a.shape == b.shape == (2, 8, 8)
        assert float((a - b).abs().max()) <= 2e-5 * float(b.abs().max()), float((a - b).abs().max())
    # the matrices the scan composes (all but the last) are slices of one dense buffer and reach the kernels as
    # that buffer, without a stacking copy
    from latent_bounded_interfaces_amd.backward.suffix_scan import _stack_for_chain

    stacked = _stack_for_chain(got[:-1])
    assert stacked.shape == (2, 2, 8, 8) and stacked.is_contiguous() and stacked.data_ptr() == got[0].data_ptr()
    assert got[-1].is_contiguous()


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
                assert dict(provider._constant_over_positions) == {model.interface: {10: True}}
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
    assert build_interface_pullback_provider("structured").basis_chunk == 0
    assert build_interface_pullback_provider("graph").name == "torch_graph"
    assert build_interface_pullback_provider("Torch-Recompute", basis_chunk=3).basis_chunk == 3
    with pytest.raises(ValueError, match="must be one of"):
        build_interface_pullback_provider("dense")
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


def _check_grads(grad_map, dense, atol=1e-5, rtol=1e-4):
    assert set(grad_map) == set(dense)
    for name, want in dense.items():
        got = grad_map[name]
        if want is None:
            assert got is None, name
            continue
        assert got is not None, name
        assert torch.allclose(got, want, atol=atol, rtol=rtol), (name, float((got - want).abs().max()))


def _step_inputs(model, device, seed=4, shape=(2, 10)):
    gen = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, 61, shape, generator=gen).to(device)
    targets = torch.randint(0, 61, shape, generator=gen).to(device)
    loss_dense, dense = olbi.dense_gradients(model, ids, targets)
    logits, cache = model.forward_with_cache(ids)
    return olbi.token_loss(logits, targets), cache, dense


def test_step_with_the_reference_argument_list(device):
    """``lbi_scan_backward_step`` called exactly as the reference's callers do (backward/reference_scan.py:27-34:
    no local-VJP provider, no extra keyword): default provider, ``interface_scan_rms`` reported."""
    from latent_bounded_interfaces_amd.backward import StructuredInterfacePullbackProvider, lbi_scan_backward_step

    model = _model(device)
    loss, cache, dense = _step_inputs(model, device)
    result = lbi_scan_backward_step(model, ce_loss=loss, cache=cache,
                                    pullback_provider=StructuredInterfacePullbackProvider())
    assert 0.0 < result.interface_scan_rms < 1e-5     # two independent device results: tiny, but not identical
    assert result.interface_jacobian_stats is None
    _check_grads(result.grad_map, dense)


@pytest.mark.parametrize("mode,chunk", [("graph", 1), ("recompute", 3), ("structured", 4)])
def test_reference_scan_backward_step_by_mode(mode, chunk, device):
    """reference backward/reference_scan.py:12-34 with its keyword list; every mode reproduces dense gradients."""
    from latent_bounded_interfaces_amd.backward import lbi_reference_scan_backward_step

    model = _model(device)
    loss, cache, dense = _step_inputs(model, device)
    result = lbi_reference_scan_backward_step(model, ce_loss=loss, cache=cache, state_jacobian_mode=mode,
                                              state_jacobian_basis_chunk=chunk,
                                              compute_interface_jacobian_stats=True,
                                              include_interface_jacobian_suffix=False)
    assert result.interface_scan_rms < 1e-5
    assert "jac_local_spec_max" in result.interface_jacobian_stats
    assert "jac_suffix_spec_max" not in result.interface_jacobian_stats
    _check_grads(result.grad_map, dense)


def test_autograd_providers_agree_with_the_structured_one(device):
    from latent_bounded_interfaces_amd.backward import build_interface_pullback_provider

    model = _model(device)
    _, cache, _ = _step_inputs(model, device)
    want = build_interface_pullback_provider("structured").materialize_state_jacobian_t(model=model, cache=cache)
    for mode, chunk in (("graph", 1), ("recompute", 1), ("recompute", 5), ("recompute", 8)):
        got = build_interface_pullback_provider(mode, basis_chunk=chunk).materialize_state_jacobian_t(model=model, cache=cache)
        for a, b in zip(got, want):
            assert a.shape == b.shape and a.is_contiguous()
            assert float((a - b).abs().max()) <= 2e-5 * float(b.abs().max()), (mode, chunk)


def test_scan_engine_as_the_training_loop_uses_it(device):
    """reference train/runners.py:368-372: ``ScanADEngine.from_config(cfg).backward(model=, loss=, cache=)``."""
    from types import SimpleNamespace

    from latent_bounded_interfaces_amd.backward import (ADResult, ReferenceScanEngine, ScanADEngine,
                                                        ScanBackpropModel, collect_named_grads)

    assert ReferenceScanEngine is ScanADEngine and ScanADEngine.name == "scan"
    model = _model(device)
    assert isinstance(model, ScanBackpropModel)
    loss, cache, dense = _step_inputs(model, device)
    for cfg_mode, provider_name in (("recompute", "torch_recompute"), ("structured", "structured")):
        cfg = SimpleNamespace(interface_jacobian_mode=cfg_mode, jacobian_basis_chunk=4,
                              log_interface_jacobian_suffix=True)
        engine = ScanADEngine.from_config(cfg, compute_interface_jacobian_stats=True)
        loss, cache, dense = _step_inputs(model, device)
        result = engine.backward(model=model, loss=loss, cache=cache)
        assert isinstance(result, ADResult)
        assert set(result.diagnostics) == {"interface_scan_rms", "interface_pullback_provider", "local_vjp_provider",
                                           "interface_jacobian_stats"}
        assert result.diagnostics["interface_pullback_provider"] == provider_name
        assert result.diagnostics["local_vjp_provider"] == "torch_autograd"
        assert result.diagnostics["interface_scan_rms"] < 1e-5
        assert "jac_suffix_spec_mean" in result.diagnostics["interface_jacobian_stats"]
        _check_grads(result.grad_map, dense)
        _check_grads(collect_named_grads(model), dense)          # backward() also wrote param.grad
    plain = ScanADEngine(state_jacobian_mode="structured", state_jacobian_basis_chunk=0)
    loss, cache, dense = _step_inputs(model, device)
    assert "interface_jacobian_stats" not in plain.backward(model=model, loss=loss, cache=cache).diagnostics
    with pytest.raises(ValueError, match="forward cache"):
        plain.backward(model=model, loss=loss)
    with pytest.raises(TypeError, match="ScanBackpropModel"):
        plain.backward(model=torch.nn.Linear(2, 2), loss=loss, cache=cache)


def test_apply_jacobian_t_accepts_double_precision(device):
    """reference backward/suffix_scan.py:24-38 promotes; here fp64 operands are converted (fp32 accuracy)."""
    from latent_bounded_interfaces_amd.backward import apply_jacobian_t

    gen = torch.Generator().manual_seed(2)
    jt = torch.randn(3, 8, 8, generator=gen, dtype=torch.float64)
    g = torch.randn(3, 8, generator=gen, dtype=torch.float64)
    want = torch.einsum("bij,bj->bi", jt, g)
    got = apply_jacobian_t(jt.to(device), g.to(device))
    assert got.dtype == torch.float64
    assert torch.allclose(got.cpu(), want, atol=1e-5, rtol=1e-5)
    got32 = apply_jacobian_t(jt.to(device), g.to(device), out_dtype=torch.float32)
    assert got32.dtype == torch.float32


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_16bit_step_at_real_head_geometry_reproduces_dense_gradients(dtype, device):
    """The end-to-end configuration's precision and kernel path at reduced width: 16-bit weights and activations,
    fp32 interface of width 64, heads of 64, conv 4, 2 regions x 2 layers and T=320, so the 64 directions of
    every region pullback run the four-kernel matrix-core attention path.  Against dense ``loss.backward()`` in
    fp32 on the same rounded weights, at the reference's 16-bit bar (atol = rtol = 5e-2,
    tests/test_lbi_gradient_parity.py:729-730), plus a relative-L2 bound per parameter that does not vanish for
    small gradients."""
    import copy

    from latent_bounded_interfaces_amd.backward import ScanADEngine

    model = _model(device, dtype=dtype, dim=128, n_heads=2, n_kv_heads=2, hidden=256, layers=4, layers_per_region=2,
                   interface_width=64, interface_hidden=96, seed=37)
    dense_model = copy.deepcopy(model).float()
    dense_model.region_backend.lowering = None
    gen = torch.Generator().manual_seed(9)
    ids = torch.randint(0, 61, (2, 320), generator=gen).to(device)
    targets = torch.randint(0, 61, (2, 320), generator=gen).to(device)
    loss_dense, dense = olbi.dense_gradients(dense_model, ids, targets)
    logits, cache = model.forward_with_cache(ids)
    loss = olbi.token_loss(logits, targets)
    assert abs(float(loss.detach()) - loss_dense) <= 5e-3 + 5e-3 * abs(loss_dense)
    engine = ScanADEngine(state_jacobian_mode="structured", state_jacobian_basis_chunk=0,
                          compute_interface_jacobian_stats=True)
    result = engine.backward(model=model, loss=loss, cache=cache)
    assert result.diagnostics["interface_scan_rms"] < 5e-5
    assert set(result.grad_map) == set(dense)
    worst = 0.0
    for name, want in dense.items():
        got = result.grad_map[name]
        assert (got is None) == (want is None), name
        if want is None:
            continue
        assert torch.allclose(got.float(), want, atol=5e-2, rtol=5e-2), (name, float((got.float() - want).abs().max()))
        rel = float((got.float() - want).norm() / want.norm().clamp_min(1e-12))
        worst = max(worst, rel)
        # (a handful of scalars has no meaningful relative error: a sum that happens to be small is all noise)
        assert rel <= 5e-2 or want.numel() < 64, (name, rel)
    # the state Jacobians themselves against the forward graph of the fp32 model
    _, dense_cache = dense_model.forward_with_cache(ids)
    want_jt = olbi.GraphInterfacePullbackProvider().materialize_state_jacobian_t(model=dense_model, cache=dense_cache)
    got_jt = engine.pullback_provider.materialize_state_jacobian_t(model=model, cache=cache)
    for a, b in zip(got_jt, want_jt):
        assert float((a.float() - b).abs().max()) <= 2e-2 * float(b.abs().max())


def test_step_on_an_autocast_forward_with_fp32_master_weights(device):
    """The reference's training loop keeps fp32 weights and runs the forward under ``autocast(bfloat16)``
    (train/runners.py:299, :361): the cache then holds 16-bit attention / MLP activations beside an fp32 residual
    stream and fp32 weights.  The structured provider follows the forward's compute dtype (weights cast per use);
    state Jacobians against the autograd graph of that same forward, step gradients against its dense backward."""
    from latent_bounded_interfaces_amd.backward import ScanADEngine

    model = _model(device, dim=128, n_heads=2, n_kv_heads=1, hidden=256, layers=4, layers_per_region=2,
                   interface_width=16, interface_hidden=24, seed=41)
    gen = torch.Generator().manual_seed(10)
    ids = torch.randint(0, 61, (2, 192), generator=gen).to(device)
    targets = torch.randint(0, 61, (2, 192), generator=gen).to(device)

    def forward():
        with torch.autocast("cuda", dtype=torch.bfloat16):
            logits, cache = model.forward_with_cache(ids)
        return olbi.token_loss(logits, targets), cache

    model.zero_grad(set_to_none=True)
    loss, cache = forward()
    loss.backward()
    dense = {n: (None if p.grad is None else p.grad.detach().clone()) for n, p in model.named_parameters()}
    model.zero_grad(set_to_none=True)

    loss, cache = forward()
    layer0 = cache["region_caches"][0].backend_cache.layer_caches[0]
    assert layer0.attention.q_rope.dtype == torch.bfloat16 and layer0.mlp.norm_input.dtype == torch.float32
    assert next(model.region_backend.parameters()).dtype == torch.float32
    engine = ScanADEngine(state_jacobian_mode="structured", state_jacobian_basis_chunk=0)
    want_jt = olbi.GraphInterfacePullbackProvider().materialize_state_jacobian_t(model=model, cache=cache)
    got_jt = engine.pullback_provider.materialize_state_jacobian_t(model=model, cache=cache)
    for a, b in zip(got_jt, want_jt):
        # the graph provider returns region 0 in the 16-bit dtype of the first state; here all regions share fp32
        assert a.dtype == torch.float32
        assert float((a - b.float()).abs().max()) <= 2e-2 * float(b.abs().max()), float((a - b.float()).abs().max())
    result = engine.backward(model=model, loss=loss, cache=cache)
    assert result.diagnostics["interface_scan_rms"] < 5e-5
    for name, want in dense.items():
        got = result.grad_map[name]
        assert (got is None) == (want is None), name
        if want is None:
            continue
        assert got.dtype == want.dtype == torch.float32
        rel = float((got - want).norm() / want.norm().clamp_min(1e-12))
        # (a handful of scalars has no meaningful relative error: a sum that happens to be small is all noise)
        assert rel <= 5e-2 or want.numel() < 64, (name, rel)
        assert torch.allclose(got, want, atol=5e-2, rtol=5e-2), name
    # parameter_vjp of a region on the same cache: fp32 gradients for fp32 parameters
    cot = torch.randn(2, 192, 128, device=device)
    rc = cache["region_caches"][1].backend_cache
    grads = model.region_backend.lowering.parameter_vjp(backend=model.region_backend, cache=rc, output_cotangent=cot)
    params = dict(model.region_backend.named_parameters())
    assert grads and all(g.dtype == params[n].dtype and g.shape == params[n].shape for n, g in grads.items())


def test_step_leaves_out_the_last_regions_jacobian_unless_statistics_read_it(device):
    """The last region's state Jacobian never enters the adjoints (reference backward/suffix_scan.py:71-74).  The
    step asks the structured provider to leave it out: one region pullback less, the same gradients bit for bit as
    with a provider that builds it; with the Jacobian statistics on it is built, since they report its norms."""
    from latent_bounded_interfaces_amd.backward import StructuredInterfacePullbackProvider, lbi_scan_backward_step

    model = _model(device)
    gen = torch.Generator().manual_seed(5)
    ids = torch.randint(0, 61, (2, 10), generator=gen).to(device)
    targets = torch.randint(0, 61, (2, 10), generator=gen).to(device)

    class BuildsAll:
        """The same provider without the option."""
        name = "structured"

        def __init__(self):
            self.inner = StructuredInterfacePullbackProvider()

        def materialize_state_jacobian_t(self, *, model, cache):
            return self.inner.materialize_state_jacobian_t(model=model, cache=cache)

    calls = []
    inner = model.region_backend.input_pullback_basis

    def spy(*, cache, output_cotangent_basis):
        calls.append(cache.region_index)
        return inner(cache=cache, output_cotangent_basis=output_cotangent_basis)

    def step(provider, **kw):
        logits, cache = model.forward_with_cache(ids)
        loss = olbi.token_loss(logits, targets)
        calls.clear()
        model.region_backend.input_pullback_basis = spy
        try:
            result = lbi_scan_backward_step(model, ce_loss=loss, cache=cache, pullback_provider=provider, **kw)
        finally:
            del model.region_backend.input_pullback_basis
        return result, list(calls), cache

    got, got_calls, cache = step(StructuredInterfacePullbackProvider())
    want, want_calls, _ = step(BuildsAll())
    assert got_calls == [0, 1] and want_calls == [0, 1, 2]
    assert got.interface_scan_rms == want.interface_scan_rms
    assert set(got.grad_map) == set(want.grad_map)
    for name, value in want.grad_map.items():
        assert (got.grad_map[name] is None) == (value is None), name
        if value is not None:
            assert torch.equal(got.grad_map[name], value), name
    with_stats, stats_calls, _ = step(StructuredInterfacePullbackProvider(), compute_interface_jacobian_stats=True)
    assert stats_calls == [0, 1, 2] and with_stats.interface_jacobian_stats is not None
    # the provider's own contract
    provider = StructuredInterfacePullbackProvider()
    full = provider.materialize_state_jacobian_t(model=model, cache=cache)
    short = provider.materialize_state_jacobian_t(model=model, cache=cache, skip_last=True)
    assert len(short) == len(full) == 3 and short[-1] is None
    assert all(torch.equal(a, b) for a, b in zip(short[:-1], full[:-1]))


def test_scan_cross_check_compares_two_independent_results_in_the_k_parallel_form(device):
    """With few batch elements and a long chain the scan runs its chunks side by side and forms the cotangents by
    applying the finished products to g.  ``interface_scan_rms`` must still compare two results that share nothing:
    the applied suffix matrices against the sequential chain of a kernel of its own, so it is tiny but not zero."""
    from latent_bounded_interfaces_amd.backward.scan import _adjoints_and_scan_rms
    from oracle import scan as oscan

    for bsz, count, rank in ((1, 16, 64), (2, 24, 256), (4, 5, 64)):
        mats, g = oscan.make_scan_inputs(bsz, count, rank, kind="near_identity", seed=5)
        jts = [mats[:, r].to(device) for r in range(count)] + [torch.zeros(bsz, rank, rank, device=device)]
        adjoints, rms = _adjoints_and_scan_rms(jts, g.to(device))
        assert 0.0 < rms < 1e-5, (bsz, count, rank, rms)
        want = oscan.suffix_cotangents_sequential(mats.double(), g.double())
        assert len(adjoints) == count + 1
        for r, a in enumerate(adjoints):
            assert torch.allclose(a.cpu().double(), want[:, r], atol=1e-5, rtol=1e-5), (bsz, count, rank, r)


def test_engine_from_a_reference_configuration_pulls_all_directions_back_in_one_call(device):
    """The reference's configuration defaults ``jacobian_basis_chunk`` to 1 and rejects values <= 0
    (train/config.py:169, :330): that knob is for its autograd providers.  ``from_config`` with
    ``interface_jacobian_mode="structured"`` must not turn it into one region pullback per direction."""
    from types import SimpleNamespace

    from latent_bounded_interfaces_amd.backward import ScanADEngine, lbi_reference_scan_backward_step

    model = _model(device)
    cfg = SimpleNamespace(interface_jacobian_mode="structured", jacobian_basis_chunk=1,
                          log_interface_jacobian_suffix=False)
    engine = ScanADEngine.from_config(cfg)
    assert engine.pullback_provider.name == "structured" and engine.pullback_provider.basis_chunk == 0
    assert ScanADEngine(state_jacobian_mode="structured").pullback_provider.basis_chunk == 0
    assert ScanADEngine(state_jacobian_mode="recompute").pullback_provider.basis_chunk == 1
    assert ScanADEngine.from_config(SimpleNamespace(interface_jacobian_mode="recompute", jacobian_basis_chunk=3,
                                                    log_interface_jacobian_suffix=False)
                                    ).pullback_provider.basis_chunk == 3
    cfg.structured_basis_chunk = 4
    assert ScanADEngine.from_config(cfg).pullback_provider.basis_chunk == 4
    calls = []
    inner = model.region_backend.input_pullback_basis

    def spy(*, cache, output_cotangent_basis):
        calls.append((cache.region_index, int(output_cotangent_basis.shape[1])))
        return inner(cache=cache, output_cotangent_basis=output_cotangent_basis)

    model.region_backend.input_pullback_basis = spy
    try:
        loss, cache, dense = _step_inputs(model, device)
        result = engine.backward(model=model, loss=loss, cache=cache)
        assert calls == [(0, 8), (1, 8)]           # one call per region that the scan reads, all 8 directions
        _check_grads(result.grad_map, dense)
        calls.clear()
        loss, cache, dense = _step_inputs(model, device)
        lbi_reference_scan_backward_step(model, ce_loss=loss, cache=cache, state_jacobian_mode="structured")
        assert calls == [(0, 8), (1, 8)]
    finally:
        del model.region_backend.input_pullback_basis


@pytest.mark.parametrize("layers,per_region", [(6, 2), (3, 1), (2, 2)])
def test_structured_local_vjp_provider_matches_the_autograd_provider_and_dense_gradients(layers, per_region, device):
    """Region parameter VJPs from the forward cache on the HIP kernels (``StructuredLocalVJPProvider``) against the
    reference's provider (autograd on the forward graph) and against ``loss.backward()``, fp32 bar of the reference
    (tests/test_lbi_gradient_parity.py:40-41); same ``None`` pattern (parameters the loss does not reach)."""
    from latent_bounded_interfaces_amd.backward import (ScanADEngine, StructuredInterfacePullbackProvider,
                                                        StructuredLocalVJPProvider, lbi_scan_backward_step)

    model = _model(device, layers=layers, layers_per_region=per_region)
    loss, cache, dense = _step_inputs(model, device)
    want = lbi_scan_backward_step(model, ce_loss=loss, cache=cache,
                                  pullback_provider=StructuredInterfacePullbackProvider())
    loss, cache, _ = _step_inputs(model, device)
    got = lbi_scan_backward_step(model, ce_loss=loss, cache=cache,
                                 pullback_provider=StructuredInterfacePullbackProvider(),
                                 local_vjp_provider=StructuredLocalVJPProvider())
    assert got.interface_scan_rms < 1e-5
    _check_grads(got.grad_map, dense)
    _check_grads(got.grad_map, want.grad_map)
    # through the engine, by mode name, and from a configuration object
    from types import SimpleNamespace

    loss, cache, _ = _step_inputs(model, device)
    engine = ScanADEngine(state_jacobian_mode="structured", local_vjp_mode="structured")
    result = engine.backward(model=model, loss=loss, cache=cache)
    assert result.diagnostics["local_vjp_provider"] == "structured"
    _check_grads(result.grad_map, dense)
    cfg = SimpleNamespace(interface_jacobian_mode="structured", jacobian_basis_chunk=1,
                          log_interface_jacobian_suffix=False, local_vjp_mode="structured")
    assert ScanADEngine.from_config(cfg).local_vjp_provider.name == "structured"


def test_structured_local_vjp_provider_on_16bit_weights(device):
    """bf16 weights and activations, fp32 interface, heads of 64 and T = 320 (the matrix-core attention kernels run
    in the sweeps): against fp32 dense gradients on the same rounded weights at the reference's 16-bit bar."""
    import copy

    from latent_bounded_interfaces_amd.backward import ScanADEngine

    model = _model(device, dtype=torch.bfloat16, dim=128, n_heads=2, n_kv_heads=2, hidden=256, layers=4,
                   layers_per_region=2, interface_width=64, interface_hidden=96, seed=37)
    dense_model = copy.deepcopy(model).float()
    dense_model.region_backend.lowering = None
    gen = torch.Generator().manual_seed(9)
    ids = torch.randint(0, 61, (2, 320), generator=gen).to(device)
    targets = torch.randint(0, 61, (2, 320), generator=gen).to(device)
    _, dense = olbi.dense_gradients(dense_model, ids, targets)
    logits, cache = model.forward_with_cache(ids)
    engine = ScanADEngine(state_jacobian_mode="structured", local_vjp_mode="structured")
    result = engine.backward(model=model, loss=olbi.token_loss(logits, targets), cache=cache)
    params = dict(model.named_parameters())
    for name, want in dense.items():
        got = result.grad_map[name]
        assert (got is None) == (want is None), name
        if want is None:
            continue
        assert got.dtype == params[name].dtype and got.shape == want.shape, name
        assert torch.allclose(got.float(), want, atol=5e-2, rtol=5e-2), (name, float((got.float() - want).abs().max()))
        rel = float((got.float() - want).norm() / want.norm().clamp_min(1e-12))
        # (a handful of scalars has no meaningful relative error: a sum that happens to be small is all noise)
        assert rel <= 5e-2 or want.numel() < 64, (name, rel)
