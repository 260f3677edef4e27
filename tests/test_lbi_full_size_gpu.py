"""The end-to-end configuration at its stated size, run as the training loop runs it
(reference train/runners.py:361-372: forward with cache, ``ScanADEngine.backward(model=, loss=, cache=)``):
12 layers of d_model 768 with 12 heads of 64, vocabulary 50257, 6 regions of 2 layers, interface width 64,
batch 8, sequence 1024, bf16 weights and activations, fp32 interface.  State Jacobians and region parameter VJPs
on the HIP kernels, interface scan on the HIP scan; gradients against the dense autograd path."""
import copy

import pytest
import torch

from oracle import lbi_model as olbi

pytestmark = pytest.mark.gpu


def _relative_l2(got, want):
    return float((got.float() - want.float()).norm() / want.float().norm().clamp_min(1e-30))


def test_end_to_end_step_at_full_size_reproduces_dense_gradients(device):
    from latent_bounded_interfaces_amd.backends import HipTransformerLowering
    from latent_bounded_interfaces_amd.backward import ScanADEngine

    model = olbi.end_to_end_model(lowering=HipTransformerLowering()).to(device)
    assert model.num_regions == 6 and next(model.region_backend.parameters()).dtype == torch.bfloat16
    assert next(model.interface.parameters()).dtype == torch.float32
    ids, targets = (t.to(device) for t in olbi.end_to_end_batch())

    # the dense path in fp32 on the same rounded weights (no lowering: plain autograd throughout)
    dense_model = copy.deepcopy(model).float()
    dense_model.region_backend.lowering = None
    loss_dense, dense = olbi.dense_gradients(dense_model, ids, targets)
    del dense_model
    torch.cuda.empty_cache()

    logits, cache = model.forward_with_cache(ids)
    loss = olbi.token_loss(logits, targets)
    # loss bar of the reference's 16-bit cases (tests/test_lbi_gradient_parity.py:731-732)
    assert abs(float(loss.detach()) - loss_dense) <= 5e-3 + 5e-3 * abs(loss_dense)
    engine = ScanADEngine(state_jacobian_mode="structured", local_vjp_mode="structured")
    result = engine.backward(model=model, loss=loss, cache=cache)
    assert result.diagnostics["interface_pullback_provider"] == "structured"
    assert result.diagnostics["local_vjp_provider"] == "structured"
    assert 0.0 < result.diagnostics["interface_scan_rms"] < 5e-5
    assert set(result.grad_map) == set(dense)

    # gradient bar of the reference's 16-bit cases (atol = rtol = 5e-2, tests/test_lbi_gradient_parity.py:729-730),
    # plus measures that do not vanish with small gradients: relative L2 per parameter group and over everything
    params = dict(model.named_parameters())
    squared_error = squared_norm = dot = got_norm = 0.0
    by_group: dict[str, list[float]] = {}
    for name, want in dense.items():
        got = result.grad_map[name]
        assert (got is None) == (want is None), name
        if want is None:
            continue
        assert got.shape == want.shape and got.dtype == params[name].dtype, name
        assert bool(torch.isfinite(got).all()), name
        assert torch.allclose(got.float(), want, atol=5e-2, rtol=5e-2), (name, float((got.float() - want).abs().max()))
        diff = got.double() - want.double()
        squared_error += float((diff * diff).sum())
        squared_norm += float((want.double() ** 2).sum())
        got_norm += float((got.double() ** 2).sum())
        dot += float((got.double() * want.double()).sum())
        group = "interface" if name.startswith("interface") else \
            ("blocks" if name.startswith("region_backend") else name.split(".")[0])
        if want.numel() >= 64:      # a handful of scalars (the update scales) has no meaningful relative error
            by_group.setdefault(group, []).append(_relative_l2(got, want))
    overall = (squared_error / squared_norm) ** 0.5
    cosine = dot / (got_norm ** 0.5 * squared_norm ** 0.5)
    worst = {group: max(values) for group, values in by_group.items()}
    print(f"\nfull-size step: loss {float(loss.detach()):.5f} (dense fp32 {loss_dense:.5f}), relative L2 overall "
          f"{overall:.3e}, cosine {cosine:.6f}, worst per group {worst}, scan rms "
          f"{result.diagnostics['interface_scan_rms']:.2e}")
    assert overall <= 5e-2, overall
    assert cosine >= 0.998, cosine
    assert max(worst.values()) <= 5e-2, worst

    # the same step with the reference's own local-VJP provider (autograd on the forward graph) agrees as well
    logits, cache = model.forward_with_cache(ids)
    loss = olbi.token_loss(logits, targets)
    default = ScanADEngine(state_jacobian_mode="structured").backward(model=model, loss=loss, cache=cache)
    for name, want in default.grad_map.items():
        got = result.grad_map[name]
        assert (got is None) == (want is None), name
        if want is not None:
            assert torch.allclose(got.float(), want.float(), atol=5e-2, rtol=5e-2), name
