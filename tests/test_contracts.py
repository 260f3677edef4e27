"""The structural contracts of the package (CPU): its classes satisfy the protocols they stand in for, and the
cache-field lists name exactly what the region code reads."""
from __future__ import annotations

import re
from pathlib import Path

from latent_bounded_interfaces_amd import contracts
from latent_bounded_interfaces_amd.backends import HipTransformerLowering
from latent_bounded_interfaces_amd.backward import StructuredInterfacePullbackProvider, build_interface_pullback_provider
from oracle import lbi_model

REGION_SOURCE = (Path(contracts.__file__).parent / "hip" / "transformer" / "region.py").read_text()

# the reference's cache dataclasses (backends/transformer.py:17-61, backends/base.py:10-13)
REFERENCE_ATTENTION_CACHE = {"norm_input", "norm_output", "qkv", "q", "k", "v", "q_rope", "k_rope", "k_expanded",
                             "v_expanded", "attn_output", "out_proj_input", "out_proj_output"}
REFERENCE_MLP_CACHE = {"norm_input", "norm_output", "fc1_output", "up", "gate", "activation", "down_input",
                       "down_output"}
REFERENCE_LAYER_CACHE = {"layer_index", "hidden_input", "residual_input", "attention", "mlp", "hidden_output",
                         "residual_output"}
REFERENCE_REGION_CACHE = {"region_index", "layer_range", "layer_caches", "region_input", "region_output"}


def test_offered_classes_satisfy_their_protocols():
    lowering = HipTransformerLowering()
    assert isinstance(lowering, contracts.TransformerLowering) and lowering.name == "hip"
    provider = StructuredInterfacePullbackProvider()
    assert isinstance(provider, contracts.InterfacePullbackProvider) and provider.name == "structured"
    assert isinstance(build_interface_pullback_provider("structured"), contracts.InterfacePullbackProvider)
    assert not isinstance(object(), contracts.TransformerLowering)


def test_default_providers_and_engine_satisfy_the_protocols():
    from latent_bounded_interfaces_amd import backward

    assert isinstance(backward.TorchAutogradLocalVJPProvider(), contracts.LocalVJPProvider)
    for mode, name in (("graph", "torch_graph"), ("recompute", "torch_recompute")):
        provider = build_interface_pullback_provider(mode)
        assert isinstance(provider, contracts.InterfacePullbackProvider) and provider.name == name
        assert provider.basis_chunk == 1
    engine = backward.ScanADEngine(state_jacobian_mode="recompute", state_jacobian_basis_chunk=32)
    assert engine.name == "scan" and engine.pullback_provider.basis_chunk == 32
    assert engine.local_vjp_provider.name == "torch_autograd"
    assert callable(backward.lbi_reference_scan_backward_step)
    # every public name of the reference's backward package that lies on this path is importable from here
    for name in ("ADEngine", "ADResult", "GradMap", "LBIBackwardResult", "ReferenceScanEngine", "ScanADEngine",
                 "ScanBackpropModel", "TorchAutogradLocalVJPProvider", "TorchGraphInterfacePullbackProvider",
                 "TorchRecomputeInterfacePullbackProvider", "assign_grad_map", "apply_jacobian_t",
                 "build_interface_pullback_provider", "collect_named_grads", "compose_suffix_jacobian_t",
                 "lbi_reference_scan_backward_step", "lbi_scan_backward_step",
                 "propagate_state_adjoint_by_autograd_chain", "propagate_state_adjoint_from_last_region_input",
                 "propagate_state_adjoint_with_jacobian_scan", "store_named_grads"):
        assert hasattr(backward, name), name


def test_test_side_providers_satisfy_the_needed_protocols():
    assert isinstance(lbi_model.AutogradLocalVJPProvider(), contracts.LocalVJPProvider)
    assert isinstance(lbi_model.GraphInterfacePullbackProvider(), contracts.InterfacePullbackProvider)


def _fields_read(prefix: str) -> set[str]:
    return set(re.findall(rf"\b{prefix}\.([a-z_0-9]+)", REGION_SOURCE))


def test_cache_field_lists_match_what_the_region_code_reads():
    assert _fields_read("a_cache") == set(contracts.ATTENTION_CACHE_FIELDS) <= REFERENCE_ATTENTION_CACHE
    assert _fields_read("m_cache") == set(contracts.MLP_CACHE_FIELDS) <= REFERENCE_MLP_CACHE
    assert _fields_read("layer_cache") == set(contracts.LAYER_CACHE_FIELDS) <= REFERENCE_LAYER_CACHE
    assert _fields_read("cache") == set(contracts.REGION_CACHE_FIELDS) <= REFERENCE_REGION_CACHE
