"""Writes ``tests/golden/reference_lbi_region.safetensors``: inputs and outputs of the REFERENCE's own Transformer region
backend, vector-MLP interface, LBI model and scan backward step on a tiny fixed-seed configuration.

Run in the build container only, where the reference checkout is mounted:

    python tests/golden/make_reference_region_fixtures.py [/root/reference]

The fixture holds tensors only (weights under the reference's parameter names, inputs, expected outputs); it is
read back with ``safetensors.torch.load_file`` (a loader that executes nothing from the file).  ``tests/test_oracle_reference_fixtures.py`` checks the CPU
restatements in ``oracle/transformer_region.py`` and ``oracle/lbi_model.py`` against it, which pins their
architecture (norm placement, residual handling, convolution, rotary pairing, head grouping, interface update) to
the reference's rather than to their own reading of it.  Nothing of the reference's source travels with the
fixture.
"""
from __future__ import annotations

import sys
from pathlib import Path

import torch

REFERENCE = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
OUT = Path(__file__).resolve().parent / "reference_lbi_region.safetensors"

# three regions (2 + 2 + 1 layers) so that the scan composes two Jacobians; grouped key/value heads; odd sizes
CONFIG = dict(vocab_size=11, dim=8, layers=5, layers_per_region=2, n_heads=2, n_kv_heads=1, d_intermediate=12, d_conv=3,
              interface_width=5, interface_hidden=6, batch=2, seq_len=5, basis=3)


def main() -> None:
    sys.path.insert(0, str(REFERENCE))
    from backbones.general import BackboneSpec
    from backward import lbi_reference_scan_backward_step
    from backward.autograd import autograd_backward_step
    from backward.pullbacks import (materialize_interface_state_jacobian_t_graph,
                                    materialize_interface_state_jacobian_t_recompute)
    from interfaces.vector_mlp import VectorMLPInterface
    from models.lbi_language_model import LBILanguageModel

    c = CONFIG
    torch.manual_seed(20240611)
    spec = BackboneSpec(name="transformer", dim=c["dim"], layers=c["layers"], n_heads=c["n_heads"],
                        n_kv_heads=c["n_kv_heads"], d_intermediate=c["d_intermediate"], d_conv=c["d_conv"],
                        use_flash_attn=False)
    interface = VectorMLPInterface(feature_dim=c["dim"], num_regions=-(-c["layers"] // c["layers_per_region"]),
                                   interface_width=c["interface_width"], interface_map_hidden_dim=c["interface_hidden"])
    model = LBILanguageModel(vocab_size=c["vocab_size"], layers_per_region=c["layers_per_region"], backbone_spec=spec,
                             interface=interface)
    # the initialisers leave biases and some gates at zero; perturb every parameter so nothing is hidden by a zero
    with torch.no_grad():
        for p in model.parameters():
            p.add_(0.05 * torch.randn_like(p))
    model = model.float()
    ids = torch.randint(0, c["vocab_size"], (c["batch"], c["seq_len"]))
    targets = torch.randint(0, c["vocab_size"], (c["batch"], c["seq_len"]))

    fix: dict[str, torch.Tensor] = {"input_ids": ids, "targets": targets}
    for name, value in c.items():
        fix[f"config.{name}"] = torch.tensor(value)
    for name, p in model.state_dict().items():
        fix[f"param.{name}"] = p.detach().clone()
    block0 = model.region_backend.backbone.blocks[0]
    for name in ("n_heads", "n_kv_heads", "head_dim", "d_conv"):
        fix[f"attn.{name}"] = torch.tensor(int(getattr(block0.attn, name)))
    fix["attn.rope_base"] = torch.tensor(float(block0.attn.rope_base))
    fix["attn.rope_interleaved"] = torch.tensor(bool(block0.attn.rope_interleaved))
    fix["attn.softmax_scale"] = torch.tensor(float(block0.attn.softmax_scale or 0.0))
    fix["block.residual_in_fp32"] = torch.tensor(bool(block0.residual_in_fp32))
    fix["norm.eps"] = torch.tensor(float(block0.norm.eps))

    logits, cache = model.forward_with_cache(ids)
    loss = torch.nn.functional.cross_entropy(logits.float().reshape(-1, c["vocab_size"]), targets.reshape(-1))
    fix["logits"] = logits.detach()
    fix["loss"] = loss.detach()
    cache_d = cache if isinstance(cache, dict) else vars(cache)
    for i, s in enumerate(cache_d["states"]):
        fix[f"state.{i}"] = s.detach()
    for i, (x, y) in enumerate(zip(cache_d["region_inputs"], cache_d["region_outputs"])):
        fix[f"region_input.{i}"] = x.detach()
        fix[f"region_output.{i}"] = y.detach()
    # the per-layer cache fields a lowering reads, for region 1 (its layers see a non-trivial residual stream)
    rc = cache_d["region_caches"][1]
    for layer_cache in rc.backend_cache.layer_caches:
        li = layer_cache.layer_index
        for part in ("attention", "mlp"):
            for field, value in vars(getattr(layer_cache, part)).items():
                if torch.is_tensor(value):
                    fix[f"cache.{li}.{part}.{field}"] = value.detach()

    gen = torch.Generator().manual_seed(7)
    basis = torch.randn(c["batch"], c["basis"], c["seq_len"], c["dim"], generator=gen)
    cot = torch.randn(c["batch"], c["seq_len"], c["dim"], generator=gen)
    fix["region1.basis"] = basis
    fix["region1.input_pullback_basis"] = model.region_backend.input_pullback_basis(
        cache=rc.backend_cache, output_cotangent_basis=basis).detach()
    fix["region1.output_cotangent"] = cot
    for name, grad in model.region_backend.parameter_vjp(cache=rc.backend_cache, output_cotangent=cot).items():
        fix[f"region1.parameter_vjp.{name}"] = grad.detach()

    eye = torch.eye(c["interface_width"]).unsqueeze(0).expand(c["batch"], -1, -1)
    upd = model.interface.apply_update_jacobian_t_to_region_output(region_cache=rc, state_out_cotangent_basis=eye)
    for name, value in upd.items():
        fix[f"interface1.update.{name}"] = value.detach().contiguous()
    g_in = torch.randn(c["batch"], c["interface_width"], c["seq_len"], c["dim"], generator=gen)
    fix["interface1.decode.region_input_cotangent_basis"] = g_in
    dec = model.interface.apply_decode_jacobian_t_to_state_input(region_cache=rc, region_input_cotangent_basis=g_in)
    for name, value in dec.items():
        fix[f"interface1.decode.{name}"] = value.detach().contiguous()

    for i, jt in enumerate(materialize_interface_state_jacobian_t_graph(model=model, cache=cache)):
        fix[f"jt_graph.{i}"] = jt.detach()
    for i, jt in enumerate(materialize_interface_state_jacobian_t_recompute(model=model, cache=cache, basis_chunk=2)):
        fix[f"jt_recompute.{i}"] = jt.detach()

    result = lbi_reference_scan_backward_step(model, ce_loss=loss, cache=cache, state_jacobian_mode="graph")
    fix["scan_step.interface_scan_rms"] = torch.tensor(float(result.interface_scan_rms))
    for name, grad in result.grad_map.items():
        if grad is not None:
            fix[f"scan_step.grad.{name}"] = grad.detach()
    logits2, _ = model.forward_with_cache(ids)
    loss2 = torch.nn.functional.cross_entropy(logits2.float().reshape(-1, c["vocab_size"]), targets.reshape(-1))
    for name, grad in autograd_backward_step(model, ce_loss=loss2).items():
        if grad is not None:
            fix[f"dense.grad.{name}"] = grad.detach()

    from safetensors.torch import save_file

    save_file({k: v.detach().clone().contiguous() for k, v in fix.items()}, str(OUT))
    print(f"wrote {OUT}: {len(fix)} tensors, {OUT.stat().st_size} bytes")


if __name__ == "__main__":
    main()
