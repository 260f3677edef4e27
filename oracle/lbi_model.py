"""Small stand-in for the reference's LBI language model and its autograd providers.
TEST INFRASTRUCTURE ONLY: nothing under the product package imports this module.

Restated (reference file:line), with the reference's attribute names so that code written
against the reference's objects runs on these:

* vector-MLP interface: initialize / decode / update and the structured pullbacks
  ``apply_update_jacobian_t_to_region_output`` / ``apply_decode_jacobian_t_to_state_input``
  (interfaces/vector_mlp.py:137-270; here the pullbacks are taken by autograd through the
  restated forward pieces, which pins them to the forward by construction)
* model forward with cache: canvas (token embedding) -> per region: condition =
  decode(state), region_input = canvas + condition, region forward, interface update ->
  readout (final RMSNorm + LM head) (models/lbi_language_model.py:150-221; cache fields
  :34-55)
* autograd local-VJP provider (backward/local_vjp.py:66-185)
* graph interface-pullback provider (backward/pullbacks.py:37-81)

Pinned by tests/test_oracle_region.py::test_lbi_model_*: the state Jacobians of the graph
provider against finite differences of the state map, and the scan backward step run with
these providers against ``loss.backward()`` of the same graph.
"""
from __future__ import annotations

from types import SimpleNamespace

import torch
import torch.nn.functional as F
from torch import nn

from . import transformer_region as oreg


class OracleVectorInterface(nn.Module):
    def __init__(self, *, feature_dim: int, num_regions: int, interface_width: int, hidden_dim: int = 0,
                 update_scale_init: float = 0.5) -> None:
        super().__init__()

        def head(i, o):
            if hidden_dim > 0:
                return nn.Sequential(nn.Linear(i, hidden_dim), nn.SiLU(), nn.Linear(hidden_dim, o))
            return nn.Linear(i, o)

        self.initial_encoder = head(feature_dim, interface_width)
        self.decoders = nn.ModuleList([head(interface_width, feature_dim) for _ in range(num_regions)])
        self.encoders = nn.ModuleList([head(feature_dim, interface_width) for _ in range(num_regions)])
        self.norms = nn.ModuleList([nn.LayerNorm(interface_width) for _ in range(num_regions)])
        self.update_scale = nn.Parameter(torch.full((num_regions,), float(update_scale_init)))

    @staticmethod
    def _run(module, x):
        return module(x.to(next(module.parameters()).dtype))

    @staticmethod
    def summarize_features(features: torch.Tensor) -> torch.Tensor:
        return features.mean(dim=1).to(features.dtype)

    def initialize(self, canvas_features):
        return self._run(self.initial_encoder, self.summarize_features(canvas_features))

    def decode(self, state, region_index):
        return self._run(self.decoders[region_index], state)

    def update(self, state, region_features, region_index):
        pooled = self.summarize_features(region_features)
        delta = self._run(self.encoders[region_index], pooled)
        scale = torch.tanh(self.update_scale[region_index])
        pre = state + scale * delta
        return SimpleNamespace(state=self.norms[region_index](pre),
                               diagnostics={"pooled_features": pooled, "delta_state": delta, "update_scale": scale,
                                            "pre_norm_state": pre})

    def initial_vjp_parameters(self):
        return list(self.initial_encoder.parameters())

    def region_vjp_parameters(self, region_index):
        return [*self.decoders[region_index].parameters(), *self.encoders[region_index].parameters(),
                *self.norms[region_index].parameters()]

    def shared_vjp_parameters(self):
        return [self.update_scale]

    @staticmethod
    def _vjp_rows(fn, x, g_out, dtype=None):
        """g_out [B, P, O] pulled back through fn at x [B, I] -> [B, P, I].  ``dtype``: the dtype fn computes in
        (its parameters'); a forward run under autocast leaves some interface activations and states in the
        autocast dtype, while the pullback runs outside autocast."""
        bsz, basis = g_out.shape[:2]
        dtype = dtype or g_out.dtype
        with torch.enable_grad():
            x_rep = (x.detach().to(dtype).unsqueeze(1).expand(bsz, basis, x.shape[-1]).reshape(bsz * basis, -1)
                     .requires_grad_(True))
            y = fn(x_rep)
            (g_in,) = torch.autograd.grad(y, x_rep, grad_outputs=g_out.reshape_as(y).to(y.dtype))
        return g_in.reshape(bsz, basis, -1).to(g_out.dtype)

    def apply_update_jacobian_t_to_region_output(self, *, region_cache, state_out_cotangent_basis):
        if state_out_cotangent_basis.dim() != 3:
            raise ValueError("state_out_cotangent_basis must have shape [B, P, R].")
        r = region_cache.region_index
        diag = region_cache.interface_step.diagnostics
        g_pre = self._vjp_rows(self.norms[r], diag["pre_norm_state"], state_out_cotangent_basis,
                              dtype=self.norms[r].weight.dtype)
        g_delta = g_pre * diag["update_scale"].to(g_pre.dtype)
        g_pooled = self._vjp_rows(lambda t: self._run(self.encoders[r], t), diag["pooled_features"], g_delta)
        seq_len = region_cache.region_output.shape[1]
        g_out = g_pooled.unsqueeze(2).expand(-1, -1, seq_len, -1) / float(seq_len)
        return {"g_pre_norm_state": g_pre, "g_state_skip": g_pre, "g_delta_state": g_delta,
                "g_pooled_features": g_pooled, "g_region_output": g_out}

    def apply_decode_jacobian_t_to_state_input(self, *, region_cache, region_input_cotangent_basis):
        if region_input_cotangent_basis.dim() != 4:
            raise ValueError("region_input_cotangent_basis must have shape [B, P, L, D].")
        r = region_cache.region_index
        g_condition = region_input_cotangent_basis.sum(dim=2)
        g_state = self._vjp_rows(lambda t: self._run(self.decoders[r], t), region_cache.state_in, g_condition)
        return {"g_condition": g_condition, "g_state_input": g_state}


class _BackendWithLowering(oreg.OracleRegionBackend):
    """Adds the lowering dispatch of the reference's backend (backends/transformer.py:248-270)."""

    def __init__(self, blocks, region_ranges, lowering=None) -> None:
        super().__init__(blocks, region_ranges)
        self.lowering = lowering

    def input_pullback_basis(self, *, cache, output_cotangent_basis):
        if self.lowering is None:
            return oreg.input_pullback_basis_autograd(self, cache, output_cotangent_basis)
        return self.lowering.input_pullback_basis(backend=self, cache=cache, output_cotangent_basis=output_cotangent_basis)

    def parameter_vjp(self, *, cache, output_cotangent):
        if self.lowering is None:
            return oreg.parameter_vjp_autograd(self, cache, output_cotangent)
        return self.lowering.parameter_vjp(backend=self, cache=cache, output_cotangent=output_cotangent)


class OracleLBIModel(nn.Module):
    def __init__(self, *, vocab_size, dim, n_heads, layers, layers_per_region, interface_width, n_kv_heads=None,
                 hidden=None, d_conv=4, interface_hidden=0, lowering=None, dtype=torch.float32, seed=0) -> None:
        super().__init__()
        self.region_ranges = [(s, min(layers, s + layers_per_region)) for s in range(0, layers, layers_per_region)]
        self.num_regions = len(self.region_ranges)
        base = oreg.make_backend(dim=dim, n_heads=n_heads, n_kv_heads=n_kv_heads, hidden=hidden, layers=layers,
                                 region_ranges=self.region_ranges, d_conv=d_conv, dtype=dtype, seed=seed)
        self.region_backend = _BackendWithLowering(list(base.backbone.blocks), self.region_ranges, lowering)
        gen = torch.Generator(device="cpu").manual_seed(seed + 1)
        self.canvas = nn.Embedding(vocab_size, dim)
        self.interface = OracleVectorInterface(feature_dim=dim, num_regions=self.num_regions,
                                               interface_width=interface_width, hidden_dim=interface_hidden)
        self.readout_norm = oreg.OracleRMSNorm(dim)
        self.lm_head = nn.Linear(dim, vocab_size, bias=False)
        with torch.no_grad():
            # every parameter from the seeded generator (none from the process-wide one, whose state depends on
            # what ran before): matrices ~ N(0, 1 / fan_in), biases ~ 0.1 N(0, 1), LayerNorm weights 1 + 0.1 N(0, 1);
            # the update scale keeps its constant initial value
            for module in (self.canvas, self.interface, self.lm_head):
                for name, p in module.named_parameters():
                    if p.dim() >= 2:
                        p.copy_(torch.randn(p.shape, generator=gen) * p.shape[-1] ** -0.5)
                    elif name == "update_scale":
                        continue
                    elif "norms." in name and name.endswith("weight"):
                        p.copy_(1.0 + 0.1 * torch.randn(p.shape, generator=gen))
                    else:
                        p.copy_(0.1 * torch.randn(p.shape, generator=gen))
        self.canvas.to(dtype)
        self.readout_norm.to(dtype)
        self.lm_head.to(dtype)

    def output_head_vjp_parameters(self):
        return [*self.readout_norm.parameters(), *self.lm_head.parameters()]

    def canvas_vjp_parameters(self):
        return list(self.canvas.parameters())

    def shared_local_vjp_parameters(self):
        return [*self.canvas_vjp_parameters(), *self.interface.shared_vjp_parameters()]

    def forward_with_cache(self, input_ids):
        canvas_features = self.canvas(input_ids)
        state = self.interface.initialize(canvas_features)
        states, region_caches = [state], []
        region_output = None
        for region_index, layer_range in enumerate(self.region_ranges):
            state_in = state
            condition = self.interface.decode(state_in, region_index)
            region_input = canvas_features + condition.unsqueeze(1).to(canvas_features.dtype)
            region_output, backend_cache = self.region_backend.forward_region(region_input=region_input,
                                                                              region_index=region_index)
            step = self.interface.update(state_in, region_output, region_index)
            state = step.state
            states.append(state)
            region_caches.append(SimpleNamespace(region_index=region_index, layer_range=layer_range,
                                                 backend_cache=backend_cache, canvas_features=canvas_features,
                                                 state_in=state_in, condition=condition, region_input=region_input,
                                                 region_output=region_output, interface_step=step, state_out=state))
        normed = self.readout_norm(region_output.to(self.readout_norm.weight.dtype))
        logits = self.lm_head(normed)
        return logits, {"canvas_features": canvas_features, "states": states,
                        "region_inputs": [rc.region_input for rc in region_caches],
                        "region_outputs": [rc.region_output for rc in region_caches],
                        "region_ranges": self.region_ranges, "region_caches": region_caches}


#: the end-to-end benchmark configuration: 12 layers, d_model 768, 12 heads of 64, vocabulary 50257, 6 regions of
#: 2 layers, vector-MLP interface of width 64 (16-bit weights and activations, fp32 interface), batch 8, T 1024
END_TO_END = dict(vocab_size=50257, dim=768, n_heads=12, n_kv_heads=12, layers=12, layers_per_region=2,
                  interface_width=64, hidden=3072, d_conv=4, interface_hidden=0)
END_TO_END_BATCH, END_TO_END_SEQ = 8, 1024


def end_to_end_model(*, dtype=torch.bfloat16, lowering=None, seed=0, **overrides) -> "OracleLBIModel":
    """The stand-in model at the end-to-end configuration (random init from a fixed seed)."""
    return OracleLBIModel(**{**END_TO_END, **overrides}, lowering=lowering, dtype=dtype, seed=seed)


def end_to_end_batch(*, batch=END_TO_END_BATCH, seq_len=END_TO_END_SEQ, vocab_size=END_TO_END["vocab_size"], seed=0):
    """Token ids and targets, uniform over the vocabulary, from a CPU generator."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randint(0, vocab_size, (batch, seq_len), generator=gen),
            torch.randint(0, vocab_size, (batch, seq_len), generator=gen))


def token_loss(logits: torch.Tensor, targets: torch.Tensor) -> torch.Tensor:
    return F.cross_entropy(logits.float().flatten(0, 1), targets.flatten())


class AutogradLocalVJPProvider:
    """Local parameter VJPs by ``torch.autograd.grad`` on the forward graph."""

    name = "torch_autograd"

    @staticmethod
    def _names(model):
        return {id(p): n for n, p in model.named_parameters() if p.requires_grad}

    def new_grad_map(self, model):
        return {n: None for n, p in model.named_parameters() if p.requires_grad}

    def _store(self, model, grad_map, params, grads):
        names = self._names(model)
        for p, g in zip(params, grads):
            grad_map[names[id(p)]] = None if g is None else g.detach().clone()

    def store_output_head_grads(self, *, model, loss, grad_map):
        params = model.output_head_vjp_parameters()
        self._store(model, grad_map, params, torch.autograd.grad(loss, params, retain_graph=True, allow_unused=True))

    def state_adjoint_from_loss(self, *, loss, state):
        return torch.autograd.grad(loss, state, retain_graph=True)[0].detach().to(state.dtype)

    def store_initial_interface_grads(self, *, model, state0, state0_adjoint, grad_map):
        params = model.interface.initial_vjp_parameters()
        grads = torch.autograd.grad(state0, params, grad_outputs=state0_adjoint.to(state0.dtype), retain_graph=True,
                                    allow_unused=True)
        self._store(model, grad_map, params, grads)

    def store_region_grads(self, *, model, loss, states, region_index, num_regions, state_adjoints, grad_map):
        params = [*model.region_backend.parameters_for_region(region_index),
                  *model.interface.region_vjp_parameters(region_index)]
        if region_index < num_regions - 1:
            grads = torch.autograd.grad(states[region_index + 1], params,
                                        grad_outputs=state_adjoints[region_index + 1].to(states[region_index + 1].dtype),
                                        retain_graph=True, allow_unused=True)
        else:
            grads = torch.autograd.grad(loss, params, retain_graph=True, allow_unused=True)
        self._store(model, grad_map, params, grads)

    def store_shared_canvas_grads(self, *, model, loss, grad_map):
        params = model.shared_local_vjp_parameters()
        self._store(model, grad_map, params, torch.autograd.grad(loss, params, retain_graph=False, allow_unused=True))


class GraphInterfacePullbackProvider:
    """``Jt[b, i, j] = d s_out[j] / d s_in[i]`` per region from the forward graph, one column at a time."""

    name = "torch_graph"

    def materialize_state_jacobian_t(self, *, model, cache):
        states = cache["states"]
        out = []
        for r in range(model.num_regions):
            s_in, s_out = states[r], states[r + 1]
            bsz, rank = s_out.shape
            cols = []
            for j in range(rank):
                g = torch.zeros(bsz, rank, dtype=s_out.dtype, device=s_out.device)
                g[:, j] = 1.0
                cols.append(torch.autograd.grad(s_out, s_in, grad_outputs=g, retain_graph=True)[0].unsqueeze(-1))
            out.append(torch.cat(cols, dim=-1))
        return out


def scan_backward_step_sequential(model, *, loss, cache, pullback_provider, local_vjp_provider):
    """The reference's scan backward step (backward/scan.py:18-97) with the state adjoints from
    the sequential chain ``g_r = Jt_r g_{r+1}`` (its own cross-check, :63-69)."""
    grad_map = local_vjp_provider.new_grad_map(model)
    states = list(cache["states"])
    n = model.num_regions
    local_vjp_provider.store_output_head_grads(model=model, loss=loss, grad_map=grad_map)
    if n == 1:
        adjoints = [local_vjp_provider.state_adjoint_from_loss(loss=loss, state=states[0])]
    else:
        g_last = local_vjp_provider.state_adjoint_from_loss(loss=loss, state=states[-2])
        jts = pullback_provider.materialize_state_jacobian_t(model=model, cache=cache)
        adjoints = [None] * n
        adjoints[-1] = g_last
        for r in reversed(range(n - 1)):
            adjoints[r] = torch.einsum("bij,bj->bi", jts[r].to(g_last.dtype), adjoints[r + 1])
    local_vjp_provider.store_initial_interface_grads(model=model, state0=states[0], state0_adjoint=adjoints[0],
                                                     grad_map=grad_map)
    for r in range(n):
        local_vjp_provider.store_region_grads(model=model, loss=loss, states=states, region_index=r, num_regions=n,
                                              state_adjoints=adjoints, grad_map=grad_map)
    local_vjp_provider.store_shared_canvas_grads(model=model, loss=loss, grad_map=grad_map)
    return grad_map


def dense_gradients(model, input_ids, targets):
    """Full-autograd gradients of the same loss (the dense path the LBI step must reproduce)."""
    model.zero_grad(set_to_none=True)
    logits, _ = model.forward_with_cache(input_ids)
    loss = token_loss(logits, targets)
    loss.backward()
    grads = {n: (None if p.grad is None else p.grad.detach().clone()) for n, p in model.named_parameters()}
    model.zero_grad(set_to_none=True)
    return float(loss.detach()), grads
