"""The entry points record into a HIP graph: they neither allocate, synchronise nor clear memory with
stream memsets, so a captured sequence replays with new input values in the same buffers.  Each replay is
checked against the eager result on the same values, with eager work and synchronisation between replays."""
from __future__ import annotations

import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def _pipeline(mats, g, q, k, v, d_out):
    from latent_bounded_interfaces_amd.hip.interface import (matrix_norms, suffix_scan_cotangents,
                                                             suffix_scan_pullbacks_and_cotangents)
    from latent_bounded_interfaces_amd.hip.transformer import attention_input_pullback_basis

    suffix, cot = suffix_scan_pullbacks_and_cotangents(mats, g)
    chain = suffix_scan_cotangents(mats, g)
    spec, frob = matrix_norms(suffix)
    dq, dk, dv = attention_input_pullback_basis(q, k, v, d_out, softmax_scale=1.0 / math.sqrt(q.shape[-1]), causal=True,
                                                kernel_mode="hip")
    return suffix, cot, chain, spec, frob, dq, dk, dv


@pytest.mark.parametrize("dtype,rank", [(torch.float16, 32), (torch.bfloat16, 256)])
def test_captured_sequence_replays_with_new_inputs(dtype, rank, device):
    gen = torch.Generator().manual_seed(17)

    def fresh():
        mats = torch.randn(2, 5, rank, rank, generator=gen) * rank ** -0.5
        g = torch.randn(2, rank, generator=gen)
        q, k, v = (torch.randn(2, 2, 128, 64, generator=gen).to(dtype) for _ in range(3))
        d_out = torch.randn(2, 4, 2, 128, 64, generator=gen).to(dtype)
        return [t.to(device) for t in (mats, g, q, k, v, d_out)]

    static = fresh()
    # first calls outside the capture: code objects load and kernel attributes are set once per device
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _pipeline(*static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = _pipeline(*static)
    for _ in range(3):
        values = fresh()
        for dst, src in zip(static, values):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = _pipeline(*values)  # eager work between replays
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b)
