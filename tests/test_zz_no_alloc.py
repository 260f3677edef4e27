"""The allocation-free attention entry (``lbi_attn_pullback_static``, scratch memory in a static device array)
against ``lbi_attn_pullback`` with a caller-provided workspace: same kernels, so the results must be bit-identical,
on two calls in a row of which the second is smaller (it finds the first call's leftovers in the array)."""
from __future__ import annotations

import ctypes

import pytest
import torch

from latent_bounded_interfaces_amd import _lib

pytestmark = pytest.mark.gpu


def _inputs(shape, basis, dtype, seed, device):
    gen = torch.Generator(device=device).manual_seed(seed)
    q, k, v = (torch.randn(*shape, device=device, dtype=dtype, generator=gen) for _ in range(3))
    g = torch.randn(shape[0], basis, *shape[1:], device=device, dtype=dtype, generator=gen)
    return q, k, v, g


def _with_workspace(lib, q, k, v, g, scale, causal):
    bsz, heads, seq, hd = q.shape
    code = _lib.dtype_code(q.dtype)
    need = int(lib.lbi_attn_pullback_workspace_bytes(bsz, heads, seq, hd, g.shape[1], code))
    ws = torch.empty(max(need, 1), device=q.device, dtype=torch.uint8)
    outs = tuple(torch.empty_like(g) for _ in range(3))
    status = lib.lbi_attn_pullback(q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), *(o.data_ptr() for o in outs),
                                   ws.data_ptr(), need, bsz, heads, seq, hd, g.shape[1], scale, int(causal), code,
                                   _lib.current_stream_ptr(q.device))
    _lib.check(status, "lbi_attn_pullback")
    return outs, need


def _static(lib, q, k, v, g, scale, causal, first_on_device=False):
    bsz, heads, seq, hd = q.shape
    outs = tuple(torch.full_like(g, float("nan")) for _ in range(3))
    torch.cuda.synchronize()
    allocations = torch.cuda.memory_stats(q.device)["allocation.all.allocated"]
    free_before = torch.cuda.mem_get_info(q.device)[0]     # the driver's own count: sees a hipMalloc of the library too
    status = lib.lbi_attn_pullback_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(),
                                          *(o.data_ptr() for o in outs), bsz, heads, seq, hd, g.shape[1], scale,
                                          int(causal), _lib.dtype_code(q.dtype), _lib.current_stream_ptr(q.device))
    _lib.check(status, "lbi_attn_pullback_static")
    torch.cuda.synchronize()
    # nothing was taken from torch's allocator between entering and leaving the call
    assert torch.cuda.memory_stats(q.device)["allocation.all.allocated"] == allocations
    if not first_on_device:
        # (the first call on a device may make the runtime load the code object that holds the array)
        assert torch.cuda.mem_get_info(q.device)[0] == free_before
    return outs


# (first call, second and smaller call): matrix-core four-kernel path, generic fp32 kernels, bf16 non-causal
CASES = [
    (((2, 4, 320, 64), 5, torch.float16, True), ((1, 2, 320, 64), 3, torch.float16, True)),
    (((2, 3, 50, 24), 3, torch.float32, True), ((1, 2, 17, 24), 2, torch.float32, False)),
    (((1, 2, 384, 128), 6, torch.bfloat16, False), ((1, 1, 192, 128), 1, torch.bfloat16, True)),
]


@pytest.mark.parametrize("first,second", CASES)
def test_static_scratch_entry_matches_the_workspace_entry(first, second, device):
    lib = _lib.load()
    with torch.cuda.device(device):
        for index, (shape, basis, dtype, causal) in enumerate((first, second)):
            q, k, v, g = _inputs(shape, basis, dtype, 50 + index, device)
            scale = shape[-1] ** -0.5
            want, need = _with_workspace(lib, q, k, v, g, scale, causal)
            assert 0 < need <= _lib.ATTN_STATIC_SCRATCH_BYTES      # the scratch array is really used
            got = _static(lib, q, k, v, g, scale, causal, first_on_device=index == 0)
            for name, a, b in zip(("dq", "dk", "dv"), got, want):
                assert torch.equal(a, b), (name, index, shape)


def test_static_scratch_entry_python_wrapper_and_limit(device):
    from latent_bounded_interfaces_amd.hip.transformer import (attention_input_pullback_basis,
                                                               attention_input_pullback_basis_static)

    q, k, v, g = _inputs((1, 2, 320, 64), 4, torch.float16, 7, device)
    want = attention_input_pullback_basis(q, k, v, g, softmax_scale=0.125, kernel_mode="hip")
    out = tuple(torch.empty_like(g) for _ in range(3))
    got = attention_input_pullback_basis_static(q, k, v, g, out, softmax_scale=0.125)
    assert all(a is b for a, b in zip(got, out)) and all(torch.equal(a, b) for a, b in zip(got, want))
    # beyond the static array: rejected on the host with a clear message, nothing launched
    lib = _lib.load()
    one = ctypes.c_void_p(256)
    assert lib.lbi_attn_pullback_workspace_bytes(4, 16, 4096, 128, 16, _lib.LBI_BF16) > _lib.ATTN_STATIC_SCRATCH_BYTES
    assert lib.lbi_attn_pullback_static(one, one, one, one, one, one, one, 4, 16, 4096, 128, 16, 0.1, 1,
                                        _lib.LBI_BF16, None) == -4
    assert b"static buffer holds" in lib.lbi_last_error()
    with pytest.raises(RuntimeError, match="contiguous"):
        attention_input_pullback_basis_static(q.transpose(1, 2).contiguous().transpose(1, 2), k, v, g, out,
                                              softmax_scale=0.125)


def test_static_scratch_entry_under_stream_capture(device):
    """What the entry is for: after one warm-up call outside the capture (which does the per-device look-ups), a
    call is captured into a graph and replayed; every replay, with eager work of the same entry in between, gives
    the eager result bit for bit."""
    lib = _lib.load()
    q, k, v, g = _inputs((2, 4, 320, 64), 5, torch.float16, 91, device)
    q2, k2, v2, g2 = _inputs((2, 4, 320, 64), 5, torch.float16, 92, device)
    scale = 0.125
    want, _ = _with_workspace(lib, q, k, v, g, scale, True)
    want2, _ = _with_workspace(lib, q2, k2, v2, g2, scale, True)
    outs = tuple(torch.zeros_like(g) for _ in range(3))
    other = tuple(torch.zeros_like(g) for _ in range(3))

    def call(args, dst):
        a, b, c, d = args
        status = lib.lbi_attn_pullback_static(a.data_ptr(), b.data_ptr(), c.data_ptr(), d.data_ptr(),
                                              *(o.data_ptr() for o in dst), 2, 4, 320, 64, 5, scale, 1,
                                              _lib.dtype_code(a.dtype), _lib.current_stream_ptr(a.device))
        _lib.check(status, "lbi_attn_pullback_static")

    call((q, k, v, g), outs)                       # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call((q, k, v, g), outs)
    for replay in range(3):
        for o in outs:
            o.zero_()
        call((q2, k2, v2, g2), other)              # eager work on the same scratch array between replays
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(other, want2)), replay
        graph.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(outs, want)), replay
