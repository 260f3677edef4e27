"""The C ABI: the built library loads without a GPU and exports what include/lbi_hip.h declares."""
from __future__ import annotations

import ctypes
import re
from pathlib import Path

import pytest

from latent_bounded_interfaces_amd import _lib

HEADER = Path(__file__).resolve().parents[1] / "include" / "lbi_hip.h"


def _declared_symbols() -> list[str]:
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(lbi_[a-z_0-9]+)\s*\(", text)))


def test_header_declares_entry_points():
    names = _declared_symbols()
    assert {"lbi_suffix_scan", "lbi_suffix_cotangents", "lbi_attn_pullback",
            "lbi_attn_pullback_workspace_bytes", "lbi_last_error", "lbi_abi_version"} <= set(names)


def test_binding_table_matches_header():
    assert sorted(_lib.SYMBOLS) == _declared_symbols()


def test_library_exports_every_declared_symbol():
    if not _lib.LIB_PATH.exists():
        pytest.fail(f"{_lib.LIB_PATH} is not built; run python -m latent_bounded_interfaces_amd.build")
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in _declared_symbols():
        assert hasattr(lib, name), f"{name} missing from liblbi_hip.so"
    assert _lib.load().lbi_abi_version() == _lib.ABI_VERSION


def test_argument_validation_needs_no_gpu():
    """Contract violations are rejected on the host before any HIP call."""
    lib = _lib.load()
    assert lib.lbi_suffix_scan(None, None, -1, 2, 4, _lib.LBI_F32, _lib.LBI_F32, None) == -1
    assert b"negative" in lib.lbi_last_error()
    assert lib.lbi_suffix_scan(None, None, 1, 2, 4, 7, _lib.LBI_F32, None) == -1
    assert b"dtype" in lib.lbi_last_error()
    assert lib.lbi_suffix_scan(None, None, 1, 2, 4, _lib.LBI_F32, _lib.LBI_F32, None) == -1
    assert b"null" in lib.lbi_last_error()
    assert lib.lbi_suffix_scan(None, None, 0, 2, 4, _lib.LBI_F32, _lib.LBI_F32, None) == 0
    assert lib.lbi_last_error() == b""
    assert lib.lbi_suffix_cotangents(None, None, None, 1, 2, 4, _lib.LBI_F32, None) == -1
    # the scan entry with flags: unknown bits, g without cot, misaligned operands
    ok = ctypes.c_void_p(256)
    assert lib.lbi_suffix_scan_ex(ok, None, ok, None, 1, 2, 4, _lib.LBI_BF16, _lib.LBI_F32, 6, None) == -1
    assert b"flag" in lib.lbi_last_error()
    assert lib.lbi_suffix_scan_ex(ok, ok, ok, None, 1, 2, 4, _lib.LBI_BF16, _lib.LBI_F32, 0, None) == -1
    assert b"both" in lib.lbi_last_error()
    assert lib.lbi_suffix_scan_ex(ok, None, ctypes.c_void_p(260), None, 1, 2, 4, _lib.LBI_F32, _lib.LBI_F32,
                                  _lib.LBI_SCAN_EXACT_SUFFIX, None) == -1
    assert b"aligned" in lib.lbi_last_error()
    assert lib.lbi_suffix_scan_ex(None, None, None, None, 0, 2, 4, _lib.LBI_F32, _lib.LBI_F32, 1, None) == 0
    assert lib.lbi_suffix_apply(None, None, None, 1, 2, 4, None) == -1
    assert b"null" in lib.lbi_last_error()
    assert lib.lbi_suffix_apply(None, None, None, -1, 2, 4, None) == -1
    assert lib.lbi_suffix_apply(None, None, None, 0, 2, 4, None) == 0
    odd = ctypes.c_void_p(260)  # not 16-byte aligned
    assert lib.lbi_suffix_apply(odd, odd, odd, 1, 2, 4, None) == -1
    assert b"aligned" in lib.lbi_last_error()


def test_region_and_norm_entry_points_validate_on_the_host():
    lib = _lib.load()
    f32 = _lib.LBI_F32
    assert lib.lbi_rmsnorm_pullback(None, None, None, None, None, None, 1, 1, 1, 8, 1e-5, 0, f32, f32, None) == -1
    assert b"null" in lib.lbi_last_error()
    assert lib.lbi_gated_mlp_pullback(None, None, None, 1, 1, 1, 8, 0, 9, None) == -1
    assert lib.lbi_attn_heads_split(None, None, 1, 1, 1, 1, 8, f32, None) == -1
    one = ctypes.c_void_p(256)  # never dereferenced: every call below is rejected before any launch
    assert lib.lbi_attn_qkv_pullback(one, one, one, one, one, one, 1, 1, 4, 3, 2, 8, 0, f32, None) == -1
    assert b"multiple" in lib.lbi_last_error()
    assert lib.lbi_attn_qkv_conv_pullback(one, one, one, one, one, one, one, 1, 1, 4, 2, 2, 7, 0, 4, f32, None) == -1
    assert b"even head dim" in lib.lbi_last_error()
    assert lib.lbi_attn_qkv_conv_pullback(one, one, one, one, one, one, one, 1, 1, 4, 2, 2, 8, 0, 9, f32, None) == -2
    assert b"above 8" in lib.lbi_last_error()
    assert lib.lbi_causal_conv1d_pullback(one, one, one, 1, 4, 8, 4, f32, None) == -1
    assert b"in-place" in lib.lbi_last_error()
    # spectral / Frobenius norms: LDS-resident sizes need no workspace, larger ones two planes per workgroup
    assert lib.lbi_matrix_norms_workspace_bytes(10, 64) == 0
    assert lib.lbi_matrix_norms_workspace_bytes(10, 88) == 0
    assert lib.lbi_matrix_norms_workspace_bytes(10, 90) == 10 * 2 * 96 * 96 * 4
    assert lib.lbi_matrix_norms_workspace_bytes(5000, 256) == 1024 * 2 * 256 * 256 * 4
    assert lib.lbi_matrix_norms(one, one, one, None, 0, 4, 0, f32, None) == -1
    assert lib.lbi_matrix_norms(one, one, one, None, 0, 4, 256, f32, None) == -4
    assert b"workspace" in lib.lbi_last_error()
    assert lib.lbi_matrix_norms(None, None, None, None, 0, 0, 16, f32, None) == 0
    # parameter gradients that are not matrix products
    assert lib.lbi_rmsnorm_weight_grad_workspace_bytes(8192, 768) == 256 * 768 * 4
    assert lib.lbi_rmsnorm_weight_grad_workspace_bytes(10, 768) == 10 * 768 * 4
    assert lib.lbi_rmsnorm_weight_grad(one, one, one, one, 1 << 30, 4, 6, 1e-5, f32, f32, None) == -2
    assert b"multiple of 4" in lib.lbi_last_error()
    assert lib.lbi_rmsnorm_weight_grad(one, one, one, None, 0, 4, 8, 1e-5, f32, f32, None) == -4
    assert lib.lbi_rmsnorm_weight_grad(one, one, one, one, 1 << 30, 4, 8, 1e-5, f32, _lib.LBI_F16, None) == -2
    assert lib.lbi_causal_conv1d_weight_grad_workspace_bytes(8, 1024, 2304, 4) == 8 * 16 * (2304 * 5) * 4
    assert lib.lbi_causal_conv1d_weight_grad(one, one, one, one, 1 << 30, 1, 4, 8, 9, f32, None) == -2
    assert b"above 8" in lib.lbi_last_error()
    assert lib.lbi_causal_conv1d_weight_grad(one, one, one, None, 0, 1, 4, 8, 4, f32, None) == -4
    # attention: short 16-bit sequences at head dim 64 run as one launch and need no workspace
    f16 = _lib.LBI_F16
    assert lib.lbi_attn_pullback_workspace_bytes(8, 8, 128, 64, 4, f16) == 0
    assert lib.lbi_attn_pullback_workspace_bytes(8, 8, 256, 64, 4, f16) == 0
    assert lib.lbi_attn_pullback_workspace_bytes(8, 8, 77, 64, 4, f16) == 0
    assert lib.lbi_attn_pullback_workspace_bytes(8, 8, 128, 128, 4, f16) == 0
    assert lib.lbi_attn_pullback_workspace_bytes(8, 8, 320, 64, 4, f16) == 4 * (64 * 320 + 256 * 320 + 64 * 320 * 64)
    assert lib.lbi_attn_pullback_workspace_bytes(8, 8, 128, 64, 4, f32) > 0
    assert lib.lbi_attn_pullback(one, one, one, one, one, one, one, None, 0, 8, 8, 320, 64, 4, 0.125, 1, f16, None) == -4
    assert b"workspace" in lib.lbi_last_error()
    # the allocation-free entry rejects, on the host, what its static scratch array cannot hold
    assert lib.lbi_attn_pullback_workspace_bytes(4, 16, 4096, 128, 16, _lib.LBI_BF16) > _lib.ATTN_STATIC_SCRATCH_BYTES
    assert lib.lbi_attn_pullback_static(one, one, one, one, one, one, one, 4, 16, 4096, 128, 16, 0.1, 1,
                                        _lib.LBI_BF16, None) == -4
    assert b"static buffer holds" in lib.lbi_last_error()
    assert lib.lbi_attn_pullback_static(None, one, one, one, one, one, one, 1, 1, 320, 64, 1, 0.1, 1, f16, None) == -1
    assert lib.lbi_attn_pullback_static(None, None, None, None, None, None, None, 0, 1, 320, 64, 1, 0.1, 1, f16, None) == 0
    header = HEADER.read_text()
    assert f"#define LBI_ATTN_STATIC_SCRATCH_BYTES ({_lib.ATTN_STATIC_SCRATCH_BYTES >> 20}u << 20)" in header


def test_wrappers_reject_bad_input_before_touching_the_device():
    import torch

    from latent_bounded_interfaces_amd.hip.interface import suffix_scan_pullbacks

    with pytest.raises(ValueError, match=r"\[B, K, R, R\]"):
        suffix_scan_pullbacks(torch.zeros(2, 3, 4))
    with pytest.raises(ValueError, match="square"):
        suffix_scan_pullbacks(torch.zeros(2, 3, 4, 5))
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        suffix_scan_pullbacks(torch.zeros(2, 3, 4, 4))
