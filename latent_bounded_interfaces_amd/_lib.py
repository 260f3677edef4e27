"""ctypes binding of liblbi_hip.so (the C ABI declared in include/lbi_hip.h).

The library is built in-tree by ``latent_bounded_interfaces_amd.build``.  There is
no fallback: if it is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes
import threading
from pathlib import Path

import torch

LIB_PATH = Path(__file__).resolve().parent / "liblbi_hip.so"

LBI_F32, LBI_F16, LBI_BF16 = 0, 1, 2
ATTN_STATIC_SCRATCH_BYTES = 32 << 20  # LBI_ATTN_STATIC_SCRATCH_BYTES of include/lbi_hip.h
ABI_VERSION = 9
LBI_SCAN_EXACT_SUFFIX = 1  # lbi_scan_flags of include/lbi_hip.h

_DTYPE_CODES = {torch.float32: LBI_F32, torch.float16: LBI_F16, torch.bfloat16: LBI_BF16}

# name -> (restype, argtypes); must list every symbol of include/lbi_hip.h.
_c = ctypes
SYMBOLS = {
    "lbi_abi_version": (_c.c_int, []),
    "lbi_last_error": (_c.c_char_p, []),
    "lbi_suffix_scan": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int, _c.c_int, _c.c_void_p],
    ),
    "lbi_suffix_scan_with_cotangents": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int, _c.c_int,
         _c.c_void_p],
    ),
    "lbi_suffix_scan_ex": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int, _c.c_int,
         _c.c_int, _c.c_void_p],
    ),
    "lbi_suffix_cotangents": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int, _c.c_void_p],
    ),
    "lbi_suffix_apply": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_void_p],
    ),
    "lbi_attn_pullback_workspace_bytes": (
        _c.c_size_t,
        [_c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int],
    ),
    "lbi_attn_pullback": (
        _c.c_int,
        [_c.c_void_p] * 7 + [_c.c_void_p, _c.c_size_t] + [_c.c_int64] * 5
        + [_c.c_float, _c.c_int, _c.c_int, _c.c_void_p],
    ),
    "lbi_attn_pullback_static": (
        _c.c_int,
        [_c.c_void_p] * 7 + [_c.c_int64] * 5 + [_c.c_float, _c.c_int, _c.c_int, _c.c_void_p],
    ),
    "lbi_rmsnorm_pullback": (
        _c.c_int,
        [_c.c_void_p] * 6 + [_c.c_int64] * 4 + [_c.c_float, _c.c_int, _c.c_int, _c.c_int, _c.c_void_p],
    ),
    "lbi_gated_mlp_pullback": (_c.c_int, [_c.c_void_p] * 3 + [_c.c_int64] * 4 + [_c.c_int, _c.c_int, _c.c_void_p]),
    "lbi_attn_heads_split": (_c.c_int, [_c.c_void_p] * 2 + [_c.c_int64] * 5 + [_c.c_int, _c.c_void_p]),
    "lbi_attn_qkv_pullback": (
        _c.c_int,
        [_c.c_void_p] * 6 + [_c.c_int64] * 6 + [_c.c_int, _c.c_int, _c.c_void_p],
    ),
    "lbi_causal_conv1d_pullback": (_c.c_int, [_c.c_void_p] * 3 + [_c.c_int64] * 4 + [_c.c_int, _c.c_void_p]),
    "lbi_attn_qkv_conv_pullback": (
        _c.c_int,
        [_c.c_void_p] * 7 + [_c.c_int64] * 6 + [_c.c_int, _c.c_int64, _c.c_int, _c.c_void_p],
    ),
    "lbi_matrix_norms_workspace_bytes": (_c.c_size_t, [_c.c_int64, _c.c_int64]),
    "lbi_matrix_norms": (
        _c.c_int,
        [_c.c_void_p] * 4 + [_c.c_size_t, _c.c_int64, _c.c_int64, _c.c_int, _c.c_void_p],
    ),
    "lbi_rmsnorm_weight_grad_workspace_bytes": (_c.c_size_t, [_c.c_int64, _c.c_int64]),
    "lbi_rmsnorm_weight_grad": (
        _c.c_int,
        [_c.c_void_p] * 4 + [_c.c_size_t, _c.c_int64, _c.c_int64, _c.c_float, _c.c_int, _c.c_int, _c.c_void_p],
    ),
    "lbi_causal_conv1d_weight_grad_workspace_bytes": (_c.c_size_t, [_c.c_int64] * 4),
    "lbi_causal_conv1d_weight_grad": (
        _c.c_int,
        [_c.c_void_p] * 4 + [_c.c_size_t] + [_c.c_int64] * 4 + [_c.c_int, _c.c_void_p],
    ),
}


class LbiLibraryError(RuntimeError):
    """liblbi_hip.so is missing, stale, or a native call reported a failure."""


_lock = threading.Lock()
_handle = None


def load() -> ctypes.CDLL:
    """Load the shared library once and type every exported entry point."""
    global _handle
    if _handle is not None:
        return _handle
    with _lock:
        if _handle is not None:
            return _handle
        if not LIB_PATH.exists():
            raise LbiLibraryError(
                f"{LIB_PATH} not found: build it with `python -m latent_bounded_interfaces_amd.build` "
                "(hipcc, gfx950). This package has no non-HIP execution path."
            )
        try:
            lib = ctypes.CDLL(str(LIB_PATH))
        except OSError as exc:  # unresolved HIP runtime, wrong arch ...
            raise LbiLibraryError(f"cannot load {LIB_PATH}: {exc}") from exc
        for name, (restype, argtypes) in SYMBOLS.items():
            try:
                fn = getattr(lib, name)
            except AttributeError as exc:
                raise LbiLibraryError(f"{LIB_PATH} does not export {name}; rebuild it") from exc
            fn.restype = restype
            fn.argtypes = argtypes
        if lib.lbi_abi_version() != ABI_VERSION:
            raise LbiLibraryError(
                f"{LIB_PATH} has ABI {lib.lbi_abi_version()}, this package expects {ABI_VERSION}; rebuild it"
            )
        _handle = lib
        return lib


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODES[dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {dtype}; expected float32, float16 or bfloat16") from None


def check(status: int, what: str) -> None:
    """Turn a negative lbi_status into a RuntimeError carrying the native message."""
    if status != 0:
        message = load().lbi_last_error().decode("utf-8", "replace")
        raise LbiLibraryError(f"{what} failed (status {status}): {message}")


def current_stream_ptr(device: torch.device) -> int:
    return int(torch.cuda.current_stream(device).cuda_stream)
