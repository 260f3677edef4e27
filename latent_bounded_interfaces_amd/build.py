"""Builds liblbi_hip.so (gfx950 code object + C ABI) in-tree with hipcc.

Usage: ``python -m latent_bounded_interfaces_amd.build`` or ``build_library()``.
hipcc cross-compiles for gfx950 without a GPU present.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "liblbi_hip.so"
SOURCES = ("lbi_common.hip", "lbi_scan.hip", "lbi_attn.hip", "lbi_region.hip", "lbi_norms.hip", "lbi_param_grads.hip")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # Keep the compiler from forming packed-fp32 VALU instructions.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(found):
        raise RuntimeError("hipcc not found; ROCm is required to build liblbi_hip.so")
    return found


def build_library(verbose: bool = False, extra_flags: tuple[str, ...] = ()) -> Path:
    """Compile every kernel source and link the shared library. Always recompiles."""
    hipcc = _hipcc()
    objs = []
    procs = []
    build_dir = PKG_DIR / "build"
    build_dir.mkdir(exist_ok=True)
    for src in SOURCES:
        src_path = CSRC / src
        if not src_path.exists():
            continue
        obj = build_dir / (src_path.stem + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, "-c", str(src_path), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(str(obj))
    for src, proc in procs:
        log, _ = proc.communicate()
        log = "\n".join(line for line in log.splitlines() if "packed-fp32-ops" not in line)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{log}")
        if verbose and log.strip():
            print(log, flush=True)
    tmp = LIB_PATH.with_suffix(".so.tmp")
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", str(tmp)]
    res = subprocess.run(link, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    path = build_library(verbose="-v" in sys.argv)
    print(path)
