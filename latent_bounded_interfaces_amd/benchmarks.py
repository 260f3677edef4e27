"""Timing harness for the attention input-pullback and the region input pullback on one GPU.

Counterpart of reference benchmarks/time_attention_pullback.py: warm-up, then the
median and best of ``iters`` device-timed calls (HIP events on the launch stream,
reference :117-138), the same CSV columns (reference :347-360), and its ``--check``
(:230, :300-305): the result compared with one SDPA forward + autograd backward per
direction, in fp32 on the device, on a bounded sample of (batch, head) pairs and
directions.  ``attention_section`` is what ``bench.py`` embeds: the long-context and the
reference benchmark shape with their roofline figures.  ``--pmc-traffic`` turns two
``rocprofv3 --pmc`` counter dumps into the small JSON ``bench.py`` reads its HBM traffic
figure from.
"""
from __future__ import annotations

import argparse
import csv
import hashlib
import json
import math
import statistics
import sys
from pathlib import Path

import torch

from . import _lib

PEAK_MFMA_16BIT_TFLOPS = 2500.0  # MI355X dense bf16 / fp16 matrix peak
CSV_COLUMNS = ["B", "H", "T", "Dh", "P", "causal", "dtype", "backend", "median_ms", "best_ms",
               "peak_memory_bytes", "max_abs_error_vs_autograd"]


def algorithmic_flops(B: int, H: int, T: int, Dh: int, P: int, causal: bool) -> float:
    """One shared Q K^T plus dP, dV, dQ, dK per direction; recomputation is not counted."""
    pairs = T * (T + 1) / 2 if causal else T * T
    return B * H * pairs * 2 * Dh * (1 + 4 * P)


def algorithmic_bytes(B: int, H: int, T: int, Dh: int, P: int, elem: int) -> float:
    return B * H * T * Dh * elem * (3 + P + 3 * P)


def make_inputs(B, H, T, Dh, P, dtype, device, seed=0):
    gen = torch.Generator(device="cpu").manual_seed(seed)
    out = []
    for shape in ((B, H, T, Dh),) * 3 + ((B, P, H, T, Dh),):
        # generate per (b) slice to bound host memory, then move
        out.append(torch.randn(shape, generator=gen, dtype=torch.float32).to(dtype).to(device))
    return out


class PullbackCall:
    """Pre-allocated outputs and workspace so the timed region holds only the kernels."""

    def __init__(self, q, k, v, g, scale: float, causal: bool):
        self.lib = _lib.load()
        self.args = (q, k, v, g)
        self.B, self.H, self.T, self.Dh = q.shape
        self.P = g.shape[1]
        self.scale, self.causal = float(scale), bool(causal)
        self.dtype = _lib.dtype_code(q.dtype)
        self.out = tuple(torch.empty_like(g) for _ in range(3))
        need = int(self.lib.lbi_attn_pullback_workspace_bytes(self.B, self.H, self.T, self.Dh, self.P, self.dtype))
        self.ws = torch.empty(max(need, 256), device=q.device, dtype=torch.uint8)
        self.device = q.device

    def __call__(self):
        q, k, v, g = self.args
        st = self.lib.lbi_attn_pullback(q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(),
                                        self.out[0].data_ptr(), self.out[1].data_ptr(), self.out[2].data_ptr(),
                                        self.ws.data_ptr(), self.ws.numel(), self.B, self.H, self.T, self.Dh, self.P,
                                        self.scale, int(self.causal), self.dtype,
                                        _lib.current_stream_ptr(self.device))
        _lib.check(st, "lbi_attn_pullback")
        return self.out


def time_call(fn, *, warmup: int, iters: int):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    peak = 0
    for _ in range(iters):
        torch.cuda.reset_peak_memory_stats()
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        stop.record()
        torch.cuda.synchronize()
        times.append(float(start.elapsed_time(stop)))
        peak = max(peak, int(torch.cuda.max_memory_allocated()))
    return statistics.median(times), min(times), statistics.fmean(times), peak


def check_against_autograd(outputs, q, k, v, g, scale: float, causal: bool, *, pairs: int = 2, directions: int = 2):
    """What the reference benchmark's ``--check`` computes (benchmarks/time_attention_pullback.py:300-305): the
    largest absolute difference to per-direction SDPA + autograd, here in fp32 on the device and on a bounded
    sample: the first and last ``pairs`` (batch, head) pairs and the first and last ``directions`` directions (all of
    them when the call is small).  Returns ``(max_abs_error, max_abs_error / max|expected|, sample description)``."""
    B, H, T, Dh = q.shape
    P = g.shape[1]
    flat = list(range(B * H))
    picked = sorted(set(flat[:pairs] + flat[-pairs:]))
    dirs = sorted(set(list(range(P))[:directions] + list(range(P))[-directions:]))
    worst, largest = 0.0, 0.0
    for bh in picked:
        b, h = divmod(bh, H)
        qs, ks, vs = (t[b:b + 1, h:h + 1].float().detach().requires_grad_(True) for t in (q, k, v))
        with torch.enable_grad():
            out = torch.nn.functional.scaled_dot_product_attention(qs, ks, vs, is_causal=causal, scale=scale)
            for p in dirs:
                want = torch.autograd.grad(out, (qs, ks, vs), grad_outputs=g[b:b + 1, p, h:h + 1].float(),
                                           retain_graph=True)
                for got, ref in zip(outputs, want):
                    worst = max(worst, float((got[b, p, h].float() - ref[0, 0]).abs().max()))
                    largest = max(largest, float(ref.abs().max()))
    sample = f"{len(picked)} of {B * H} (batch, head) pairs x {len(dirs)} of {P} directions, fp32 SDPA + autograd on the device"
    return worst, worst / max(largest, 1e-30), sample


def measure(B, H, T, Dh, P, dtype, *, causal=True, warmup=3, iters=10, device="cuda", check=False):
    q, k, v, g = make_inputs(B, H, T, Dh, P, dtype, device)
    call = PullbackCall(q, k, v, g, 1.0 / math.sqrt(Dh), causal)
    median_ms, best_ms, mean_ms, peak = time_call(call, warmup=warmup, iters=iters)
    first = tuple(t.clone() for t in call())
    again = call()
    torch.cuda.synchronize()
    stable = all(torch.equal(a, b) for a, b in zip(first, again))
    err = rel_err = sample = None
    if check:
        err, rel_err, sample = check_against_autograd(first, q, k, v, g, 1.0 / math.sqrt(Dh), causal)
    flops = algorithmic_flops(B, H, T, Dh, P, causal)
    tflops = flops / (mean_ms * 1e-3) / 1e12
    return {
        "B": B, "H": H, "T": T, "Dh": Dh, "P": P, "causal": causal, "dtype": str(dtype).replace("torch.", ""),
        "backend": "hip", "median_ms": median_ms, "best_ms": best_ms, "mean_ms": mean_ms,
        "peak_memory_bytes": peak, "max_abs_error_vs_autograd": err, "max_rel_error_vs_autograd": rel_err,
        "check_sample": sample, "algorithmic_flops": flops, "tflops": tflops, "bit_stable_rerun": stable,
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_MFMA_16BIT_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / PEAK_MFMA_16BIT_TFLOPS},
    }


def attention_section(steps: int = 5) -> dict:
    """The two attention configurations reported beside the scan headline, each checked against autograd."""
    out = {}
    out["attn_pullback_bf16_B4_H16_T4096_Dh128_P16"] = measure(4, 16, 4096, 128, 16, torch.bfloat16, iters=steps,
                                                               check=True)
    torch.cuda.empty_cache()
    out["attn_pullback_fp16_B8_H8_T128_Dh64_P4"] = measure(8, 8, 128, 64, 4, torch.float16, iters=max(steps, 20),
                                                           check=True)
    return out


# ---------------------------------------------------------------------------------------
# HBM traffic of a kernel from rocprofv3 counter dumps
# ---------------------------------------------------------------------------------------
PACKAGE_DIR = Path(__file__).resolve().parent


def source_digest(files) -> str:
    """sha256 over the named kernel sources (paths relative to the package), the tie between a measured
    counter figure and the code it was measured on."""
    h = hashlib.sha256()
    for name in sorted(files):
        h.update(name.encode())
        h.update((PACKAGE_DIR / name).read_bytes())
    return h.hexdigest()


def _per_dispatch(csv_path: Path, counter: str, kernel_substring: str, *, first_only: bool = False) -> tuple[float, int]:
    rows = []
    with open(csv_path, newline="") as fh:
        for row in csv.DictReader(fh):
            if row["Counter_Name"] == counter and kernel_substring in row["Kernel_Name"]:
                rows.append((int(row["Dispatch_Id"]), float(row["Counter_Value"])))
    if not rows:
        raise SystemExit(f"{csv_path}: no {counter} rows for a kernel containing {kernel_substring!r}")
    rows.sort()
    values = [v for _, v in rows[:1]] if first_only else [v for _, v in rows]
    return statistics.fmean(values), len(values)


def pmc_traffic(fetch_dir: str, write_dir: str, *, kernel: str, copy_kernel: str, copy_bytes: int, sources) -> dict:
    """HBM bytes per dispatch of ``kernel`` from two ``rocprofv3 --pmc`` runs (FETCH_SIZE, then WRITE_SIZE, KiB per
    dispatch), each counter scaled by what it reads for a plain device copy of ``copy_bytes`` in the same run: the
    FIRST dispatch of ``copy_kernel``, which is where ``bench.py --copy-calibration`` puts it."""
    def one(directory, counter):
        path = next(Path(directory).rglob("*counter_collection.csv"))
        value, calls = _per_dispatch(path, counter, kernel)
        copy_value, _ = _per_dispatch(path, counter, copy_kernel, first_only=True)
        return value, calls, copy_value

    fetch, calls, copy_fetch = one(fetch_dir, "FETCH_SIZE")
    write, _, copy_write = one(write_dir, "WRITE_SIZE")
    fetch_scale = (copy_bytes / 1024.0) / copy_fetch
    write_scale = (copy_bytes / 1024.0) / copy_write
    return {
        "kernel": kernel, "dispatches_averaged": calls,
        "fetch_size_kib": fetch, "write_size_kib": write,
        "copy_kernel": copy_kernel, "copy_bytes": copy_bytes,
        "copy_fetch_size_kib": copy_fetch, "copy_write_size_kib": copy_write,
        "fetch_scale": fetch_scale, "write_scale": write_scale,
        "traffic_bytes": int((fetch * fetch_scale + write * write_scale) * 1024),
        "sources": sorted(sources), "source_sha256": source_digest(sources),
    }


def load_traffic(json_path, kernel_substring: str):
    """The measured traffic figure, or None when the file is missing, names another kernel, or the kernel sources
    have changed since it was measured (the figure would describe code that no longer exists)."""
    try:
        record = json.loads(Path(json_path).read_text())
        if kernel_substring not in record["kernel"] and record["kernel"] not in kernel_substring:
            return None
        if source_digest(record["sources"]) != record["source_sha256"]:
            return None
        return int(record["traffic_bytes"])
    except (OSError, KeyError, ValueError):
        return None


# ---------------------------------------------------------------------------------------
# Region-level input pullback (a range of Transformer layers, P cotangent directions)
# ---------------------------------------------------------------------------------------
class _Holder(torch.nn.Module):
    """Parameter container with the attribute layout of the reference's Transformer block
    (no forward: the benchmarks feed synthetic caches)."""


def synthetic_region(*, dim, n_heads, n_kv_heads, head_dim, hidden, layers, d_conv, batch, seq_len, dtype, device,
                     residual_in_fp32=True, seed=0):
    """Random weights and a random forward cache with the attribute names of the reference's
    ``TransformerRegionBackend`` / ``TransformerRegionCache`` (the fields the pullbacks read).
    Values are synthetic (N(0,1) activations, N(0,1/fan_in) weights); shapes and dtypes are the real ones."""
    from types import SimpleNamespace as NS

    gen = torch.Generator(device="cpu").manual_seed(seed)

    def rand(*shape, std=1.0, dt=dtype):
        return (torch.randn(*shape, generator=gen) * std).to(dt).to(device)

    def linear(out_features, in_features):
        mod = torch.nn.Linear(in_features, out_features, bias=False, device=device, dtype=dtype)
        with torch.no_grad():
            mod.weight.copy_(rand(out_features, in_features, std=in_features ** -0.5))
        return mod

    def norm():
        mod = _Holder()
        mod.weight = torch.nn.Parameter(rand(dim) * 0.1 + 1)
        mod.eps = 1e-5
        return mod

    res_dtype = torch.float32 if residual_in_fp32 else dtype
    qkv_dim = (n_heads + 2 * n_kv_heads) * head_dim
    blocks, caches = [], []
    for layer in range(layers):
        attn = _Holder()
        attn.n_heads, attn.n_kv_heads, attn.head_dim = n_heads, n_kv_heads, head_dim
        attn.rope_base, attn.rope_interleaved, attn.softmax_scale, attn.d_conv = 10000.0, False, None, d_conv
        attn.in_proj = linear(qkv_dim, dim)
        attn.out_proj = linear(dim, n_heads * head_dim)
        if d_conv > 0:
            attn.conv1d = _Holder()
            attn.conv1d.weight = torch.nn.Parameter(rand(qkv_dim, 1, d_conv, std=d_conv ** -0.5))
            attn.conv1d.bias = None
        mlp = _Holder()
        mlp.fc1 = linear(2 * hidden, dim)
        mlp.fc2 = linear(dim, hidden)
        block = _Holder()
        block.attn, block.mlp, block.norm, block.norm2 = attn, mlp, norm(), norm()
        block.residual_in_fp32 = residual_in_fp32
        blocks.append(block)
        a_cache = NS(norm_input=rand(batch, seq_len, dim, dt=res_dtype if layer else dtype),
                     norm_output=rand(batch, seq_len, dim),
                     q_rope=rand(batch, n_heads, seq_len, head_dim), k_expanded=rand(batch, n_heads, seq_len, head_dim),
                     v_expanded=rand(batch, n_heads, seq_len, head_dim),
                     out_proj_input=rand(batch, seq_len, n_heads * head_dim))
        m_cache = NS(norm_input=rand(batch, seq_len, dim, dt=res_dtype), norm_output=rand(batch, seq_len, dim),
                     fc1_output=rand(batch, seq_len, 2 * hidden), down_input=rand(batch, seq_len, hidden))
        caches.append(NS(layer_index=layer, attention=a_cache, mlp=m_cache))
    backend = _Holder()
    backend.backbone = _Holder()
    backend.backbone.blocks = torch.nn.ModuleList(blocks)
    cache = NS(region_index=0, layer_range=(0, layers), layer_caches=caches,
               region_input=rand(batch, seq_len, dim))
    return backend, cache


def region_flops(*, dim, n_heads, n_kv_heads, head_dim, hidden, layers, batch, seq_len, basis) -> dict:
    """Algorithmic flops of the region input pullback: the four transposed projections per
    layer on B*P*T cotangent rows, plus the attention pullback."""
    rows = batch * basis * seq_len
    qkv_dim = (n_heads + 2 * n_kv_heads) * head_dim
    gemm = 2.0 * rows * (dim * hidden + 2 * hidden * dim + dim * n_heads * head_dim + qkv_dim * dim) * layers
    attn = algorithmic_flops(batch, n_heads, seq_len, head_dim, basis, True) * layers
    return {"gemm": gemm, "attention": attn, "total": gemm + attn}


def measure_region(*, dim=768, n_heads=12, n_kv_heads=12, head_dim=64, hidden=3072, layers=2, d_conv=4, batch=8,
                   seq_len=1024, basis=64, dtype=torch.bfloat16, warmup=2, iters=5, device="cuda") -> dict:
    from .backends import HipTransformerLowering

    backend, cache = synthetic_region(dim=dim, n_heads=n_heads, n_kv_heads=n_kv_heads, head_dim=head_dim, hidden=hidden,
                                      layers=layers, d_conv=d_conv, batch=batch, seq_len=seq_len, dtype=dtype,
                                      device=device)
    gen = torch.Generator(device="cpu").manual_seed(1)
    cot = torch.randn(batch, basis, seq_len, dim, generator=gen).to(device)
    lowering = HipTransformerLowering()

    def call():
        return lowering.input_pullback_basis(backend=backend, cache=cache, output_cotangent_basis=cot)

    median_ms, best_ms, mean_ms, peak = time_call(call, warmup=warmup, iters=iters)
    first = call().clone()
    stable = bool(torch.equal(first, call()))
    flops = region_flops(dim=dim, n_heads=n_heads, n_kv_heads=n_kv_heads, head_dim=head_dim, hidden=hidden, layers=layers,
                         batch=batch, seq_len=seq_len, basis=basis)
    tflops = flops["total"] / (mean_ms * 1e-3) / 1e12
    return {
        "workload": f"region input pullback: {layers} layers, d_model {dim}, {n_heads} heads x {head_dim}, "
                    f"hidden {hidden}, conv {d_conv}, B={batch} T={seq_len} P={basis}, {str(dtype).replace('torch.', '')}",
        "median_ms": median_ms, "best_ms": best_ms, "mean_ms": mean_ms, "peak_memory_bytes": peak,
        "algorithmic_flops": flops, "tflops": tflops, "bit_stable_rerun": stable,
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_MFMA_16BIT_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / PEAK_MFMA_16BIT_TFLOPS},
    }


def region_section(steps: int = 5) -> dict:
    """One region of the end-to-end configuration (2 of 12 layers, d_model 768, 12 heads, interface width 64
    = 64 cotangent directions, batch 8, sequence 1024, bf16)."""
    return {"region_input_pullback_bf16_L2_D768_B8_T1024_P64": measure_region(iters=steps)}


def measure_lbi_step(*, regions=6, layers_per_region=2, dim=768, n_heads=12, head_dim=64, hidden=3072, d_conv=4,
                     batch=8, seq_len=1024, interface_width=64, dtype=torch.bfloat16, warmup=1, iters=3,
                     device="cuda") -> dict:
    """Device work of one LBI scan backward step at the end-to-end configuration (12 layers in 6
    regions of 2, interface width 64): the state-Jacobian build (region input pullback for 64
    directions) of every region but the last, whose Jacobian the step leaves out (the reference
    builds all six and drops the last), the parameter VJP of every region, and the interface suffix scan
    (cotangent chain over the 5 inner Jacobians).  The region-output cotangents are constant over positions
    (mean-pooling interface).  The forward caches are synthetic and shared by the six regions
    (same shapes); the interface's own small MLP pullbacks and the readout/canvas VJPs are not part
    of this library and are left out."""
    from .backends import HipTransformerLowering
    from .hip.interface import suffix_scan_cotangents

    backend, cache = synthetic_region(dim=dim, n_heads=n_heads, n_kv_heads=n_heads, head_dim=head_dim, hidden=hidden,
                                      layers=layers_per_region, d_conv=d_conv, batch=batch, seq_len=seq_len,
                                      dtype=dtype, device=device)
    gen = torch.Generator(device="cpu").manual_seed(2)
    # what the structured provider hands over for a mean-pooling interface: one cotangent per direction,
    # the same at every position, as a stride-0 view
    basis = (torch.randn(batch, interface_width, 1, dim, generator=gen) / seq_len).to(device).expand(-1, -1, seq_len, -1)
    cot = torch.randn(batch, seq_len, dim, generator=gen).to(device)
    jts = (torch.eye(interface_width) + 0.05 * torch.randn(batch, regions - 1, interface_width, interface_width,
                                                          generator=gen)).to(device)
    g_state = torch.randn(batch, interface_width, generator=gen).to(device)
    lowering = HipTransformerLowering()
    parts = {}

    def pullbacks():
        for _ in range(regions - 1):
            lowering.input_pullback_basis(backend=backend, cache=cache, output_cotangent_basis=basis)

    def vjps():
        for _ in range(regions):
            lowering.parameter_vjp(backend=backend, cache=cache, output_cotangent=cot)

    def scan():
        suffix_scan_cotangents(jts, g_state)

    def whole():
        pullbacks()
        scan()
        vjps()

    for name, fn in (("state_jacobian_pullbacks", pullbacks), ("parameter_vjps", vjps), ("interface_scan", scan),
                     ("step", whole)):
        median_ms, best_ms, mean_ms, peak = time_call(fn, warmup=warmup, iters=iters)
        parts[name] = {"median_ms": median_ms, "best_ms": best_ms, "peak_memory_bytes": peak}
    return {
        "state_jacobians_built": regions - 1,
        "workload": f"LBI scan backward step, device work: {regions} regions x {layers_per_region} layers, d_model {dim}, "
                    f"{n_heads} heads x {head_dim}, hidden {hidden}, interface width {interface_width}, B={batch} "
                    f"T={seq_len}, {str(dtype).replace('torch.', '')}, synthetic caches",
        **parts,
    }


def lbi_step_section(steps: int = 3) -> dict:
    return {"lbi_backward_step_bf16_L12_D768_B8_T1024_d64": measure_lbi_step(iters=steps)}


def measure_scan(B: int, K: int, d: int, dtype, *, warmup=3, iters=10, device="cuda", matrices_only=False) -> dict:
    """One suffix scan of near-identity matrices, as the scan benchmark feeds it: all K suffix matrices and all K
    cotangents in one call, or (``matrices_only``) the matrices alone; rates on the algorithmic flops and bytes."""
    lib = _lib.load()
    gen = torch.Generator(device="cpu").manual_seed(0)
    mats = torch.eye(d).expand(B, K, d, d) + torch.randn(B, K, d, d, generator=gen) * (0.01 / d) ** 0.5
    mats = mats.to(dtype).to(device)
    g = torch.randn(B, d, generator=gen).to(device)
    out = torch.empty(B, K + 1, d, d, device=device)
    cot = torch.empty(B, K + 1, d, device=device)

    def call():
        if matrices_only:
            _lib.check(lib.lbi_suffix_scan(mats.data_ptr(), out.data_ptr(), B, K, d, _lib.dtype_code(mats.dtype),
                                           _lib.LBI_F32, _lib.current_stream_ptr(mats.device)), "lbi_suffix_scan")
            return
        _lib.check(lib.lbi_suffix_scan_with_cotangents(mats.data_ptr(), g.data_ptr(), out.data_ptr(), cot.data_ptr(), B,
                                                       K, d, _lib.dtype_code(mats.dtype), _lib.LBI_F32,
                                                       _lib.current_stream_ptr(mats.device)),
                   "lbi_suffix_scan_with_cotangents")

    median_ms, best_ms, mean_ms, peak = time_call(call, warmup=warmup, iters=iters)
    flops = B * (K - 1) * 2.0 * d ** 3
    nbytes = B * K * d * d * (mats.element_size() + 4.0)
    return {"B": B, "K": K, "d": d, "dtype": str(dtype).replace("torch.", ""), "matrices_only": matrices_only,
            "median_ms": median_ms, "best_ms": best_ms,
            "pullbacks_per_s": B * K / (median_ms * 1e-3), "tflops": flops / (median_ms * 1e-3) / 1e12,
            "algorithmic_gbs": nbytes / (median_ms * 1e-3) / 1e9, "algorithmic_bytes": nbytes}


def measure_cotangent_chain(B: int, K: int, d: int, dtype, *, warmup=2, iters=10, device="cuda") -> dict:
    """The cotangent-only chain (``lbi_suffix_cotangents``): one pass over the matrices, no d x d product; the
    rate is quoted on the bytes of the matrices, which is all it has to move."""
    lib = _lib.load()
    gen = torch.Generator(device=device).manual_seed(0)
    mats = torch.randn(B, K, d, d, device=device, generator=gen).mul_((0.01 / d) ** 0.5)
    mats.diagonal(dim1=-2, dim2=-1).add_(1.0)
    mats = mats.to(dtype)
    g = torch.randn(B, d, device=device, generator=gen)
    out = torch.empty(B, K + 1, d, device=device)

    def call():
        _lib.check(lib.lbi_suffix_cotangents(mats.data_ptr(), g.data_ptr(), out.data_ptr(), B, K, d,
                                             _lib.dtype_code(mats.dtype), _lib.current_stream_ptr(mats.device)),
                   "lbi_suffix_cotangents")

    median_ms, best_ms, mean_ms, _ = time_call(call, warmup=warmup, iters=iters)
    nbytes = float(mats.numel() * mats.element_size())
    gbs = nbytes / (mean_ms * 1e-3) / 1e9
    return {"B": B, "K": K, "d": d, "dtype": str(dtype).replace("torch.", ""), "kernel_ms_avg": mean_ms,
            "best_ms": best_ms, "pullbacks_per_s": B * K / (mean_ms * 1e-3),
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": 8000.0, "unit": "GB/s", "frac": gbs / 8000.0}}


def scan_section(steps: int = 10) -> dict:
    """Scan variants beside the headline: the cotangent-only chain at a batch that gives every CU a batch element
    (one workgroup runs one chain), and the K-parallel form of the scan at the batch sizes the reference's own
    tests and paper launcher use (one to a few elements)."""
    out = {}
    for dtype, tag in ((torch.float32, "fp32"), (torch.bfloat16, "bf16")):
        out[f"scan_cotangent_only_{tag}_B256"] = measure_cotangent_chain(256, 128, 256, dtype, iters=steps)
        torch.cuda.empty_cache()
    for batch in (1, 8):
        row = measure_scan(batch, 128, 256, torch.float32, iters=steps)
        row["roofline"] = {"bound": "mfma", "achieved": row["tflops"], "peak": 157.3, "unit": "TFLOP/s",
                           "frac": row["tflops"] / 157.3}
        out[f"scan_kparallel_fp32_B{batch}_K128_d256"] = row
    return out


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--shapes", nargs="*", default=["1,8,128,64,4"], help="B,H,T,Dh,P tuples")
    ap.add_argument("--dtype", default="float16", choices=["float16", "bfloat16", "float32"])
    ap.add_argument("--non-causal", action="store_true")
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--csv", default=None)
    ap.add_argument("--json", default=None)
    ap.add_argument("--region", action="store_true",
                    help="time the region-level input pullback at the end-to-end configuration instead")
    ap.add_argument("--basis", type=int, default=64, help="cotangent directions of the --region run")
    ap.add_argument("--lbi-step", action="store_true",
                    help="time the device work of one LBI scan backward step at the end-to-end configuration")
    ap.add_argument("--check", action="store_true",
                    help="compare with per-direction SDPA + autograd (fp32, on the device, bounded sample) and fail "
                         "when the largest error exceeds --check-tol")
    ap.add_argument("--check-tol", type=float, default=None,
                    help="bound on max|error| / max|expected| (default 2e-5 for float32, 2e-2 for 16-bit storage)")
    ap.add_argument("--pmc-traffic", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"), default=None,
                    help="write the HBM-traffic JSON of --kernel from two rocprofv3 --pmc output folders")
    ap.add_argument("--kernel", default="scan_mfma_kernel<float, 256, 32, 64, true, 0>")
    ap.add_argument("--copy-kernel", default="__amd_rocclr_copyBuffer")
    ap.add_argument("--copy-bytes", type=int, default=1 << 30)
    ap.add_argument("--sources", nargs="*", default=["csrc/lbi_scan.hip", "csrc/lbi_common.h"])
    ap.add_argument("--out", default=None, help="--pmc-traffic: where to write the JSON (default: stdout)")
    ap.add_argument("--scan", nargs="*", default=None, help="time the fused suffix scan instead: B,K,d tuples")
    ap.add_argument("--matrices-only", action="store_true", help="--scan: the suffix matrices without the cotangents")
    ap.add_argument("--cotangent-chain", nargs="*", default=None,
                    help="time the cotangent-only chain (lbi_suffix_cotangents) instead: B,K,d tuples")
    args = ap.parse_args(argv)
    if args.pmc_traffic is not None:
        record = pmc_traffic(*args.pmc_traffic, kernel=args.kernel, copy_kernel=args.copy_kernel,
                             copy_bytes=args.copy_bytes, sources=args.sources)
        text = json.dumps(record, indent=2) + "\n"
        if args.out:
            Path(args.out).write_text(text)
        else:
            sys.stdout.write(text)
        return 0
    if args.cotangent_chain is not None:
        for spec in args.cotangent_chain:
            B, K, d = (int(x) for x in spec.split(","))
            print(json.dumps(measure_cotangent_chain(B, K, d, getattr(torch, args.dtype), warmup=args.warmup,
                                                     iters=args.iters)), flush=True)
        return 0
    if args.scan is not None:
        for spec in args.scan:
            B, K, d = (int(x) for x in spec.split(","))
            print(json.dumps(measure_scan(B, K, d, getattr(torch, args.dtype), warmup=args.warmup, iters=args.iters,
                                          matrices_only=args.matrices_only)), flush=True)
        return 0
    if args.lbi_step:
        print(json.dumps(measure_lbi_step(dtype=getattr(torch, args.dtype), warmup=args.warmup, iters=args.iters)),
              flush=True)
        return 0
    if args.region:
        print(json.dumps(measure_region(basis=args.basis, dtype=getattr(torch, args.dtype), warmup=args.warmup,
                                        iters=args.iters)), flush=True)
        return 0
    rows = []
    failed = False
    tol = args.check_tol if args.check_tol is not None else (2e-5 if args.dtype == "float32" else 2e-2)
    for spec in args.shapes:
        B, H, T, Dh, P = (int(x) for x in spec.split(","))
        rows.append(measure(B, H, T, Dh, P, getattr(torch, args.dtype), causal=not args.non_causal,
                            warmup=args.warmup, iters=args.iters, check=args.check))
        print(json.dumps(rows[-1]), flush=True)
        if args.check and rows[-1]["max_rel_error_vs_autograd"] > tol:
            print(f"check failed for {spec}: {rows[-1]['max_rel_error_vs_autograd']:.3e} > {tol:.1e}", file=sys.stderr)
            failed = True
    if args.csv:
        with open(args.csv, "w", newline="") as fh:
            writer = csv.DictWriter(fh, fieldnames=CSV_COLUMNS, extrasaction="ignore")
            writer.writeheader()
            writer.writerows(rows)
    if args.json:
        with open(args.json, "w") as fh:
            json.dump(rows, fh, indent=2)
    return 1 if failed else 0


if __name__ == "__main__":
    sys.exit(main())
