"""Timing harness for the attention input-pullback on one GPU.

Counterpart of reference benchmarks/time_attention_pullback.py: warm-up, then the
median and best of ``iters`` device-timed calls (HIP events on the launch stream,
reference :117-138), the same CSV columns (reference :347-360), an optional error
check against a caller-supplied expected result.  ``attention_section`` is what
``bench.py`` embeds: the long-context and the reference benchmark shape with their
roofline figures.
"""
from __future__ import annotations

import argparse
import csv
import json
import math
import statistics
import sys

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
        self.stream = _lib.current_stream_ptr(q.device)

    def __call__(self):
        q, k, v, g = self.args
        st = self.lib.lbi_attn_pullback(q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(),
                                        self.out[0].data_ptr(), self.out[1].data_ptr(), self.out[2].data_ptr(),
                                        self.ws.data_ptr(), self.ws.numel(), self.B, self.H, self.T, self.Dh, self.P,
                                        self.scale, int(self.causal), self.dtype, self.stream)
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


def measure(B, H, T, Dh, P, dtype, *, causal=True, warmup=3, iters=10, device="cuda", expected=None):
    q, k, v, g = make_inputs(B, H, T, Dh, P, dtype, device)
    call = PullbackCall(q, k, v, g, 1.0 / math.sqrt(Dh), causal)
    median_ms, best_ms, mean_ms, peak = time_call(call, warmup=warmup, iters=iters)
    first = tuple(t.clone() for t in call())
    again = call()
    torch.cuda.synchronize()
    stable = all(torch.equal(a, b) for a, b in zip(first, again))
    err = None
    if expected is not None:
        err = max(float((a.float() - b.float().to(a.device)).abs().max()) for a, b in zip(first, expected))
    flops = algorithmic_flops(B, H, T, Dh, P, causal)
    tflops = flops / (mean_ms * 1e-3) / 1e12
    return {
        "B": B, "H": H, "T": T, "Dh": Dh, "P": P, "causal": causal, "dtype": str(dtype).replace("torch.", ""),
        "backend": "hip", "median_ms": median_ms, "best_ms": best_ms, "mean_ms": mean_ms,
        "peak_memory_bytes": peak, "max_abs_error_vs_autograd": err,
        "algorithmic_flops": flops, "tflops": tflops, "bit_stable_rerun": stable,
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_MFMA_16BIT_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / PEAK_MFMA_16BIT_TFLOPS},
    }


def attention_section(steps: int = 5) -> dict:
    """The two attention configurations reported beside the scan headline."""
    out = {}
    out["attn_pullback_bf16_B4_H16_T4096_Dh128_P16"] = measure(4, 16, 4096, 128, 16, torch.bfloat16, iters=steps)
    torch.cuda.empty_cache()
    out["attn_pullback_fp16_B8_H8_T128_Dh64_P4"] = measure(8, 8, 128, 64, 4, torch.float16, iters=max(steps, 20))
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
    args = ap.parse_args(argv)
    rows = []
    for spec in args.shapes:
        B, H, T, Dh, P = (int(x) for x in spec.split(","))
        rows.append(measure(B, H, T, Dh, P, getattr(torch, args.dtype), causal=not args.non_causal,
                            warmup=args.warmup, iters=args.iters))
        print(json.dumps(rows[-1]), flush=True)
    if args.csv:
        with open(args.csv, "w", newline="") as fh:
            writer = csv.DictWriter(fh, fieldnames=CSV_COLUMNS, extrasaction="ignore")
            writer.writeheader()
            writer.writerows(rows)
    if args.json:
        with open(args.json, "w") as fh:
            json.dump(rows, fh, indent=2)
    return 0


if __name__ == "__main__":
    sys.exit(main())
