#!/usr/bin/env python3
"""Benchmark of the LBI bounded-interface backward hot path on one MI355X.

One "step" is one pass of the interface suffix scan at the scale configuration
(B=64 batch elements, K=128 regions, d=256 interface width, fp32): all K suffix
matrices plus all K suffix cotangents, computed by one call of
``lbi_suffix_scan_with_cotangents``, inputs resident in HBM.  ``value`` is composed
pullbacks per second, ``B*K / t_step``.

Prints ONE JSON line.  Besides the contract keys it carries

* ``roofline``      - the dominant kernel (the d x d suffix-product kernel) against the
                      MI355X fp32-MFMA peak, from HIP-event timing of that kernel alone;
* ``cpu_baseline``  - the reference's CPU algorithm (log-depth torch scan) timed on the
                      host cores of the same box on a bounded batch slice;
* ``extra``         - the other measured variants (bf16 storage, cotangent-only chain,
                      attention input-pullback, region-level input pullback, the end-to-end LBI
                      backward step on a real forward cache) with their own roofline figures; the
                      attention and end-to-end entries carry a ``cpu_baseline`` of their own (the
                      reference's per-direction SDPA + autograd loop, resp. dense fp32
                      ``loss.backward()``, on a bounded sample).
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

PEAK_FP32_MFMA_TFLOPS = 157.3   # MI355X dense fp32 matrix peak
PEAK_BF16_MFMA_TFLOPS = 2500.0  # MI355X dense bf16/fp16 matrix peak
PEAK_HBM_GBS = 8000.0           # MI355X HBM3E peak

SCAN_B, SCAN_K, SCAN_D = 64, 128, 256

# HBM bytes per launch of the scan kernel at this shape come from a small JSON beside the counter summary in
# profiles/ (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE, KiB per dispatch, each scaled by the same counter's
# reading for a 1 GiB device copy).  The file names the kernel and carries a hash of the kernel's sources; when
# either no longer matches, the line reports "traffic": null rather than a figure measured on other code.
SCAN_KERNEL = "scan_mfma_kernel<float, 256, 32, 64, true, 0>"
SCAN_TRAFFIC_JSON = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles",
                                 "scan_fp32_B64_K128_d256_pmc.json")


def _parse() -> argparse.Namespace:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20,
                    help="untimed steps first: the part needs ~40 ms of load before its clock and the first-touch "
                         "cost of the 2 GiB result settle")
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-side baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="only the headline scan (used for profiling)")
    ap.add_argument("--cpu-sample-batch", type=int, default=64)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy (a known-size reference for scaling the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    return ap.parse_args()


def _time_events(fn, steps: int, warmup: int):
    """Per-call milliseconds from HIP events on the current torch stream (which is
    the stream every kernel of this library is launched on)."""
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(steps):
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        stop.record()
        stop.synchronize()
        times.append(float(start.elapsed_time(stop)))
    return times


def _scan_inputs(device, dtype):
    import torch

    gen = torch.Generator(device="cpu").manual_seed(0)
    noise = torch.randn(SCAN_B, SCAN_K, SCAN_D, SCAN_D, generator=gen, dtype=torch.float32)
    mats = torch.eye(SCAN_D, dtype=torch.float32) + noise * (0.01 / SCAN_D) ** 0.5
    g = torch.randn(SCAN_B, SCAN_D, generator=gen, dtype=torch.float32)
    return mats.to(dtype).to(device), g.to(device)


def _cpu_baseline(sample_batch: int) -> dict:
    """The reference's CPU path (log-depth torch scan) on `sample_batch` batch elements."""
    import torch

    from oracle import scan as oscan

    mats, g = oscan.make_scan_inputs(sample_batch, SCAN_K, SCAN_D, kind="near_identity", seed=0)
    oscan.suffix_scan_levels(mats[:1, :8])  # warm the BLAS threads
    t0 = time.perf_counter()
    suffix = oscan.suffix_scan_levels(mats)
    oscan.suffix_cotangents_from_matrices(suffix[:, :SCAN_K], g)
    dt = time.perf_counter() - t0
    return {
        "value": sample_batch * SCAN_K / dt,
        "unit": "composed_pullbacks/s",
        "cores": int(torch.get_num_threads()),
        "kind": "port",
        "sample": f"B={sample_batch} of {SCAN_B} batch elements, K={SCAN_K}, d={SCAN_D}, fp32, "
                  f"log-depth torch scan + mat-vecs, {dt:.2f} s wall",
    }


def _cpu_attention_baselines() -> dict:
    """The reference's CPU path for the attention pullback (one SDPA forward + autograd backward per direction,
    fp32) on bounded samples of the two attention workloads; rates in algorithmic TFLOP/s."""
    import math
    import statistics as st

    import torch

    from oracle import attention as oattn

    def flops(b, h, t, dh, p):
        return b * h * (t * (t + 1) / 2) * 2 * dh * (1 + 4 * p)

    cores = int(torch.get_num_threads())
    out = {}
    # long-context workload: 4 of its 64 (batch, head) pairs, all 16 directions
    q, k, v, g = oattn.make_attention_inputs(1, 4, 4096, 128, 16, dtype=torch.float32, seed=0)
    t0 = time.perf_counter()
    oattn.attention_pullback_sdpa_loop(q, k, v, g, softmax_scale=128 ** -0.5, causal=True)
    dt = time.perf_counter() - t0
    out["attn_pullback_bf16_B4_H16_T4096_Dh128_P16"] = {
        "value": flops(1, 4, 4096, 128, 16) / dt / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "sample": f"4 of the 64 (batch, head) pairs, all 16 directions, fp32, per-direction SDPA + autograd, "
                  f"{dt:.2f} s wall",
    }
    # the small workload runs whole
    q, k, v, g = oattn.make_attention_inputs(8, 8, 128, 64, 4, dtype=torch.float32, seed=0)
    times = []
    for _ in range(7):
        t0 = time.perf_counter()
        oattn.attention_pullback_sdpa_loop(q, k, v, g, softmax_scale=1.0 / math.sqrt(64), causal=True)
        times.append(time.perf_counter() - t0)
    dt = st.median(times[2:])
    out["attn_pullback_fp16_B8_H8_T128_Dh64_P4"] = {
        "value": flops(8, 8, 128, 64, 4) / dt / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "sample": f"the whole workload in fp32, per-direction SDPA + autograd, median of 5 runs, {dt * 1e3:.1f} ms",
    }
    return out


def _end_to_end_step(steps: int, with_cpu_baseline: bool) -> dict:
    """One LBI scan backward step at the end-to-end configuration, run as the training loop runs it (reference
    train/runners.py:361-372): 12 layers of d_model 768 (12 heads of 64), vocabulary 50257, 6 regions of 2 layers,
    interface width 64, batch 8, sequence 1024, bf16 weights and activations, fp32 interface.  The forward (the
    stand-in model of the test suite; the reference's own model in a deployment) runs outside the timed region;
    timed is ``ScanADEngine.backward``: readout VJP, state Jacobians of the five regions the scan reads (region
    input pullback, 64 directions), interface scan with its cross-check, parameter VJPs of all six regions, canvas
    VJP - every region-level product on the HIP kernels.  Checked against dense fp32 ``loss.backward()`` of the same
    rounded weights on the device; the host baseline is that dense backward in fp32 on the host threads."""
    import copy

    import torch

    from latent_bounded_interfaces_amd import benchmarks as lbi_bench
    from latent_bounded_interfaces_amd.backends import HipTransformerLowering
    from latent_bounded_interfaces_amd.backward import ScanADEngine
    from latent_bounded_interfaces_amd.backward.suffix_scan import propagate_state_adjoint_from_last_region_input
    from oracle import lbi_model as olbi

    device = torch.device("cuda", 0)
    cfg = olbi.END_TO_END
    batch, seq_len = olbi.END_TO_END_BATCH, olbi.END_TO_END_SEQ
    cpu_model = olbi.end_to_end_model()
    ids, targets = olbi.end_to_end_batch()
    model = copy.deepcopy(cpu_model).to(device)
    model.region_backend.lowering = HipTransformerLowering()
    ids_d, targets_d = ids.to(device), targets.to(device)
    engine = ScanADEngine(state_jacobian_mode="structured", local_vjp_mode="structured")

    def forward():
        logits, cache = model.forward_with_cache(ids_d)
        return olbi.token_loss(logits, targets_d), cache

    def timed(fn, count):
        out = []
        for _ in range(count):
            loss, cache = forward()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            result = fn(loss, cache)
            torch.cuda.synchronize()
            out.append((time.perf_counter() - t0) * 1e3)
            del loss, cache
        return out, result

    step = lambda loss, cache: engine.backward(model=model, loss=loss, cache=cache)
    timed(step, 1)                                                    # warm-up (allocator, verify-once probe)
    step_ms, result = timed(step, steps)
    jac = lambda loss, cache: engine.pullback_provider.materialize_state_jacobian_t(model=model, cache=cache,
                                                                                     skip_last=True)
    jac_ms, jts = timed(jac, max(2, steps // 2))
    g_last = torch.randn(batch, cfg["interface_width"], device=device)
    scan_ms = _time_events(lambda: propagate_state_adjoint_from_last_region_input(
        jts, g_last, num_regions=len(jts), materialize_suffix=True), 10, 2)

    # error against the dense fp32 path on the device
    dense_model = copy.deepcopy(model).float()
    dense_model.region_backend.lowering = None
    _, dense = olbi.dense_gradients(dense_model, ids_d, targets_d)
    del dense_model
    err = norm = 0.0
    for name, want in dense.items():
        if want is not None:
            got = result.grad_map[name].double()
            err += float(((got - want.double()) ** 2).sum())
            norm += float((want.double() ** 2).sum())
    del dense
    torch.cuda.empty_cache()

    # algorithmic work: region pullbacks with 64 directions (5 regions), one-direction sweeps with the weight
    # gradients (as many flops again as the cotangent products) for all 6 regions, readout products (logits
    # cotangent times the head weight, and its weight gradient)
    shape = dict(dim=cfg["dim"], n_heads=cfg["n_heads"], n_kv_heads=cfg["n_kv_heads"],
                 head_dim=cfg["dim"] // cfg["n_heads"], hidden=cfg["hidden"], layers=cfg["layers_per_region"],
                 batch=batch, seq_len=seq_len)
    regions = cfg["layers"] // cfg["layers_per_region"]
    jac_flops = (regions - 1) * lbi_bench.region_flops(basis=cfg["interface_width"], **shape)["total"]
    one = lbi_bench.region_flops(basis=1, **shape)
    vjp_flops = regions * (2 * one["gemm"] + one["attention"])
    head_flops = 2 * 2.0 * batch * seq_len * cfg["dim"] * cfg["vocab_size"]
    flops = jac_flops + vjp_flops + head_flops
    step_avg = statistics.fmean(step_ms)
    tflops = flops / (step_avg * 1e-3) / 1e12
    out = {
        "workload": "LBI scan backward step as the training loop runs it (ScanADEngine.backward on a real forward "
                    "cache): 12 layers d_model 768, 12 heads x 64, hidden 3072, conv 4, vocab 50257, 6 regions x 2 "
                    "layers, interface width 64, B=8 T=1024, bf16 weights and activations, fp32 interface; forward "
                    "outside the timed region",
        "step_ms_avg": step_avg, "step_ms_min": min(step_ms), "steps_per_s": 1e3 / step_avg,
        "tokens_per_s": batch * seq_len * 1e3 / step_avg,
        "state_jacobians_ms": statistics.fmean(jac_ms), "interface_scan_ms": statistics.fmean(scan_ms),
        "readout_local_vjps_canvas_ms": step_avg - statistics.fmean(jac_ms) - statistics.fmean(scan_ms),
        "interface_scan_rms": result.diagnostics["interface_scan_rms"],
        "relative_l2_error_vs_dense_fp32": (err / norm) ** 0.5,
        "algorithmic_flops": {"state_jacobians": jac_flops, "local_vjps": vjp_flops, "readout": head_flops},
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / PEAK_BF16_MFMA_TFLOPS},
    }
    del model
    torch.cuda.empty_cache()
    if with_cpu_baseline:
        # dense fp32 loss.backward() of the same model on the host threads, one of the eight sequences
        host = cpu_model.float()
        logits, _ = host.forward_with_cache(ids[:1])
        loss = olbi.token_loss(logits, targets[:1])
        t0 = time.perf_counter()
        loss.backward()
        dt = time.perf_counter() - t0
        out["cpu_baseline"] = {
            "value": 1.0 / (dt * batch), "unit": "steps/s", "cores": int(torch.get_num_threads()), "kind": "port",
            "sample": f"dense fp32 loss.backward() of the same 12-layer model on 1 of the {batch} sequences "
                      f"({dt:.2f} s wall), scaled by {batch}",
        }
    return out


def main() -> int:
    args = _parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (the path has no cross-GPU "
              "dependency; shard the batch and run one process per GPU); rerun with --gpus 1",
              file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)

    from latent_bounded_interfaces_amd import _lib
    from latent_bounded_interfaces_amd import benchmarks as lbi_bench

    lib = _lib.load()
    stream = _lib.current_stream_ptr(device)

    def scan_call(mats, out):
        _lib.check(lib.lbi_suffix_scan(mats.data_ptr(), out.data_ptr(), SCAN_B, SCAN_K, SCAN_D,
                                       _lib.dtype_code(mats.dtype), _lib.LBI_F32, stream), "lbi_suffix_scan")

    def cot_call(mats, g, out):
        _lib.check(lib.lbi_suffix_cotangents(mats.data_ptr(), g.data_ptr(), out.data_ptr(), SCAN_B, SCAN_K,
                                             SCAN_D, _lib.dtype_code(mats.dtype), stream),
                   "lbi_suffix_cotangents")

    if args.copy_calibration:
        src = torch.empty(256 * 1024 * 1024, device=device, dtype=torch.float32)  # 1 GiB
        src.fill_(1.0)
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    mats, g = _scan_inputs(device, torch.float32)
    out = torch.empty((SCAN_B, SCAN_K + 1, SCAN_D, SCAN_D), device=device, dtype=torch.float32)
    cot = torch.empty((SCAN_B, SCAN_K + 1, SCAN_D), device=device, dtype=torch.float32)

    def step():
        _lib.check(lib.lbi_suffix_scan_with_cotangents(mats.data_ptr(), g.data_ptr(), out.data_ptr(), cot.data_ptr(),
                                                       SCAN_B, SCAN_K, SCAN_D, _lib.dtype_code(mats.dtype),
                                                       _lib.LBI_F32, stream), "lbi_suffix_scan_with_cotangents")

    # ---- headline: exactly `steps` timed steps between synchronisations ----------------
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    value = SCAN_B * SCAN_K / (wall / args.steps)

    # ---- dominant kernel alone, HIP events on its stream ------------------------------
    scan_ms = _time_events(step, args.steps, 2)
    scan_avg = statistics.fmean(scan_ms)
    scan_flops = SCAN_B * (SCAN_K - 1) * 2 * SCAN_D ** 3
    scan_bytes = SCAN_B * SCAN_K * SCAN_D * SCAN_D * (4 + 4)
    achieved_tflops = scan_flops / (scan_avg * 1e-3) / 1e12
    first, first_cot = out.clone(), cot.clone()
    step()
    torch.cuda.synchronize()
    bit_stable = bool(torch.equal(first, out)) and bool(torch.equal(first_cot, cot))
    del first, first_cot

    result = {
        "metric": "scan composed-pullbacks/s + attn-pullback TFLOP/s, % of MI355X roofline",
        "value": value,
        "unit": "composed_pullbacks/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "interface suffix scan B=64 K=128 d=256 fp32: all K suffix matrices + all K cotangents",
            "B": SCAN_B, "K": SCAN_K, "d": SCAN_D,
        },
        "roofline": {
            "bound": "mfma",
            "kernel": SCAN_KERNEL + " (lbi_suffix_scan_with_cotangents)",
            "achieved": achieved_tflops,
            "peak": PEAK_FP32_MFMA_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved_tflops / PEAK_FP32_MFMA_TFLOPS,
            "traffic": lbi_bench.load_traffic(SCAN_TRAFFIC_JSON, SCAN_KERNEL),
            "kernel_ms_avg": scan_avg,
            "kernel_ms_min": min(scan_ms),
            "algorithmic_flops": scan_flops,
            "algorithmic_bytes": scan_bytes,
            "hbm_gbs": scan_bytes / (scan_avg * 1e-3) / 1e9,
        },
        "bit_stable_rerun": bit_stable,
    }

    if not args.no_extra:
        extra = {}
        only_ms = _time_events(lambda: scan_call(mats, out), args.steps, 2)
        extra["scan_matrices_only_fp32"] = {
            "kernel_ms_avg": statistics.fmean(only_ms),
            "tflops": scan_flops / (statistics.fmean(only_ms) * 1e-3) / 1e12,
        }
        cot_ms = _time_events(lambda: cot_call(mats, g, cot), args.steps, 2)
        cot_avg = statistics.fmean(cot_ms)
        cot_bytes = SCAN_B * SCAN_K * SCAN_D * SCAN_D * 4
        extra["scan_cotangent_only_fp32"] = {
            "kernel_ms_avg": cot_avg, "pullbacks_per_s": SCAN_B * SCAN_K / (cot_avg * 1e-3),
            "roofline": {"bound": "hbm", "achieved": cot_bytes / (cot_avg * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                         "unit": "GB/s", "frac": cot_bytes / (cot_avg * 1e-3) / 1e9 / PEAK_HBM_GBS},
        }
        mats_bf16 = mats.to(torch.bfloat16)
        bf_bytes = SCAN_B * SCAN_K * SCAN_D * SCAN_D * (2 + 4)

        def fused_bf16():
            _lib.check(lib.lbi_suffix_scan_with_cotangents(mats_bf16.data_ptr(), g.data_ptr(), out.data_ptr(),
                                                           cot.data_ptr(), SCAN_B, SCAN_K, SCAN_D, _lib.LBI_BF16,
                                                           _lib.LBI_F32, stream), "lbi_suffix_scan_with_cotangents")

        # the same workload as the headline (matrices + cotangents) with bf16 storage, and the matrices alone
        for key, fn in (("scan_bf16_storage_fp32_accumulate", fused_bf16),
                        ("scan_bf16_storage_matrices_only", lambda: scan_call(mats_bf16, out))):
            bf_avg = statistics.fmean(_time_events(fn, args.steps, 2))
            extra[key] = {
                "kernel_ms_avg": bf_avg, "pullbacks_per_s": SCAN_B * SCAN_K / (bf_avg * 1e-3),
                "tflops": scan_flops / (bf_avg * 1e-3) / 1e12,
                "roofline": {"bound": "hbm", "achieved": bf_bytes / (bf_avg * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                             "unit": "GB/s", "frac": bf_bytes / (bf_avg * 1e-3) / 1e9 / PEAK_HBM_GBS},
            }
        del mats_bf16
        extra.update(lbi_bench.scan_section(steps=max(5, args.steps // 2)))
        extra.update(lbi_bench.attention_section(steps=max(3, args.steps // 4)))
        torch.cuda.empty_cache()
        extra.update(lbi_bench.region_section(steps=max(3, args.steps // 4)))
        torch.cuda.empty_cache()
        extra["lbi_backward_step_bf16_L12_D768_V50257_B8_T1024_d64"] = _end_to_end_step(3, not args.no_cpu_baseline)
        result["extra"] = extra

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = _cpu_baseline(args.cpu_sample_batch)
        if "extra" in result:
            for key, base in _cpu_attention_baselines().items():
                if key in result["extra"]:
                    result["extra"][key]["cpu_baseline"] = base

    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
