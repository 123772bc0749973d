"""Benchmark of the DiT joint-attention hot path on one MI355X.

A "step" is one pass of the fused QK-norm + rope + attention over the Klein
1024^2 workload (B=1, H=24, S=4608 = 512 text + 64x64 image tokens, D=128,
bf16 in and out), with every operand already resident in HBM. Prints one JSON
line: TFLOP/s from the algorithmic FLOPs 4*S^2*D*H, the roofline fraction of
the dense bf16 MFMA peak from HIP events on the library's stream, and the
scalar CPU oracle timed on this host for comparison.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA peak (2.5 PFLOP/s)


def cpu_baseline(w, seconds_target=15.0):
    """The oracle's scalar fp32 path (norm + rope on every K row, then
    attention for a sample of query tokens, all heads), one host thread."""
    import numpy as np

    from oracle import zoracle as zo
    from tests import refimpl

    t0 = time.perf_counter()
    qn, kn = refimpl.prepared_qk(w, 0)
    prep_s = time.perf_counter() - t0
    cfg = zo.Config(w.tokens, w.heads, w.heads, 128)
    per_token_flops = 4.0 * 128 * w.heads * w.tokens
    # calibrate on 2 tokens, then size the sample for the time target
    t0 = time.perf_counter()
    zo.attention_rows(qn, kn, w.v[0], cfg, 0, 2)
    per_tok = (time.perf_counter() - t0) / 2
    n = int(max(8, min(w.tokens, seconds_target / max(per_tok, 1e-6))))
    start = (w.tokens - n) // 2
    t0 = time.perf_counter()
    zo.attention_rows(qn, kn, w.v[0], cfg, start, start + n)
    dt = time.perf_counter() - t0
    tflops = per_token_flops * n / dt / 1e12
    return {
        "value": tflops,
        "unit": "TFLOP/s",
        "cores": 1,
        "kind": "port",
        "sample": f"{n} of {w.tokens} query tokens x {w.heads} heads against all keys in {dt:.1f} s "
                  f"(+{prep_s:.1f} s norm+rope of all rows); full call extrapolates to "
                  f"{dt / n * w.tokens:.0f} s on one core of {os.cpu_count()}",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="klein_1024")
    ap.add_argument("--k-site", choices=["tile", "prepass"], default=os.environ.get("ZDRAW_BENCH_K_SITE", "tile"))
    ap.add_argument("--variant", type=int, default=0, help="kernel build: 0 default, 1/2 the 32-row kernel")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path has no multi-GPU part (run with --gpus 1)")

    import numpy as np

    from zdraw_amd import hip, host, workloads as wl

    L = hip.lib()
    ctx = host.Context.init()
    L.zdraw_hip_set_attention_variant(args.variant)
    w = wl.by_name(args.workload, seed=0)
    k_site = hip.K_PREPASS if args.k_site == "prepass" else hip.K_IN_TILE_LOAD
    res = wl.Resident(ctx, w, dtype=hip.BF16, k_site=k_site)

    def enqueue(n):
        b = L.zdraw_hip_batch_begin(ctx.queue)
        for _ in range(n):
            rc = res.launch(b)
            if rc != 0:
                raise RuntimeError(f"launch rc={rc}: {hip.last_error()}")
        return b

    # warm-up (untimed)
    if L.zdraw_hip_batch_end(enqueue(args.warmup)) != 0:
        raise RuntimeError(hip.last_error())
    L.zdraw_hip_queue_sync(ctx.queue)

    # timed region: K launches back to back on the library's stream, bracketed
    # by a full synchronisation on both sides (wall clock) and by HIP events
    # recorded on that same stream (device time of the launches).
    ev0, ev1 = L.zdraw_hip_event_create(), L.zdraw_hip_event_create()
    L.zdraw_hip_queue_sync(ctx.queue)
    t0 = time.perf_counter()
    L.zdraw_hip_event_record(ev0, ctx.queue)
    b = enqueue(args.steps)
    L.zdraw_hip_event_record(ev1, ctx.queue)
    if L.zdraw_hip_batch_end(b) != 0:
        raise RuntimeError(hip.last_error())
    L.zdraw_hip_queue_sync(ctx.queue)
    wall = time.perf_counter() - t0
    dev_ms = L.zdraw_hip_event_elapsed_ms(ev0, ev1)
    L.zdraw_hip_event_release(ev0)
    L.zdraw_hip_event_release(ev1)

    out = res.read_output()
    if not np.isfinite(out).all():
        raise RuntimeError("non-finite output")

    desc = (f"{w.name}: B={w.batch} H={w.heads} S={w.tokens} D=128 bf16, fused QK-RMSNorm + axial RoPE, "
            + ("no mask" if w.key_pad is None else "ragged key-padding mask"))
    flops = w.flops
    ms_per_step = wall * 1e3 / args.steps
    value = flops / (wall / args.steps) / 1e12
    kern_ms = dev_ms / args.steps
    achieved = flops / (kern_ms * 1e-3) / 1e12
    line = {
        "metric": "attn TFLOP/s + % of bf16 MFMA peak, Klein 1024^2 (H=24,S=4608,D=128)",
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": desc,
            "k_norm_rope_site": args.k_site,
            "kernel_variant": args.variant,
            "pct_of_bf16_mfma_peak": 100.0 * value / PEAK_BF16_TFLOPS,
        },
        "roofline": {
            "bound": "mfma",
            "achieved": achieved,
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / PEAK_BF16_TFLOPS,
            "traffic": None,
            "kernel": "attn_fwd_kernel" + (" (+ qk_prepass_kernel in the same events)" if args.k_site == "prepass" else ""),
            "kernel_ms": kern_ms,
        },
    }
    res.release()
    ctx.deinit()
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(w)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
