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


class ContextOnCus:
    """The host context with its queue swapped for one confined to `cu_count` compute units
    (zdraw_hip_create_queue_on_cus, a measurement aid): `--cu-count`."""

    def __init__(self, L, ctx, cu_count):
        self._L, self._ctx = L, ctx
        self.queue = L.zdraw_hip_create_queue_on_cus(ctx.device, cu_count)
        if not self.queue:
            raise RuntimeError("zdraw_hip_create_queue_on_cus failed")

    def __getattr__(self, name):
        return getattr(self._ctx, name)

    def deinit(self):
        self._L.zdraw_hip_release_queue(self.queue)
        self._ctx.deinit()


def timed_region(L, ctx, res, steps):
    """K launches back to back on the library's stream, bracketed by a full
    synchronisation on both sides (wall clock); the attention kernel of every
    launch is bracketed by its own HIP events on that stream (device time)."""
    L.zdraw_hip_queue_sync(ctx.queue)
    L.zdraw_hip_metrics_reset()
    L.zdraw_hip_trace_attention(1)
    t0 = time.perf_counter()
    b = L.zdraw_hip_batch_begin(ctx.queue)
    for _ in range(steps):
        rc = res.launch(b)
        if rc != 0:
            raise RuntimeError(f"launch rc={rc}")
    if L.zdraw_hip_batch_end(b) != 0:
        raise RuntimeError("batch_end failed")
    L.zdraw_hip_queue_sync(ctx.queue)
    wall = time.perf_counter() - t0
    n = C.c_uint64(0)
    kern_ns = L.zdraw_hip_trace_attention_ns(C.byref(n))
    L.zdraw_hip_trace_attention(0)
    if n.value != steps:
        raise RuntimeError(f"traced {n.value} attention launches, expected {steps}")
    return wall, kern_ns / 1e6 / steps


def spin_up(L, ctx, res, ms):
    """Untimed launches until `ms` of wall time have passed: the device leaves
    its idle power state and settles at its sustained clock before anything is
    measured (the first tens of milliseconds after idle run measurably slower)."""
    t0 = time.perf_counter()
    n = 0
    while (time.perf_counter() - t0) * 1e3 < ms:
        b = L.zdraw_hip_batch_begin(ctx.queue)
        for _ in range(100):
            if res.launch(b) != 0:
                raise RuntimeError("launch failed during spin-up")
        if L.zdraw_hip_batch_end(b) != 0:
            raise RuntimeError("batch_end failed during spin-up")
        n += 100
    return n


def side_leg(L, ctx, w, *, bounded=True, staging=0, spin_ms=300.0, warm=10, steps=100):
    """A short measurement of one workload outside the driver-timed region: whole step
    (pre-pass + attention, wall clock) and the attention kernel alone (its own HIP events)."""
    from zdraw_amd import hip, workloads as wl

    res = wl.Resident(ctx, w, dtype=hip.BF16, k_site=hip.K_PREPASS, bounded=bounded, staging=staging)
    spin_up(L, ctx, res, spin_ms)
    timed_region(L, ctx, res, warm)
    wall, kern_ms = timed_region(L, ctx, res, steps)
    res.release()
    return {"value": w.flops / (wall / steps) / 1e12, "kernel_tflops": w.flops / (kern_ms * 1e-3) / 1e12,
            "kernel_frac": w.flops / (kern_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, "ms_per_step": wall * 1e3 / steps,
            "kernel_ms": kern_ms, "steps": steps}


def attn_scale_main(args):
    """`--workload attn_scale`: the reference's attention scaling measurement
    (cmd/gemmbench.zig:631-678): plain attention through the standalone blocking entry on resident
    f32 buffers, heads 30, head_dim 128, tokens 4224 / 8448 / 16896, best wall time of three calls
    after one untimed call, as the reference takes it; the attention kernel's own device time
    beside it. The line's `value` is the 16896-token figure."""
    import numpy as np

    from zdraw_amd import hip, host, workloads as wl

    L = hip.lib()
    ctx = host.Context.init()
    heads = wl.ATTN_SCALE_HEADS
    rows = {}
    for tokens in wl.ATTN_SCALE_TOKENS:
        x = wl.attn_scale_input(tokens)
        qb, kb, vb = ctx.buffer(x), ctx.buffer(x), ctx.buffer(x)
        ob = ctx.buffer(nbytes=x.nbytes)
        p = hip.AttnParams(tokens, heads, heads, 128, 0, 0)

        def call():
            rc = L.zdraw_hip_run_attention(ctx.queue, ctx.block_pipeline, qb.handle, kb.handle, vb.handle, ob.handle,
                                           C.byref(p), hip.K_BLOCK, 512)
            if rc != 0:
                raise RuntimeError(f"attention rc={rc}: {hip.last_error()}")

        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < args.spinup_ms / 3:
            call()
        best = float("inf")
        L.zdraw_hip_metrics_reset()
        L.zdraw_hip_trace_attention(1)
        for _ in range(max(args.steps, 3) if args.steps < 50 else 3):
            t0 = time.perf_counter()
            call()
            best = min(best, time.perf_counter() - t0)
        n = C.c_uint64(0)
        kern_ns = L.zdraw_hip_trace_attention_ns(C.byref(n))
        L.zdraw_hip_trace_attention(0)
        out = ob.read(np.float32, x.shape)
        if not np.isfinite(out).all():
            raise RuntimeError("non-finite output")
        flops = 4.0 * tokens * tokens * 128 * heads
        rows[str(tokens)] = {"ms": best * 1e3, "tflops": flops / best / 1e12,
                             "kernel_ms": kern_ns / 1e6 / max(n.value, 1),
                             "kernel_tflops": flops / (kern_ns / 1e9 / max(n.value, 1)) / 1e12}
        for b in (qb, kb, vb, ob):
            b.release()
    ctx.deinit()
    last = rows[str(wl.ATTN_SCALE_TOKENS[-1])]
    line = {
        "metric": "attention TFLOP/s across token counts (heads 30, head_dim 128, resident f32 buffers, blocking call)",
        "value": last["tflops"], "unit": "TFLOP/s", "n_gpus": 1, "steps": 3, "warmup": 1, "ms_per_step": last["ms"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "attn_scale: plain attention, H=30, D=128, S in 4224 / 8448 / 16896, f32 in and out "
                               "(rounded to bf16 once, ahead of the kernel), best of three blocking calls",
                   "tokens": rows},
        "roofline": {"bound": "mfma", "achieved": last["kernel_tflops"], "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": last["kernel_tflops"] / PEAK_BF16_TFLOPS, "traffic": None, "kernel": "attn_fwd_kernel",
                     "kernel_ms": last["kernel_ms"]},
    }
    print(json.dumps(line), flush=True)


def gemm_main(args):
    """`--path gemm`: the projection GEMM C[m][n] = A[m][k] x W[n][k]^T on its own (bf16 operands
    and output, fp32 accumulation), by default the fused Q/K/V projection of a Klein 1024^2 block
    (4608 tokens, hidden 3072 -> 3 x 3072). Same timing discipline as the attention line."""
    import numpy as np

    from zdraw_amd import hip, host

    L = hip.lib()
    ctx = host.Context.init()
    m, k, n = args.m, args.k, args.n
    rng = np.random.default_rng(0)
    a = rng.standard_normal((m, k), dtype=np.float32)
    w = rng.standard_normal((n, k), dtype=np.float32) * np.float32(k ** -0.5)
    ab, wb = ctx.buffer(host.f32_to_bf16_bits(a)), ctx.buffer(host.f32_to_bf16_bits(w))
    cb = ctx.buffer(nbytes=m * n * 2)
    params = hip.GemmParams(m, k, n, hip.W_BF16, hip.GEMM_HALF, 0)
    ext = hip.GemmExt(0, 0, 0, 0, 0, hip.BF16, hip.BF16)

    def burst(count):
        b = L.zdraw_hip_batch_begin(ctx.queue)
        for _ in range(count):
            rc = L.zdraw_hip_run_gemm_ext_enc(b, ab.handle, wb.handle, cb.handle, C.byref(params), C.byref(ext))
            if rc != 0:
                raise RuntimeError(f"gemm rc={rc}: {hip.last_error()}")
        if L.zdraw_hip_batch_end(b) != 0:
            raise RuntimeError("batch_end failed")

    t0 = time.perf_counter()
    spun = 0
    while (time.perf_counter() - t0) * 1e3 < args.spinup_ms:
        burst(100)
        spun += 100
    burst(max(args.warmup, 1))
    # HIP events on the library's stream around the K timed launches (no other kernel runs between them)
    e0, e1 = L.zdraw_hip_event_create(), L.zdraw_hip_event_create()
    L.zdraw_hip_queue_sync(ctx.queue)
    t0 = time.perf_counter()
    L.zdraw_hip_event_record(e0, ctx.queue)
    burst(args.steps)
    L.zdraw_hip_event_record(e1, ctx.queue)
    L.zdraw_hip_event_sync(e1)
    wall = time.perf_counter() - t0
    kern_ms = L.zdraw_hip_event_elapsed_ms(e0, e1) / args.steps
    out = host.bf16_bits_to_f32(cb.read(np.uint16, (m, n)))
    if not np.isfinite(out).all():
        raise RuntimeError("non-finite output")
    flops = 2.0 * m * k * n
    value = flops / (wall / args.steps) / 1e12
    achieved = flops / (kern_ms * 1e-3) / 1e12
    line = {
        "metric": "projection GEMM TFLOP/s + % of bf16 MFMA peak",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall * 1e3 / args.steps, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"gemm: C[{m}][{n}] = A[{m}][{k}] x W[{n}][{k}]^T, bf16 in and out, fp32 accumulate",
                   "pct_of_bf16_mfma_peak": 100.0 * value / PEAK_BF16_TFLOPS, "untimed_spinup_launches": spun},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS, "traffic": None, "kernel": "gemm_kernel", "kernel_ms": kern_ms},
    }
    if not args.no_cpu:
        from oracle import zoracle as zo
        rows = 16
        t0 = time.perf_counter()
        zo.linear_batch(a[:rows], w)
        dt = time.perf_counter() - t0
        rows = int(max(16, min(m, rows * 10.0 / max(dt, 1e-6))))
        t0 = time.perf_counter()
        zo.linear_batch(a[:rows], w)
        dt = time.perf_counter() - t0
        line["cpu_baseline"] = {"value": 2.0 * rows * k * n / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
                                "sample": f"{rows} of {m} rows in {dt:.1f} s; full call extrapolates to {dt / rows * m:.0f} s"}
    for b in (ab, wb, cb):
        b.release()
    ctx.deinit()
    return line


def chain_main(args):
    """`--path chain`: the attention segment of one Z-Image layer at the zimage_1024 shape
    (4608 tokens, 30 heads, hidden 3840): q/k/v projections, QK-norm + rope pre-pass, attention,
    output projection, bf16 activations and weights. FLOPs = 4 projections + attention."""
    import numpy as np

    from zdraw_amd import hip, host
    from zdraw_amd import workloads as wl

    L = hip.lib()
    ctx = host.Context.init()
    w = wl.by_name("zimage_1024", seed=0)
    tokens, heads = w.tokens, (args.chain_heads or w.heads)
    hidden = inner = heads * 128
    rng = np.random.default_rng(0)
    bits = lambda a: host.f32_to_bf16_bits(a)
    x = rng.standard_normal((tokens, hidden), dtype=np.float32)
    wall_w = rng.standard_normal((4, inner, hidden), dtype=np.float32) * np.float32(hidden ** -0.5)
    act32 = args.chain_act == "f32"
    nb, wb = ctx.buffer(x if act32 else bits(x)), ctx.buffer(bits(wall_w))
    qb, kb, vb, mixb, ob = (ctx.buffer(nbytes=tokens * inner * (4 if act32 else 2)) for _ in range(5))
    ones = ctx.buffer(np.ones(128, np.float32))
    posb = ctx.buffer(np.ascontiguousarray(w.pos, dtype=np.uint64))
    ropeb = ctx.buffer(w.rope_pairs)
    p = hip.ChainAttnParams()
    for i, name in enumerate(("q", "k", "v", "proj")):
        setattr(p, name, hip.GemmParams(tokens, hidden, inner, hip.W_BF16, hip.GEMM_HALF, i * inner * hidden * 2))
    p.qk = hip.QkNormParams(tokens, heads, heads, 128, hip.W_F32, hip.W_F32, *wl.ZIMAGE_DIMS, wl.ZIMAGE_EPS, 0, 0,
                            *w.rope_bases)
    p.attn = hip.AttnParams(tokens, heads, heads, 128, 0, 0)
    p.act_dtype = hip.F32 if act32 else hip.BF16
    p.score_bound = host.score_bound(np.ones(128, np.float32), np.ones(128, np.float32), None, None)
    bufs = hip.ChainAttnBuffers(nb.handle, qb.handle, kb.handle, vb.handle, mixb.handle, ob.handle)
    wts = hip.ChainAttnWeights(wb.handle, wb.handle, wb.handle, ones.handle, ones.handle, posb.handle, ropeb.handle,
                               wb.handle)

    def burst(count):
        b = L.zdraw_hip_batch_begin(ctx.queue)
        for _ in range(count):
            rc = L.zdraw_hip_run_chain_attn_enc(b, C.byref(bufs), C.byref(wts), C.byref(p))
            if rc != 0:
                raise RuntimeError(f"chain rc={rc}: {hip.last_error()}")
        if L.zdraw_hip_batch_end(b) != 0:
            raise RuntimeError("batch_end failed")

    t0 = time.perf_counter()
    spun = 0
    while (time.perf_counter() - t0) * 1e3 < args.spinup_ms:
        burst(20)
        spun += 20
    burst(max(args.warmup, 1))
    e0, e1 = L.zdraw_hip_event_create(), L.zdraw_hip_event_create()
    L.zdraw_hip_queue_sync(ctx.queue)
    t0 = time.perf_counter()
    L.zdraw_hip_event_record(e0, ctx.queue)
    burst(args.steps)
    L.zdraw_hip_event_record(e1, ctx.queue)
    L.zdraw_hip_event_sync(e1)
    wall = time.perf_counter() - t0
    dev_ms = L.zdraw_hip_event_elapsed_ms(e0, e1) / args.steps
    out = ob.read(np.float32, (tokens, hidden)) if act32 else host.bf16_bits_to_f32(ob.read(np.uint16, (tokens, hidden)))
    if not np.isfinite(out).all():
        raise RuntimeError("non-finite output")
    gemm_flops = 4 * 2.0 * tokens * hidden * inner
    attn_flops = 4.0 * 128 * heads * tokens * tokens
    flops = gemm_flops + attn_flops
    value = flops / (wall / args.steps) / 1e12
    line = {
        "metric": "Z-Image layer attention segment TFLOP/s (4 projections + attention)",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall * 1e3 / args.steps, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"zimage chain segment: tokens {tokens}, heads {heads}, hidden {hidden}, {args.chain_act} activations, bf16 weights",
                   "gemm_gflop": gemm_flops / 1e9, "attention_gflop": attn_flops / 1e9,
                   "pct_of_bf16_mfma_peak": 100.0 * value / PEAK_BF16_TFLOPS, "untimed_spinup_segments": spun},
        "roofline": {"bound": "mfma", "achieved": flops / (dev_ms * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": flops / (dev_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, "traffic": None,
                     "kernel": "3 x gemm + qk_prepass + attn_fwd + gemm", "kernel_ms": dev_ms},
    }
    if args.chain_check_rows and not act32:
        line["parity_check"] = chain_check(w, tokens, heads, x, wall_w, out, args.chain_check_rows)
    for b in (nb, wb, qb, kb, vb, mixb, ob, ones, posb, ropeb):
        b.release()
    ctx.deinit()
    return line


def chain_check(w, tokens, heads, x, weights, got, nrows):
    """The segment's output rows `rows` against the oracle chain (runtime/ops.zig linear ->
    zimage/zattn.zig norm -> rope -> attention.run -> linear) with the same bf16 hand-overs:
    K and V of every token, Q and the output projection of the sampled rows only."""
    import numpy as np

    from oracle import zoracle as zo
    from zdraw_amd import host
    from zdraw_amd import workloads as wl

    t0 = time.perf_counter()
    rb = lambda a: host.bf16_bits_to_f32(host.f32_to_bf16_bits(np.ascontiguousarray(a, np.float32)))
    rows = sorted(set(int(t) for t in np.random.default_rng(1).choice(tokens, nrows, replace=False)) | {0, tokens - 1})
    xr, wr = rb(x), [rb(weights[i]) for i in range(4)]
    cfg = zo.RopeConfig(wl.ZIMAGE_DIMS, wl.ZIMAGE_LENS, wl.ZIMAGE_THETA)
    vals = zo.zrope_fill(cfg)
    pos = np.ascontiguousarray(w.pos, dtype=np.uintp)
    ones = np.ones(128, np.float32)
    k = rb(zo.linear_batch(xr, wr[1])).reshape(tokens, heads, 128)
    v = rb(zo.linear_batch(xr, wr[2])).reshape(tokens, heads, 128)
    q = np.zeros((tokens, heads, 128), np.float32)
    q[rows] = rb(zo.linear_batch(xr[rows], wr[0])).reshape(len(rows), heads, 128)
    qn = np.zeros_like(q)
    qn[rows] = zo.zimage_rotate(zo.zimage_norm_heads(q[rows], ones, wl.ZIMAGE_EPS), vals, cfg, pos[rows])
    kn = zo.zimage_rotate(zo.zimage_norm_heads(k, ones, wl.ZIMAGE_EPS), vals, cfg, pos)
    mix = zo.attention_token_list(qn, kn, v, zo.Config(tokens, heads, heads, 128), rows, threads=1)
    want = zo.linear_batch(rb(mix.reshape(len(rows), heads * 128)), wr[3])
    err = np.abs(got[rows].astype(np.float64) - want)
    s = max(float(np.sqrt(np.mean(want.astype(np.float64) ** 2))), 1.0)
    if err.max() > 2e-2 * s or err.mean() > 2e-3 * s:
        raise RuntimeError(f"chain segment differs from the oracle chain on sampled rows: max {err.max():.3e} mean {err.mean():.3e}")
    return {"rows": len(rows), "max_abs": float(err.max()), "mean_abs": float(err.mean()), "output_rms": s,
            "oracle_s": time.perf_counter() - t0}


def wide_main(args):
    """`--path wide`: one wide head (heads 1, head_dim 512) at the VAE mid-block shape of a 1024 px
    render, 16384 tokens, f32 token-major in and out as the reference passes them. The step is the
    rounding pass + the attention kernel; FLOPs = 4 x 512 x tokens^2."""
    import numpy as np

    from zdraw_amd import hip, host

    L = hip.lib()
    ctx = host.Context.init()
    tokens = args.wide_tokens
    rng = np.random.default_rng(0)
    q, k, v = (rng.standard_normal((tokens, 512), dtype=np.float32) for _ in range(3))
    qb, kb, vb = ctx.buffer(q), ctx.buffer(k), ctx.buffer(v)
    ob = ctx.buffer(nbytes=q.nbytes)
    err = C.create_string_buffer(128)
    pipe = L.zdraw_hip_compile(ctx.device, None, b"attention_wide_mfma", err, 128)
    if not pipe:
        raise RuntimeError(err.value)
    p = hip.AttnParams(tokens, 1, 1, 512, 0, 0)

    def burst(count):
        b = L.zdraw_hip_batch_begin(ctx.queue)
        for _ in range(count):
            rc = L.zdraw_hip_run_attention_enc(b, pipe, qb.handle, kb.handle, vb.handle, ob.handle, C.byref(p),
                                               hip.K_WIDE, 512)
            if rc != 0:
                raise RuntimeError(f"wide rc={rc}: {hip.last_error()}")
        if L.zdraw_hip_batch_end(b) != 0:
            raise RuntimeError("batch_end failed")

    t0 = time.perf_counter()
    spun = 0
    while (time.perf_counter() - t0) * 1e3 < args.spinup_ms:
        burst(20)
        spun += 20
    burst(max(args.warmup, 1))
    L.zdraw_hip_queue_sync(ctx.queue)
    t0 = time.perf_counter()
    burst(args.steps)
    wall = time.perf_counter() - t0
    # the attention kernel alone: its own HIP events on the launch stream
    L.zdraw_hip_queue_sync(ctx.queue)
    L.zdraw_hip_metrics_reset()  # (the totals are the process's: an earlier leg may have traced too)
    L.zdraw_hip_trace_attention(1)
    burst(args.steps)
    launches = C.c_uint64(0)
    ns = L.zdraw_hip_trace_attention_ns(C.byref(launches))
    L.zdraw_hip_trace_attention(0)
    kern_ms = ns / max(launches.value, 1) / 1e6
    out = ob.read(np.float32, (tokens, 512))
    if not np.isfinite(out).all():
        raise RuntimeError("non-finite output")
    flops = 4.0 * 512 * tokens * tokens
    value = flops / (wall / args.steps) / 1e12
    achieved = flops / (kern_ms * 1e-3) / 1e12
    line = {
        "metric": "wide-head attention TFLOP/s (heads 1, head_dim 512)",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall * 1e3 / args.steps, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"vae mid-block attention: tokens {tokens}, heads 1, head_dim 512, f32 in and out",
                   "pct_of_bf16_mfma_peak": 100.0 * value / PEAK_BF16_TFLOPS, "untimed_spinup_launches": spun},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS, "traffic": None, "kernel": "attn_wide_kernel + wide_merge_kernel + attn_wide_safe_kernel (no tile flagged)",
                     "kernel_ms": kern_ms},
    }
    if not args.no_cpu:
        from oracle import zoracle as zo
        rows = list(range(0, tokens, max(tokens // 64, 1)))[:64]
        t0 = time.perf_counter()
        want = zo.attention_token_list(q.reshape(tokens, 1, 512), k.reshape(tokens, 1, 512), v.reshape(tokens, 1, 512),
                                       zo.Config(tokens, 1, 1, 512), rows, threads=1)
        dt = time.perf_counter() - t0
        err_max = float(np.abs(out[rows] - want.reshape(len(rows), 512)).max())
        if err_max > 2e-2:
            raise RuntimeError(f"wide attention differs from the oracle on sampled rows: {err_max}")
        line["cpu_baseline"] = {"value": 4.0 * 512 * len(rows) * tokens / dt / 1e12, "unit": "TFLOP/s", "cores": 1,
                                "kind": "port", "sample": f"{len(rows)} of {tokens} query rows in {dt:.1f} s (max abs "
                                f"difference from the GPU rows {err_max:.1e}); full call extrapolates to {dt / len(rows) * tokens:.0f} s"}
    L.zdraw_hip_release_pipeline(pipe)
    for b in (qb, kb, vb, ob):
        b.release()
    ctx.deinit()
    return line


PATH_MAINS = {"gemm": gemm_main, "chain": chain_main, "wide": wide_main}


def other_paths(args):
    """Short legs of the other kernels on this path's either side (`--path gemm|chain|wide` at their
    default shapes), outside the driver-timed region, for the record in the same line."""
    import copy

    out = {}
    for name, steps in (("gemm", 200), ("chain", 60), ("wide", 60)):
        a = copy.copy(args)
        # the wide leg keeps its oracle check of 64 sampled rows (under a second of CPU work)
        a.path, a.steps, a.warmup, a.spinup_ms, a.no_cpu = name, steps, 10, 400.0, name != "wide"
        a.chain_heads, a.chain_check_rows = 0, 0
        line = PATH_MAINS[name](a)
        out[name] = {"workload": line["config"]["workload"], "value": line["value"], "ms_per_step": line["ms_per_step"],
                     "kernel_frac": line["roofline"]["frac"], "kernel": line["roofline"]["kernel"]}
        if name == "wide":
            out[name]["parity_check"] = line["cpu_baseline"]["sample"]
        if name == "chain":
            # the same segment at the full sequence length with 4 heads (hidden 512), where the
            # oracle chain finishes in seconds: sampled output rows against it
            a.chain_heads, a.chain_check_rows, a.steps, a.warmup, a.spinup_ms = 4, 8, 3, 1, 0.0
            small = PATH_MAINS[name](a)
            out[name]["parity_check"] = {"workload": small["config"]["workload"], **small["parity_check"]}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--path", choices=["attention", "gemm", "chain", "wide"], default="attention",
                    help="attention (the headline metric) or the projection GEMM beside it")
    ap.add_argument("--wide-tokens", type=int, default=16384, help="--path wide: sequence length (multiple of 64)")
    ap.add_argument("--chain-heads", type=int, default=0, help="--path chain: heads (hidden = 128 x heads); 0 = the model's 30")
    ap.add_argument("--chain-check-rows", type=int, default=0,
                    help="--path chain: check this many sampled output rows against the oracle chain (use with few heads)")
    ap.add_argument("--chain-act", choices=["bf16", "f32"], default="bf16",
                    help="--path chain: activation buffers as bf16, or f32 as the reference's chain keeps them")
    ap.add_argument("--m", type=int, default=4608)
    ap.add_argument("--k", type=int, default=3072)
    ap.add_argument("--n", type=int, default=9216)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--spinup-ms", type=float, default=1500.0,
                    help="untimed launches for this long before the warm-up steps (clock ramp from idle)")
    ap.add_argument("--workload", default="klein_1024",
                    help="a benchmark shape (klein_1024, klein_512_x4, zimage_1024, klein_edit_ragged), or attn_scale: "
                         "the reference's attention-scaling measurement (heads 30, 4224 / 8448 / 16896 tokens)")
    ap.add_argument("--k-site", choices=["tile", "prepass"], default=os.environ.get("ZDRAW_BENCH_K_SITE", "prepass"),
                    help="where K's norm+rope runs: inside the K-block load, or one pre-pass kernel per call")
    ap.add_argument("--variant", type=int, default=0, help="kernel shape: 0 = 8 waves, 1 = 4 waves x 2 workgroups")
    ap.add_argument("--dynamic-max", action="store_true", help="withhold the score bound (running-maximum softmax)")
    ap.add_argument("--staging", choices=["bf16", "f16"], default="bf16",
                    help="element type of the prepared Q and K (the scores' MFMA operands); P and V are bf16 either way")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-side-legs", action="store_true",
                    help="skip the short untimed-by-value legs (other softmax form, other benchmark shapes, the GEMM, chain and wide-head paths)")
    ap.add_argument("--cu-count", type=int, default=0,
                    help="(attention path) confine the stream to this many compute units (0 = all): shows whether "
                         "the kernel's time follows the CU count or the board's power limit")
    ap.add_argument("--copy-calibration-mib", type=int, default=0,
                    help="also run one plain device copy of this many MiB (a known-size kernel to scale "
                         "the profiler's FETCH_SIZE / WRITE_SIZE counters against)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path has no multi-GPU part (run with --gpus 1)")
    if args.path in PATH_MAINS:
        print(json.dumps(PATH_MAINS[args.path](args)), flush=True)
        return
    if args.workload == "attn_scale":
        return attn_scale_main(args)

    import numpy as np

    from zdraw_amd import hip, host, workloads as wl

    L = hip.lib()
    ctx = host.Context.init()
    if args.cu_count > 0:
        ctx = ContextOnCus(L, ctx, args.cu_count)
    L.zdraw_hip_set_attention_variant(args.variant)
    w = wl.by_name(args.workload, seed=0)
    k_site = hip.K_PREPASS if args.k_site == "prepass" else hip.K_IN_TILE_LOAD
    staging = hip.F16 if args.staging == "f16" else 0
    res = wl.Resident(ctx, w, dtype=hip.BF16, k_site=k_site, bounded=not args.dynamic_max, staging=staging)

    # untimed: leave the idle power state, then the warm-up steps
    spun = spin_up(L, ctx, res, args.spinup_ms)
    timed_region(L, ctx, res, max(args.warmup, 1))
    wall, kern_ms = timed_region(L, ctx, res, args.steps)

    # one more launch with the clock probe on: the shader clock the kernel really ran at
    L.zdraw_hip_clock_probe(1)
    timed_region(L, ctx, res, 20)
    L.zdraw_hip_clock_probe(0)
    cyc = (C.c_uint64 * 4096)()
    ref = (C.c_uint64 * 4096)()
    nwg = L.zdraw_hip_clock_probe_read(cyc, ref, 4096)
    clock = None
    if nwg:
        cy = np.array(cyc[:nwg], dtype=np.float64)
        rt = np.array(ref[:nwg], dtype=np.float64)
        ghz = cy / np.maximum(rt, 1.0) * 0.1  # reference counter ticks at 100 MHz
        first = slice(0, min(nwg, 256))      # workgroups resident while every CU is busy
        clock = {
            "workgroups": int(nwg),
            "cycles_per_workgroup_median": float(np.median(cy)),
            "ghz_all_cus_busy_median": float(np.median(ghz[first])),
            "ghz_last_round_median": float(np.median(ghz[256:])) if nwg > 256 else None,
            "us_per_workgroup_all_cus_busy_median": float(np.median(rt[first]) / 100.0),
        }

    out = res.read_output()
    if not np.isfinite(out).all():
        raise RuntimeError("non-finite output")

    # the other K site, for the record (short, untimed by the driver's clock)
    other = "tile" if args.k_site == "prepass" else "prepass"
    res.ext.k_site = hip.K_IN_TILE_LOAD if other == "tile" else hip.K_PREPASS
    res.ext.staging = 0  # (the tile-load site stages bf16 only)
    timed_region(L, ctx, res, 20)
    o_wall, _ = timed_region(L, ctx, res, 100)

    res.release()
    # Short legs outside the driver-timed region, for the record: the running-maximum softmax on
    # the same workload (no score bound from the caller), and the other benchmark shapes.
    side = {}
    if not args.no_side_legs:
        dyn = side_leg(L, ctx, w, bounded=args.dynamic_max, staging=staging)  # the softmax form the timed region did not run
        side["dyn"] = dyn
        side["stg"] = side_leg(L, ctx, w, bounded=not args.dynamic_max, staging=0 if staging else hip.F16)  # the other staging type
        for name in ("klein_512_x4", "zimage_1024", "klein_edit_ragged"):
            if name == w.name:
                continue
            leg = side_leg(L, ctx, wl.by_name(name, seed=0), bounded=not args.dynamic_max,
                           steps=50 if name == "klein_edit_ragged" else 100)
            side[name] = {"value": leg["value"], "kernel_frac": leg["kernel_frac"], "ms_per_step": leg["ms_per_step"]}

    desc = (f"{w.name}: B={w.batch} H={w.heads} S={w.tokens} D=128 bf16, fused QK-RMSNorm + axial RoPE, "
            + ("no mask" if w.key_pad is None else "ragged key-padding mask"))
    flops = w.flops
    ms_per_step = wall * 1e3 / args.steps
    value = flops / (wall / args.steps) / 1e12
    achieved = flops / (kern_ms * 1e-3) / 1e12
    # HBM bytes per launch come from profiler counters, which this run does not collect: the
    # figure is the committed summary's (another run, another box) and is labelled as such
    traffic, traffic_source = None, None
    tpath = os.path.join(ROOT, "profiles", f"attn_fwd_{w.name}_traffic.json")
    if os.path.exists(tpath):
        traffic = json.load(open(tpath)).get("hbm_bytes_per_launch")
        traffic_source = f"profiles/attn_fwd_{w.name}_traffic.json (static: rocprofv3 counters of an earlier run)"
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
            "softmax": "running maximum" if args.dynamic_max else "bounded scores (QK-norm bound supplied by the caller)",
            "kernel_variant": args.variant,
            "qk_staging": args.staging,
            "pct_of_bf16_mfma_peak": 100.0 * value / PEAK_BF16_TFLOPS,
            f"tflops_with_k_site_{other}": flops / (o_wall / 100) / 1e12,
            "untimed_spinup_launches": spun,
            **({"cu_count": args.cu_count} if args.cu_count > 0 else {}),
            **({("tflops_bounded" if args.dynamic_max else "tflops_running_max"): side["dyn"]["value"],
                ("kernel_frac_bounded" if args.dynamic_max else "kernel_frac_running_max"): side["dyn"]["kernel_frac"],
                ("tflops_bf16_staging" if staging else "tflops_f16_staging"): side["stg"]["value"],
                ("kernel_frac_bf16_staging" if staging else "kernel_frac_f16_staging"): side["stg"]["kernel_frac"],
                "other_workloads": {k: v for k, v in side.items() if k not in ("dyn", "stg")}} if side else {}),
        },
        "roofline": {
            "bound": "mfma",
            "achieved": achieved,
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / PEAK_BF16_TFLOPS,
            "traffic": traffic,
            "traffic_source": traffic_source,
            "kernel": "attn_fwd_kernel",
            "kernel_ms": kern_ms,
            "shader_clock": clock,
        },
    }
    ctx.deinit()
    if not args.no_side_legs:
        line["config"]["other_paths"] = other_paths(args)
    if args.copy_calibration_mib:
        import torch

        n = args.copy_calibration_mib << 20
        src = torch.full((n,), 3, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)  # reads n bytes, writes n bytes
        torch.cuda.synchronize()
        line["config"]["copy_calibration_bytes"] = n
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(w)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
