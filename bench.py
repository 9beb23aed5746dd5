#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

Workload (benchmark config 1 at M=1): one decode pass over the seven 4-bit g64 projections of a
Llama-3-8B layer (q, k, v, o, gate, up, down).  One "step" = those seven GEMV launches on one
stream.  `--layers` distinct copies of the layer's weights (default 32, 3.9 GB) are resident in
HBM and steps rotate through them, so every launch streams its weights from HBM rather than
from the 256 MB last-level cache.  The headline value is weight bytes / time, the convention of
the reference's own GB/s figure.

Prints exactly one JSON line on stdout; progress and secondary figures go to stderr.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBPS = 8000.0            # MI355X published HBM3E bandwidth
LAYER_SHAPES = [("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
                ("gate", 14336, 4096), ("up", 14336, 4096), ("down", 4096, 14336)]
BITS, GROUP = 4, 64
MFMA_BF16_PEAK_TFLOPS = 2500.0    # MI355X published dense bf16 matrix-core peak
# HBM bytes per launch from the FETCH_SIZE and WRITE_SIZE counters, each scaled by what the same counter reads for a
# plain copy of the same size (profiles/gemv_rows_q4_g64_gate_up_pmc_and_hbm_traffic.md).  Measured offline with the
# profiler: the figure only holds for the kernel and launch shape it was measured on, so it is keyed by both and the
# line carries null when the library picks anything else.
# The same for the M = 2048 gate launch of the prefill GEMM (keyed by kernel and grid; FETCH_SIZE 180 400 and WRITE_SIZE
# 69 080 per dispatch against 16 140 and 32 260 for a copy of 33 030 144 bytes: 369 MB read past the L2s, most of it the
# activations once per round of column tiles and served by the last-level cache, and 71 MB written;
# profiles/qgemm_wide_q4_g64_prefill_m2048_kernel_trace_pmc.md).
PREFILL_TRAFFIC_BYTES = {("qgemm_wide_q4_g64", 448): 369_200_000 + 70_700_000}
TRAFFIC_BYTES = {("gemv_rows_q4_g64", "gate_up", 3584, 256): 66171661 + 114688, ("gemv_rows_q4_g64", "gate", 1792, 256): 33159518 + 57344}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def weight_bytes(n, k, bits=BITS, group=GROUP):
    return n * (k // group) * (4 + group * bits // 8)


def time_region(ctx, fn, reps, stream=0):
    """Average milliseconds per call of fn over `reps` calls, HIP events on the launch stream."""
    e0, e1 = ctx.event_create(), ctx.event_create()
    ctx.event_record(e0, stream)
    for i in range(reps):
        fn(i)
    ctx.event_record(e1, stream)
    ctx.event_synchronize(e1)
    ms = ctx.event_elapsed_ms(e0, e1) / reps
    ctx.event_destroy(e0); ctx.event_destroy(e1)
    return ms


def steady_region(ctx, fn, reps, stream=0, most=16, tol=0.01):
    """Sustained-load figure of a compute-bound launch: samples of `reps` calls, back to back, until one is within
    `tol` of the one before (at least four, at most `most`).  After idle the part needs some tens of milliseconds of
    matrix work before its clocks settle: the first 24 M = 2048 prefill launches take 227 us each, later ones 194 us.
    Returns (steady ms per call, first sample's ms per call, samples taken)."""
    first = prev = time_region(ctx, fn, reps, stream)
    taken = 1
    while taken < most:
        ms = time_region(ctx, fn, reps, stream)
        taken += 1
        settled = taken >= 4 and abs(ms - prev) <= tol * prev
        prev = ms
        if settled:
            break
    return prev, first, taken


def cpu_baseline(seconds: float):
    """The reference's loop nest (row -> block -> k, fp32 accumulate) on the host cores, timed on
    benchmark config 0 (q4 g64, 2048 -> 8192, M=1) for a bounded number of passes."""
    import kat
    import oracle
    n, k = 8192, 2048
    words, s, z = oracle.quantize_affine(kat.seeded_weights(11, n, k), BITS, GROUP, oracle.BF16)
    x = oracle.bf16_to_f32(oracle.bf16_from_f32(kat.seeded_activations(12, 1, k))).reshape(1, k)
    host_cores = os.cpu_count() or 1
    cores = min(host_cores, 16)           # the GPU box gives one job 16 cores' worth of CPU time, whatever it reports
    oracle.qgemm_planes_ref_f32(BITS, GROUP, words, s, z, oracle.BF16, x, n, k, threads=cores)  # warm-up
    passes, t0 = 0, time.perf_counter()
    while True:
        oracle.qgemm_planes_ref_f32(BITS, GROUP, words, s, z, oracle.BF16, x, n, k, threads=cores)
        passes += 1
        dt = time.perf_counter() - t0
        if dt >= seconds or passes >= 20000:
            break
    gbps = weight_bytes(n, k) * passes / dt / 1e9
    return {"value": round(gbps, 4), "unit": "GB/s", "cores": cores, "host_cores_reported": host_cores, "kind": "port",
            "sample": f"{passes} passes of config 0 (q4 g64 2048->8192, M=1, 9437184 weight bytes each) "
                      f"in {dt:.1f} s, rows split over {cores} pthreads (the host reports {host_cores} cores; "
                      f"a job's CPU share on the GPU box is 16)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=320,
                    help="timed steps; at least 256 are timed whatever is asked (rounded up to whole passes over the layer copies)")
    ap.add_argument("--warmup", type=int, default=32, help="untimed warm-up steps; at least 32 are run")
    ap.add_argument("--layers", type=int, default=32, help="distinct weight copies resident in HBM")
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--skip-parity", action="store_true")
    ap.add_argument("--no-prefill", action="store_true", help="skip the secondary prefill-GEMM figure")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the secondary per-launch figures of benchmark configs 0, 2 and 4")
    ap.add_argument("--no-batch-sweep", action="store_true", help="skip the secondary M = 1 to 64 figures")
    ap.add_argument("--no-f16-step", action="store_true", help="skip the layer step with f16 activations")
    ap.add_argument("--all-formats", action="store_true",
                    help="add 4096->14336 at M = 1 and 8 for every registered format, planes and blocks in place (half a minute)")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (one process, one device); "
                 f"--gpus {a.gpus} is not supported")

    import kat
    import oracle
    from __graft_entry__ import load_package
    pkg = load_package()
    ctx = pkg.Context(0)
    info = ctx.device_info()
    log(f"device: {info.name.decode()} {info.arch.decode()} CUs={info.compute_units}")
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(BITS, GROUP)

    # ---- synthetic layer: W ~ N(0, 0.02^2) quantised per group, bf16 scale/bias planes
    host = {}
    for i, (name, n, k) in enumerate(LAYER_SHAPES):
        t0 = time.perf_counter()
        words, s, z = oracle.quantize_affine(kat.seeded_weights(1000 + i, n, k), BITS, GROUP, oracle.BF16)
        host[name] = (words, s, z)
        log(f"  synthesised {name} {k}->{n} in {time.perf_counter() - t0:.1f}s")
    xs = {k: oracle.bf16_to_f32(oracle.bf16_from_f32(kat.seeded_activations(77 + k, 1, k))).reshape(1, k)
          for k in (4096, 14336)}
    xdev = {k: ctx.upload(oracle.bf16_from_f32(v)) for k, v in xs.items()}
    ydev = {name: ctx.alloc(n * 2) for name, n, _ in LAYER_SHAPES}

    layers = []
    for _ in range(a.layers):
        layers.append({name: ctx.weight_prepare_mlx(fmt, *host[name], pkg.BF16, pkg.LAYOUT_PLANES)
                       for name, _, _ in LAYER_SHAPES})
    layer_bytes = sum(weight_bytes(n, k) for _, n, k in LAYER_SHAPES)
    log(f"resident: {a.layers} layers x {layer_bytes} B = {a.layers * layer_bytes / 1e9:.2f} GB")

    stream = ctx.stream_create()
    # The headline must not depend on what the driver passes: at least 256 timed steps (1024 launches of the 4-launch
    # schedule) after at least 32 warm-up steps, in whole passes over the resident layer copies.
    steps = max(a.steps, 256)
    steps = (steps + a.layers - 1) // a.layers * a.layers
    warmup = max(a.warmup, 32)

    # ---- parity gate: no number is reported from a run whose outputs were not verified
    if not a.skip_parity:
        for name, n, k in LAYER_SHAPES:
            words, s, z = host[name]
            wq = oracle.dequant_planes_f32(BITS, GROUP, n, k, words, s, z, oracle.BF16)
            want = oracle.gemm_f64(wq, xs[k])[0]
            y32 = ctx.alloc(n * 4)
            ctx.qgemv(layers[-1][name], xdev[k], pkg.BF16, y32, pkg.F32, 1)
            ctx.synchronize()
            got = y32.download(np.float32)
            rel = float(np.linalg.norm(got - want) / np.linalg.norm(want))
            mx = float(np.max(np.abs(got - want)))
            y32.free()
            if not (rel <= 1e-3 and mx <= 2e-2):
                sys.exit(f"bench.py: parity gate failed on {name}: rel-L2 {rel:.3e} max-abs {mx:.3e}")
            log(f"  parity {name}: rel-L2 {rel:.2e} max-abs {mx:.2e}")

    # ---- the decode plans, built once, replayed from C -----------------------------------------
    #   "7-launch": one launch per projection, the reference's decode schedule
    #   "4-launch": q+k+v and gate+up share their input and run as one launch each
    def build_plan(fused, xd=None, xt=None):
        xd = xdev if xd is None else xd
        xt = pkg.BF16 if xt is None else xt
        plan = pkg.DispatchPlan(ctx)
        for li, L in enumerate(layers):
            def lin(name, k):
                plan.add_linear(L[name], xd[k], xt, ydev[name], xt, 1, layer_index=li,
                                tensor_name=f"layers.{li}.{name}_proj.weight")
            if fused:
                plan.add_batched_linear([L["q"], L["k"], L["v"]], xd[4096], xt,
                                        [ydev["q"], ydev["k"], ydev["v"]], xt, 1, layer_index=li,
                                        tensor_name=f"layers.{li}.qkv_proj.weight")
                lin("o", 4096)
                plan.add_batched_linear([L["gate"], L["up"]], xd[4096], xt, [ydev["gate"], ydev["up"]],
                                        xt, 1, layer_index=li, tensor_name=f"layers.{li}.gate_up_proj.weight")
                lin("down", 14336)
            else:
                for name, n, k in LAYER_SHAPES:
                    lin(name, k)
        return plan

    results, spreads = {}, {}
    group = 8                                              # steps per event pair of the spread measurement
    for label, fused in (("7-launch", False), ("4-launch", True)):
        plan = build_plan(fused)
        per_layer = len(plan) // a.layers

        def step(i, plan=plan, per_layer=per_layer):
            plan.encode(stream, (i % a.layers) * per_layer, per_layer)

        for i in range(warmup):
            step(i)
        ctx.synchronize(stream)
        ms = time_region(ctx, step, steps, stream)
        ctx.synchronize(stream)
        results[label + " stream"] = ms
        log(f"{label} stream replay: {ms * 1e3:.2f} us/step over {steps} steps, {layer_bytes / (ms * 1e-3) / 1e9:.1f} GB/s")
        # spread: one HIP event pair around every `group` consecutive steps (a pair costs 2-3 us, so 0.3 us per step)
        per_group = []
        ea, eb = ctx.event_create(), ctx.event_create()
        for g in range(steps // group):
            ctx.event_record(ea, stream)
            for i in range(group):
                step(g * group + i)
            ctx.event_record(eb, stream)
            ctx.event_synchronize(eb)
            per_group.append(ctx.event_elapsed_ms(ea, eb) / group)
        ctx.event_destroy(ea); ctx.event_destroy(eb)
        per_group.sort()
        n_g = len(per_group)
        spreads[label + " stream"] = {"median_us": round(per_group[n_g // 2] * 1e3, 2), "p10_us": round(per_group[n_g // 10] * 1e3, 2),
                                      "p90_us": round(per_group[n_g * 9 // 10] * 1e3, 2), "samples": n_g, "steps_per_sample": group}
        # the same plan captured once into a HIP graph (one launch per pass over all layers)
        plan.graph_build(stream)
        for _ in range(2):
            plan.graph_launch(stream)
        ctx.synchronize(stream)
        passes = steps // a.layers
        ms_pass = time_region(ctx, lambda i, plan=plan: plan.graph_launch(stream), passes, stream)
        ctx.synchronize(stream)
        results[label + " hip-graph"] = ms_pass / a.layers
        per_pass = []
        ea, eb = ctx.event_create(), ctx.event_create()
        for g in range(max(passes, 16)):
            ctx.event_record(ea, stream)
            plan.graph_launch(stream)
            ctx.event_record(eb, stream)
            ctx.event_synchronize(eb)
            per_pass.append(ctx.event_elapsed_ms(ea, eb) / a.layers)
        ctx.event_destroy(ea); ctx.event_destroy(eb)
        per_pass.sort()
        n_p = len(per_pass)
        spreads[label + " hip-graph"] = {"median_us": round(per_pass[n_p // 2] * 1e3, 2), "p10_us": round(per_pass[n_p // 10] * 1e3, 2),
                                         "p90_us": round(per_pass[n_p * 9 // 10] * 1e3, 2), "samples": n_p, "steps_per_sample": a.layers}
        log(f"{label} graph replay:  {ms_pass / a.layers * 1e3:.2f} us/step, "
            f"{layer_bytes / (ms_pass / a.layers * 1e-3) / 1e9:.1f} GB/s; spread {spreads[label + ' hip-graph']}")
        plan.destroy()
    # the reference decodes in f16: the same 4-launch step with f16 activations and outputs, graph replay
    f16_step = None
    if not a.no_f16_step:
        x16dev = {k: ctx.upload(v.astype(np.float16).view(np.uint16)) for k, v in xs.items()}
        plan16 = build_plan(True, x16dev, pkg.F16)
        f16_kernel = plan16.step(2)[0].device_kernel
        plan16.graph_build(stream)
        for _ in range(2):
            plan16.graph_launch(stream)
        ctx.synchronize(stream)
        ms16 = time_region(ctx, lambda i: plan16.graph_launch(stream), max(1, steps // a.layers), stream) / a.layers
        ctx.synchronize(stream)
        plan16.destroy()
        f16_step = {"us_per_step": round(ms16 * 1e3, 2), "GBps": round(layer_bytes / (ms16 * 1e-3) / 1e9, 1),
                    "gate_up_kernel": f16_kernel, "vs_bf16": round(ms16 / results["4-launch hip-graph"], 3)}
        log(f"4-launch graph replay with f16 activations: {f16_step}")
    mode = min(results, key=results.get)
    ms_step = results[mode]
    value = layer_bytes / (ms_step * 1e-3) / 1e9
    replay_gbps = {k: round(layer_bytes / (v * 1e-3) / 1e9, 1) for k, v in results.items()}

    # ---- per-launch durations over rotating copies (HIP events on the launch stream) ------------
    per_shape = {}
    probes = [("gate", ["gate"], 4096), ("gate_up", ["gate", "up"], 4096), ("down", ["down"], 14336),
              ("q", ["q"], 4096), ("qkv", ["q", "k", "v"], 4096), ("k", ["k"], 4096)]
    dims = {name: (n, k) for name, n, k in LAYER_SHAPES}
    for label, names, k in probes:
        p1 = pkg.DispatchPlan(ctx)
        for L in layers:
            if len(names) == 1:
                p1.add_linear(L[names[0]], xdev[k], pkg.BF16, ydev[names[0]], pkg.BF16, 1)
            else:
                p1.add_batched_linear([L[n] for n in names], xdev[k], pkg.BF16, [ydev[n] for n in names], pkg.BF16, 1)
        p1.encode(stream)
        ctx.synchronize(stream)
        reps = max(1, max(steps, 8 * a.layers) // a.layers)      # at least 256 launches per figure
        ms = time_region(ctx, lambda i: p1.encode(stream), reps, stream) / a.layers
        # the same launches replayed from a HIP graph: for the small projections the host cannot issue stream
        # launches as fast as the GPU retires them, so the stream figure measures the host there
        p1.graph_build(stream)
        p1.graph_launch(stream)
        ctx.synchronize(stream)
        ms_graph = time_region(ctx, lambda i: p1.graph_launch(stream), reps, stream) / a.layers
        ms = min(ms, ms_graph)
        nbytes = sum(weight_bytes(*dims[n]) for n in names)
        per_shape[label] = {"us": round(ms * 1e3, 3), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1), "weight_bytes": nbytes}
        # spread of single launches: one HIP event pair around each of 192 launches over the rotating copies
        # (an event pair adds two to three microseconds to what it brackets; "us" above is the back-to-back figure)
        singles = []
        ea, eb = ctx.event_create(), ctx.event_create()
        for i in range(192):
            ctx.event_record(ea, stream)
            p1.encode(stream, i % a.layers, 1)
            ctx.event_record(eb, stream)
            ctx.event_synchronize(eb)
            singles.append(ctx.event_elapsed_ms(ea, eb) * 1e3)
        singles.sort()
        per_shape[label]["single_launch_us"] = {"median": round(singles[96], 2), "p10": round(singles[19], 2),
                                                "p90": round(singles[172], 2)}
        log(f"  {label:8s}: {ms * 1e3:.2f} us/launch, {per_shape[label]['GBps']} GB/s; single launches "
            f"{per_shape[label]['single_launch_us']}")
        p1.destroy()
    # ---- secondary: the same layer step at M = 1 to 64 activation rows (benchmark config 1), on
    # the split-plane layout and on the matrix-core tile layout (4-launch schedule, stream replay)
    batch_sweep = None
    if not a.no_batch_sweep:
        batch_sweep = {}
        n_t16 = min(a.layers, 8)                       # 8 x 123 MB: well past the 256 MB last-level cache
        for lname, layout, pool in (("planes", pkg.LAYOUT_PLANES, layers[:n_t16]), ("tile16", pkg.LAYOUT_TILE16, None)):
            if pool is None:
                pool = [{name: ctx.weight_prepare_mlx(fmt, *host[name], pkg.BF16, layout) for name, _, _ in LAYER_SHAPES}
                        for _ in range(n_t16)]
            batch_sweep[lname] = {}
            # both layouts take up to 16 rows a launch of the decode kernels; 32 and 64 rows on the planes run on the
            # streamed-weight matrix-core kernel, on the records on the tiled prefill kernel
            for m in (1, 2, 4, 8, 16, 32, 64):
                xm = {k: ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(900 + m, m, k))) for k in (4096, 14336)}   # N(0,1)
                ym = {name: ctx.alloc(m * n * 2) for name, n, _ in LAYER_SHAPES}
                pl = pkg.DispatchPlan(ctx)
                for L in pool:
                    pl.add_batched_linear([L["q"], L["k"], L["v"]], xm[4096], pkg.BF16, [ym["q"], ym["k"], ym["v"]],
                                          pkg.BF16, m)
                    pl.add_linear(L["o"], xm[4096], pkg.BF16, ym["o"], pkg.BF16, m)
                    pl.add_batched_linear([L["gate"], L["up"]], xm[4096], pkg.BF16, [ym["gate"], ym["up"]], pkg.BF16, m)
                    pl.add_linear(L["down"], xm[14336], pkg.BF16, ym["down"], pkg.BF16, m)
                pl.encode(stream)
                ctx.synchronize(stream)
                ms = time_region(ctx, lambda i: pl.encode(stream), 32, stream) / len(pool)     # 256 steps
                batch_sweep[lname][f"M={m}"] = {"us_per_step": round(ms * 1e3, 2),
                                                "GBps": round(layer_bytes / (ms * 1e-3) / 1e9, 1)}
                pl.destroy()
                for b in list(xm.values()) + list(ym.values()):
                    b.free()
            log(f"  batch sweep {lname} (N(0,1) activations): " + ", ".join(f"{k} {v['us_per_step']} us" for k, v in batch_sweep[lname].items()))
            if True:
                # the reference's decode type: the small-batch kernels stage an f16 row as two bf16 rows; from nine rows
                # the planes run the streamed-weight kernel with f16 weights
                key16 = lname + "_f16_activations"
                batch_sweep[key16] = {}
                for m in ((1, 8) if lname == "tile16" else (8, 32, 64)):
                    xm = {k: ctx.upload(kat.seeded_activations(950 + m, m, k).astype(np.float16).view(np.uint16)) for k in (4096, 14336)}
                    ym = {name: ctx.alloc(m * n * 2) for name, n, _ in LAYER_SHAPES}
                    pl = pkg.DispatchPlan(ctx)
                    for L in pool:
                        pl.add_batched_linear([L["q"], L["k"], L["v"]], xm[4096], pkg.F16, [ym["q"], ym["k"], ym["v"]], pkg.F16, m)
                        pl.add_linear(L["o"], xm[4096], pkg.F16, ym["o"], pkg.F16, m)
                        pl.add_batched_linear([L["gate"], L["up"]], xm[4096], pkg.F16, [ym["gate"], ym["up"]], pkg.F16, m)
                        pl.add_linear(L["down"], xm[14336], pkg.F16, ym["down"], pkg.F16, m)
                    pl.encode(stream)
                    ctx.synchronize(stream)
                    ms = time_region(ctx, lambda i: pl.encode(stream), 32, stream) / len(pool)
                    batch_sweep[key16][f"M={m}"] = {
                        "us_per_step": round(ms * 1e3, 2), "GBps": round(layer_bytes / (ms * 1e-3) / 1e9, 1),
                        "kernel": pl.step(2)[0].device_kernel}
                    pl.destroy()
                    for b in list(xm.values()) + list(ym.values()):
                        b.free()
                log(f"  batch sweep {lname}, f16 activations: {batch_sweep[key16]}")
            if lname == "tile16":
                for L in pool:
                    for w in L.values():
                        w.destroy()

    # the dominant kernel of the reported schedule: the fused gate+up launch, or the gate launch
    dom = "gate_up" if mode.startswith("4-launch") else "gate"
    dom_bytes = per_shape[dom]["weight_bytes"]
    achieved = per_shape[dom]["GBps"]
    # the kernel and launch shape of that launch, from the plan record of the step that ran it
    pd = pkg.DispatchPlan(ctx)
    if dom == "gate_up":
        pd.add_batched_linear([layers[0]["gate"], layers[0]["up"]], xdev[4096], pkg.BF16, [ydev["gate"], ydev["up"]], pkg.BF16, 1)
    else:
        pd.add_linear(layers[0]["gate"], xdev[4096], pkg.BF16, ydev["gate"], pkg.BF16, 1)
    dom_rec = pd.step(0)[0]
    dom_kernel, dom_grid, dom_block = dom_rec.device_kernel, int(dom_rec.grid[0]), int(dom_rec.block[0])
    pd.destroy()
    traffic = TRAFFIC_BYTES.get((dom_kernel, dom, dom_grid, dom_block))

    # ---- plain copy of the gate tensor's size: the calibration launch for the HBM counters ------
    gate_bytes = weight_bytes(14336, 4096)
    csrc, cdst = ctx.alloc(gate_bytes), ctx.alloc(gate_bytes)
    ctx.fill(csrc, 0x01020304, stream)
    ctx.copy(cdst, csrc, gate_bytes, stream)
    ctx.synchronize(stream)
    ms_copy = time_region(ctx, lambda i: ctx.copy(cdst, csrc, gate_bytes, stream), 8, stream)
    log(f"  copy  {gate_bytes} B: {ms_copy * 1e3:.2f} us/launch, {2 * gate_bytes / (ms_copy * 1e-3) / 1e9:.1f} GB/s "
        "read+write")

    # ---- secondary: one launch each of benchmark config 0 (2048->8192), config 2 (4096->14336 at 8, 6, 3 and 2 bits)
    # and config 4 (LM head 2048->65536 fused with argmax), over rotating copies of more than 512 MB in total
    other = None
    if not a.no_other_configs:
        other = {}
        P, S = pkg.LAYOUT_PLANES, pkg.LAYOUT_STAF_BLOCKS
        cases = [("config0 q4g64 2048->8192", 4, 64, 8192, 2048, False, P), ("config2 q8g32 4096->14336", 8, 32, 14336, 4096, False, P),
                 ("config2 q6g64 4096->14336", 6, 64, 14336, 4096, False, P), ("config2 q3g64 4096->14336", 3, 64, 14336, 4096, False, P),
                 ("config2 q2g64 4096->14336", 2, 64, 14336, 4096, False, P),
                 ("config4 q4g64 lm head 2048->65536 + argmax", 4, 64, 65536, 2048, True, P),
                 # the same gate / down projections left in the reference's interleaved blocks (no re-layout at load)
                 ("config1 gate q4g64 4096->14336, STAF blocks in place", 4, 64, 14336, 4096, False, S),
                 ("config1 down q4g64 14336->4096, STAF blocks in place", 4, 64, 4096, 14336, False, S)]
        for ci, (label, bits, group, n, k, head, layout) in enumerate(cases):
            f2 = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
            words, s, z = oracle.quantize_affine(kat.seeded_weights(3000 + ci, n, k), bits, group, oracle.BF16)
            nbytes = n * (k // group) * (4 + group * bits // 8)
            copies = max(2, min(64, int(5.4e8 // nbytes) + 1))
            ws = [ctx.weight_prepare_mlx(f2, words, s, z, pkg.BF16, layout) for _ in range(copies)]
            x1 = oracle.bf16_to_f32(oracle.bf16_from_f32(kat.seeded_activations(3100 + ci, 1, k))).reshape(1, k)
            xd1 = ctx.upload(oracle.bf16_from_f32(x1))
            yd1, logits, tok = ctx.alloc(n * 2), ctx.alloc(n * 4), ctx.alloc(16)
            pl = pkg.DispatchPlan(ctx)
            for w in ws:
                if head:
                    pl.add_output_head(w, xd1, pkg.BF16, logits, tok)
                else:
                    pl.add_linear(w, xd1, pkg.BF16, yd1, pkg.BF16, 1)
            pl.encode(stream)
            ctx.synchronize(stream)
            if not a.skip_parity:                       # the launch just timed is checked before its number is used
                wq = oracle.dequant_planes_f32(bits, group, n, k, words, s, z, oracle.BF16)
                want = oracle.gemm_f64(wq, x1)[0]
                if head:
                    got = logits.download(np.float32)
                    t = int(tok.download(np.int32)[0])
                    if t != oracle.argmax_lowest(got):
                        sys.exit(f"bench.py: {label}: token {t} is not the lowest-index argmax of the logits")
                    # and against the CPU reference logits: only a near-tie between the top two can differ
                    top2 = np.sort(want)[-2:]
                    head_check = {"token": t, "token_of_cpu_reference_logits": int(np.argmax(want)),
                                  "top2_gap": float(top2[1] - top2[0])}
                    if head_check["token"] != head_check["token_of_cpu_reference_logits"] and head_check["top2_gap"] > 1e-3:
                        sys.exit(f"bench.py: {label}: token {t} differs from the CPU reference's {head_check}")
                else:
                    got = oracle.bf16_to_f32(yd1.download(np.uint16))
                    want = oracle.bf16_to_f32(oracle.bf16_from_f32(want.astype(np.float32)))
                rel = float(np.linalg.norm(got - want) / np.linalg.norm(want))
                if rel > (1e-3 if head else 4e-3):      # bf16 outputs carry their own rounding
                    sys.exit(f"bench.py: parity gate failed on {label}: rel-L2 {rel:.3e}")
            ms = time_region(ctx, lambda i: pl.encode(stream), 6, stream) / copies
            other[label] = {"us": round(ms * 1e3, 2), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1), "weight_bytes": nbytes}
            if head and not a.skip_parity:
                other[label]["argmax_parity"] = head_check
            if bits == 8:                                # the same matrix at eight activation rows, as dispatched
                xb = ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(3200 + ci, 8, k)))
                yb = ctx.alloc(8 * n * 2)
                for i in range(copies):
                    ctx.qgemm(ws[i], xb, pkg.BF16, yb, pkg.BF16, 8, 0, 0, 0, stream)
                ctx.synchronize(stream)
                ms8 = time_region(ctx, lambda i: ctx.qgemm(ws[i % copies], xb, pkg.BF16, yb, pkg.BF16, 8, 0, 0, 0, stream),
                                  6 * copies, stream)
                other[label]["M=8"] = {"us": round(ms8 * 1e3, 2), "GBps": round(nbytes / (ms8 * 1e-3) / 1e9, 1),
                                       "kernel": ws[0].plan_decode_step(8).device_kernel}
                xb.free(); yb.free()
            log(f"  {label}: {other[label]['us']} us/launch, {other[label]['GBps']} GB/s" +
                (f"; M=8 {other[label]['M=8']}" if "M=8" in other[label] else ""))
            pl.destroy()
            for w in ws:
                w.destroy()
            for b in (xd1, yd1, logits, tok):
                b.free()

    # ---- on request: every registered format at the gate shape, one and eight rows, both decode layouts of the format
    all_formats = None
    if a.all_formats:
        all_formats = {}
        n, k = 14336, 4096
        for bits, group in kat.ALL_FORMATS:
            f2 = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
            words, s, z = oracle.quantize_affine(kat.seeded_weights(3300 + bits + group, n, k), bits, group, oracle.BF16)
            nbytes = n * (k // group) * (4 + group * bits // 8)
            entry = {"weight_bytes": nbytes}
            for lname, layout in (("planes", pkg.LAYOUT_PLANES), ("staf_blocks", pkg.LAYOUT_STAF_BLOCKS)):
                ws = [ctx.weight_prepare_mlx(f2, words, s, z, pkg.BF16, layout) for _ in range(8)]
                for m in (1, 8):
                    xb = ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(3400 + m, m, k)))
                    yb = ctx.alloc(m * n * 2)
                    for w in ws:
                        ctx.qgemv(w, xb, pkg.BF16, yb, pkg.BF16, m, 0, 0, 0, stream)
                    ctx.synchronize(stream)
                    ms = time_region(ctx, lambda i: ctx.qgemv(ws[i % 8], xb, pkg.BF16, yb, pkg.BF16, m, 0, 0, 0, stream), 32, stream)
                    entry[f"{lname} M={m}"] = {"us": round(ms * 1e3, 2), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                                               "kernel": ws[0].plan_decode_step(m).device_kernel}
                    xb.free(); yb.free()
                for w in ws:
                    w.destroy()
            all_formats[f"q{bits} g{group}"] = entry
            log(f"  q{bits} g{group}: " + ", ".join(f"{k2} {v['us']} us ({v['kernel']})" for k2, v in entry.items() if isinstance(v, dict)))

    # ---- what HBM delivers to one launch of the dominant launch's size: a kernel that only reads that many bytes
    # (cold: eight buffers in rotation, as the weights of the layer copies are)
    probe_copies = 8
    pbuf = ctx.alloc(probe_copies * dom_bytes)
    ctx.fill(pbuf, 0x01020304, stream)
    ctx.synchronize(stream)
    ms_read = time_region(ctx, lambda i: ctx.read_probe(pbuf.ptr + (i % probe_copies) * dom_bytes, dom_bytes, stream),
                          64, stream)
    stream_read = {"bytes": dom_bytes, "us": round(ms_read * 1e3, 2), "GBps": round(dom_bytes / (ms_read * 1e-3) / 1e9, 1)}
    log(f"  read-only launch of {dom_bytes} B: {stream_read['us']} us, {stream_read['GBps']} GB/s "
        f"(the {dom} launch reaches {achieved / stream_read['GBps'] * 100:.0f} % of it)")
    pbuf.free()

    # ---- secondary: the same 4-launch step over weights left in the reference's interleaved STAF blocks (what a
    # model.staf payload wrapped with no copy gives): 8 resident layer copies (1 GB), stream replay
    staf_step = None
    if not a.no_other_configs:
        saved, layers = layers, []
        for _ in range(8):
            layers.append({name: ctx.weight_prepare_mlx(fmt, *host[name], pkg.BF16, pkg.LAYOUT_STAF_BLOCKS)
                           for name, _, _ in LAYER_SHAPES})
        if not a.skip_parity:
            name, n, k = LAYER_SHAPES[-1]
            words, s_, z_ = host[name]
            want = oracle.gemm_f64(oracle.dequant_planes_f32(BITS, GROUP, n, k, words, s_, z_, oracle.BF16), xs[k])[0]
            y32 = ctx.alloc(n * 4)
            ctx.qgemv(layers[-1][name], xdev[k], pkg.BF16, y32, pkg.F32, 1)
            ctx.synchronize()
            got = y32.download(np.float32)
            y32.free()
            rel = float(np.linalg.norm(got - want) / np.linalg.norm(want))
            if rel > 1e-3:
                sys.exit(f"bench.py: parity gate failed on the in-place STAF {name} projection: rel-L2 {rel:.3e}")
        plan = build_plan(True)
        per_layer = len(plan) // len(layers)
        for i in range(16):
            plan.encode(stream, (i % 8) * per_layer, per_layer)
        ctx.synchronize(stream)
        ms = time_region(ctx, lambda i: plan.encode(stream, (i % 8) * per_layer, per_layer), 160, stream)
        ctx.synchronize(stream)
        staf_step = {"us_per_step": round(ms * 1e3, 2), "GBps": round(layer_bytes / (ms * 1e-3) / 1e9, 1),
                     "kernel": plan.step(per_layer - 1)[0].device_kernel}
        log(f"4-launch step on STAF blocks in place: {staf_step['us_per_step']} us/step, {staf_step['GBps']} GB/s")
        plan.destroy()
        # a batch of sequences on the blocks in place: the layer step at 8 and 32 rows (N(0,1) activations), as dispatched
        staf_step["batch"] = {}
        for m in (8, 32):
            xm = {k: ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(970 + m, m, k))) for k in (4096, 14336)}
            ym = {name: ctx.alloc(m * n * 2) for name, n, _ in LAYER_SHAPES}
            pl = pkg.DispatchPlan(ctx)
            for L in layers:
                pl.add_batched_linear([L["q"], L["k"], L["v"]], xm[4096], pkg.BF16, [ym["q"], ym["k"], ym["v"]], pkg.BF16, m)
                pl.add_linear(L["o"], xm[4096], pkg.BF16, ym["o"], pkg.BF16, m)
                pl.add_batched_linear([L["gate"], L["up"]], xm[4096], pkg.BF16, [ym["gate"], ym["up"]], pkg.BF16, m)
                pl.add_linear(L["down"], xm[14336], pkg.BF16, ym["down"], pkg.BF16, m)
            pl.encode(stream)
            ctx.synchronize(stream)
            ms_b = time_region(ctx, lambda i: pl.encode(stream), 32, stream) / len(layers)
            staf_step["batch"][f"M={m}"] = {"us_per_step": round(ms_b * 1e3, 2), "GBps": round(layer_bytes / (ms_b * 1e-3) / 1e9, 1),
                                            "down_kernel": layers[0]["down"].plan_prefill_steps(m, 14336)[0].device_kernel}
            pl.destroy()
            for b in list(xm.values()) + list(ym.values()):
                b.free()
        log(f"  batches on the blocks in place: {staf_step['batch']}")
        if not a.no_prefill:
            # prefill straight from the blocks: the gate projection over four rotating copies, as dispatched
            staf_step["prefill_gate_4096_14336"] = {}
            wts = [L["gate"] for L in layers[:4]]
            for mm in (64, 512, 2048):
                xb = ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(500 + mm, mm, 4096)))
                yb = ctx.alloc(mm * 14336 * 2)
                for i in range(4):
                    ctx.qgemm(wts[i], xb, pkg.BF16, yb, pkg.BF16, mm, 0, 0, 0, stream)
                ctx.synchronize(stream)
                ms, _, _ = steady_region(ctx, lambda i: ctx.qgemm(wts[i % 4], xb, pkg.BF16, yb, pkg.BF16, mm, 0, 0, 0, stream), 24, stream)
                staf_step["prefill_gate_4096_14336"][f"M={mm}"] = {
                    "us": round(ms * 1e3, 1), "TFLOPs": round(2.0 * mm * 14336 * 4096 / (ms * 1e-3) / 1e12, 1),
                    "route": " + ".join(st.device_kernel for st in wts[0].plan_prefill_steps(mm, 4096))}
                xb.free(); yb.free()
            log(f"  prefill from the blocks (N(0,1)): {staf_step['prefill_gate_4096_14336']}")
        for L in layers:
            for w in L.values():
                w.destroy()
        layers = saved

    # ---- secondary: the rows either side of the projections (embedding gather, container load, KV cache), one
    # figure each; HBM-bound byte movers, bytes = what the launch must read plus what it must write
    next_rows = None
    if not a.no_other_configs:
        import tempfile
        next_rows = {}
        rng = np.random.default_rng(11)
        table = layers[0]["gate"]                              # 14336 x 4096 q4 g64 as a vocabulary table
        seq = 2048
        ids = ctx.upload(rng.integers(0, 14336, seq).astype(np.int32))
        emb = ctx.alloc(seq * 4096 * 2)
        ctx.embedding_lookup(table, ids, seq, emb, pkg.BF16, 0, None, stream)
        ctx.synchronize(stream)
        ms = time_region(ctx, lambda i: ctx.embedding_lookup(table, ids, seq, emb, pkg.BF16, 0, None, stream), 20, stream)
        moved = seq * (4096 // 64) * 36 + seq * 4096 * 2
        next_rows["embedding gather 2048 tokens x 4096, q4 g64 -> bf16"] = {
            "us": round(ms * 1e3, 2), "GBps": round(moved / (ms * 1e-3) / 1e9, 1), "bytes": moved}
        ids.free(); emb.free()
        spec = pkg.KVCacheSpecification(0x10, pkg.KV_SEQUENCE_MAJOR, 8, 128, 4096)
        cache = ctx.alloc(spec.bytes_per_layer)
        rows = ctx.upload(oracle.bf16_from_f32(rng.standard_normal((seq, 1024)).astype(np.float32)))
        back = ctx.alloc(seq * 1024 * 2)
        for label, fn, count in (("KV cache write q8 g32, 2048 positions x 8 heads x 128", lambda i: ctx.kv_cache_write(spec, cache, rows, pkg.BF16, 0, seq, 0, stream), seq),
                                 ("KV cache read q8 g32, 2048 positions x 8 heads x 128", lambda i: ctx.kv_cache_read(spec, cache, back, pkg.BF16, 0, seq, 0, stream), seq),
                                 ("KV cache append q8 g32, 1 position", lambda i: ctx.kv_cache_write(spec, cache, rows, pkg.BF16, seq, 1, 0, stream), 1)):
            fn(0)
            ctx.synchronize(stream)
            ms = time_region(ctx, fn, 20, stream)
            moved = count * 1024 * 2 + count * 8 * (128 // 32) * 36
            next_rows[label] = {"us": round(ms * 1e3, 2), "GBps": round(moved / (ms * 1e-3) / 1e9, 1), "bytes": moved}
        for b in (cache, rows, back):
            b.free()
        # the gated MLP projection (gate_proj + up_proj + SwiGLU, 4096 -> 2 x 14336) as dispatched, beside the batched
        # projection followed by the elementwise launch; the plan names what the one call runs
        gated = {}
        for mm in (1, 8, 64, 512, 2048):
            xg = ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(900 + mm, mm, 4096)))
            yg, gb, ub = (ctx.alloc(mm * 14336 * 2) for _ in range(3))
            nl = min(len(layers), 4)
            one = lambda i: ctx.gated_qgemm(layers[i % nl]["gate"], layers[i % nl]["up"], xg, pkg.BF16, yg, pkg.BF16, mm,
                                            pkg.GATED_SILU, 0, 0, 0, stream)
            def apart(i):
                ctx.batched_qgemm([layers[i % nl]["gate"], layers[i % nl]["up"]], xg, pkg.BF16, [gb, ub], pkg.BF16, mm, 0, 0, stream)
                ctx.gated_activation(gb, ub, yg, pkg.BF16, 14336, mm, 0, pkg.GATED_SILU, stream)
            for fn in (one, apart):
                for i in range(4):
                    fn(i)
            ctx.synchronize(stream)
            # samples of the two forms in turn, medians (whichever form is timed first after a change of shape reads
            # 5 to 10 % slow)
            reps = 48 if mm <= 64 else 16
            samples = ([], [])
            for _ in range(7):
                samples[0].append(time_region(ctx, one, reps, stream))
                samples[1].append(time_region(ctx, apart, reps, stream))
            t_one, t_apart = (sorted(v)[len(v) // 2] for v in samples)
            probe = pkg.DispatchPlan(ctx)
            probe.add_gated_mlp(layers[0]["gate"], layers[0]["up"], xg, pkg.BF16, yg, pkg.BF16, mm, activation=pkg.GATED_SILU)
            rec = probe.step(0)[0]
            gated[f"M={mm}"] = {"us": round(t_one * 1e3, 2), "projections_then_elementwise_us": round(t_apart * 1e3, 2),
                                "kernel": rec.device_kernel, "family": rec.kernel_family}
            probe.destroy()
            for b in (xg, yg, gb, ub):
                b.free()
        next_rows["gated MLP projection 4096 -> 2 x 14336 q4 g64 + swiglu, bf16"] = gated
        # prompts: q+k+v (4096 -> 4096 + 1024 + 1024) through mi355q_batched_qgemm as dispatched, beside a call per
        # projection; the table names what the projections run as together
        shared = {}
        for mm in (128, 512, 2048):
            xq = ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(950 + mm, mm, 4096)))
            outs = [ctx.alloc(mm * n_ * 2) for n_ in (4096, 1024, 1024)]
            nl = min(len(layers), 4)
            qkv = lambda i: [layers[i % nl][t] for t in ("q", "k", "v")]
            one = lambda i: ctx.batched_qgemm(qkv(i), xq, pkg.BF16, outs, pkg.BF16, mm, 0, 0, stream)
            def apart(i):
                for w_, o_ in zip(qkv(i), outs):
                    ctx.qgemm(w_, xq, pkg.BF16, o_, pkg.BF16, mm, 0, 0, 0, stream)
            for fn in (one, apart):
                for i in range(4):
                    fn(i)
            ctx.synchronize(stream)
            samples = ([], [])
            for _ in range(7):
                samples[0].append(time_region(ctx, one, 16, stream))
                samples[1].append(time_region(ctx, apart, 16, stream))
            t_one, t_apart = (sorted(v)[len(v) // 2] for v in samples)
            route, kernel = pkg.probe_shared_route(fmt, pkg.LAYOUT_PLANES, (4096, 1024, 1024), 4096, pkg.BF16, mm)
            shared[f"M={mm}"] = {"us": round(t_one * 1e3, 2), "a_call_per_projection_us": round(t_apart * 1e3, 2),
                                 "route": route, "kernel": kernel}
            for b in [xq] + outs:
                b.free()
        next_rows["q+k+v 4096 -> 4096 + 1024 + 1024 q4 g64 at prompts, bf16"] = shared
        # container: one q4 g64 gate tensor written, opened, validated, uploaded as one device buffer, wrapped with no copy
        words, s_, z_ = host["gate"]
        blocks = pkg.repack_mlx_to_staf(fmt, words, s_, z_, pkg.BF16)
        with tempfile.TemporaryDirectory() as tmp:
            path = os.path.join(tmp, "bench.staf")
            pkg.staf_write(path, [dict(name="layers.0.gate_proj.weight", scheme_identifier=fmt.scheme_identifier,
                                       shape=[14336, 4096 * BITS // 32], payload=blocks.tobytes())], None)
            t0 = time.perf_counter()
            ok = pkg.staf_is_valid(path)
            f = pkg.STAFFile(path)
            t1 = time.perf_counter()
            region = f.upload(ctx)
            ctx.synchronize()
            t2 = time.perf_counter()
            w = f.weight(ctx, "layers.0.gate_proj.weight", pkg.LAYOUT_STAF_BLOCKS, region)
            t3 = time.perf_counter()
            next_rows["model.staf with one 33 MB q4 tensor (host side, ms)"] = {
                "validate_and_open_ms": round((t1 - t0) * 1e3, 2), "upload_ms": round((t2 - t1) * 1e3, 2),
                "wrap_zero_copy_ms": round((t3 - t2) * 1e3, 3), "valid": bool(ok)}
            w.destroy(); region.free(); f.close()
        for k_, v_ in next_rows.items():
            log(f"  {k_}: {v_}")

    # ---- the second half of the metric: the prefill GEMM (benchmark config 3) on N(0,1) activations ------------
    # both MLP shapes at M = 128, 512, 2048, 4096, as dispatched (tile shape, K split and route are the library's choice),
    # over four rotating weight copies; the M = 2048 gate projection is the roofline figure.
    prefill, roofline_prefill = None, None
    if not a.no_prefill:
        sweep = {}
        for name, n, k in (("gate 4096->14336", 14336, 4096), ("down 14336->4096", 4096, 14336)):
            wts = [L["gate" if n == 14336 else "down"] for L in layers[:4]]
            for mm in (128, 512, 2048, 4096):
                xb = ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(500 + mm, mm, k)))        # N(0,1)
                yb = ctx.alloc(mm * n * 2)
                for i in range(len(wts)):
                    ctx.qgemm(wts[i], xb, pkg.BF16, yb, pkg.BF16, mm, 0, 0, 0, stream)
                ctx.synchronize(stream)
                reps = 24 if mm >= 2048 else 48
                ms, ms_first, taken = steady_region(
                    ctx, lambda i: ctx.qgemm(wts[i % len(wts)], xb, pkg.BF16, yb, pkg.BF16, mm, 0, 0, 0, stream), reps, stream)
                steps_p = wts[0].plan_prefill_steps(mm, k)
                if mm == 2048 and not a.skip_parity:
                    # parity gate on the output just timed (the last launch read copy (reps - 1) % 4, all copies hold the
                    # same tensor): every row, 32 columns spread over the matrix, against an fp64 accumulation of the
                    # bf16-rounded weights; the output is bf16, so the bar is that of a bf16 rounding (2^-9) on top
                    ctx.synchronize(stream)
                    cols = np.unique(np.concatenate([np.arange(0, n, n // 24), [1, 255, 256, n - 257, n - 2, n - 1]]))
                    words, s_, z_ = host["gate" if n == 14336 else "down"]
                    wq = oracle.dequant_planes_f32(BITS, GROUP, n, k, words, s_, z_, oracle.BF16)[cols]
                    wb = oracle.bf16_to_f32(oracle.bf16_from_f32(wq)).reshape(wq.shape)
                    xh = oracle.bf16_to_f32(oracle.bf16_from_f32(kat.seeded_activations(500 + mm, mm, k))).reshape(mm, k)
                    want = oracle.gemm_f64(np.ascontiguousarray(wb), xh)
                    got = oracle.bf16_to_f32(yb.download(np.uint16, (mm, n))[:, cols]).reshape(mm, len(cols))
                    rel = float(np.linalg.norm(got - want) / np.linalg.norm(want))
                    mx = float(np.max(np.abs(got - want)))
                    if not (rel <= 3e-3 and mx <= 2e-2 + 4e-3 * float(np.max(np.abs(want)))):
                        sys.exit(f"bench.py: prefill parity gate failed on {name} M={mm}: rel-L2 {rel:.3e} max-abs {mx:.3e}")
                    log(f"  parity {name} M={mm} ({steps_p[0].device_kernel}): rel-L2 {rel:.2e} max-abs {mx:.2e} (bf16 output)")
                sweep[f"{name} M={mm}"] = {"us": round(ms * 1e3, 1), "TFLOPs": round(2.0 * mm * n * k / (ms * 1e-3) / 1e12, 1),
                                           "route": " + ".join(st.device_kernel for st in steps_p),
                                           "first_sample_us": round(ms_first * 1e3, 1), "samples_of": [taken, reps]}
                xb.free(); yb.free()
        # the reference prefills with f16 or fp32 activations: the same launch in those types, as dispatched, M = 2048 gate
        for tname, xt, npdt in (("f16", pkg.F16, np.float16), ("f32", pkg.F32, np.float32)):  # fp32: [hi | lo] bf16 halves, 2 K
            wts = [L["gate"] for L in layers[:4]]
            xa = kat.seeded_activations(2548, 2048, 4096).astype(npdt)
            xb = ctx.upload(xa.view(np.uint16) if tname == "f16" else xa)
            yb = ctx.alloc(2048 * 14336 * 4)
            for i in range(len(wts)):
                ctx.qgemm(wts[i], xb, xt, yb, xt, 2048, 0, 0, 0, stream)
            ctx.synchronize(stream)
            ms, ms_first, taken = steady_region(ctx, lambda i: ctx.qgemm(wts[i % len(wts)], xb, xt, yb, xt, 2048, 0, 0, 0, stream), 12, stream)
            sweep[f"gate 4096->14336 M=2048 {tname} activations"] = {
                "us": round(ms * 1e3, 1), "TFLOPs": round(2.0 * 2048 * 14336 * 4096 / (ms * 1e-3) / 1e12, 1),
                "first_sample_us": round(ms_first * 1e3, 1), "samples_of": [taken, 12],
                "route": " + ".join(st.device_kernel for st in wts[0].plan_prefill_steps(2048, 4096, x_dtype=xt))}
            xb.free(); yb.free()
        sweep["activations"] = "N(0,1) bf16, seeded"
        sweep["timing"] = ("sustained load: samples of 24 (48 below M = 2048) launches back to back until one is within 1 % of "
                           "the one before; `us` is that sample, `first_sample_us` the first one after the part was idle")
        log("  prefill sweep (N(0,1)): " + ", ".join(f"{k2} {v['us']} us ({v['TFLOPs']} TFLOP/s, {v['route']})"
                                                   for k2, v in sweep.items() if isinstance(v, dict)))
        # the same M = 2048 gate launch on the fused kernel with the in-kernel clock probe (what clock the matrix cores
        # held), and on constant activations as a labelled aside (the part clocks higher when operand bits do not toggle)
        m = 2048
        xg = ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(5, m, 4096)))
        yg = ctx.alloc(m * 14336 * 2)
        wg = layers[0]["gate"]
        probe = pkg.FLAG_FORCE_MFMA | pkg.FLAG_PROBE_CLOCK

        def gemm_figure(xbuf):
            nonlocal probe
            ctx.qgemm(wg, xbuf, pkg.BF16, yg, pkg.BF16, m, 0, 0, probe, stream)
            ctx.synchronize(stream)
            ms, _, _ = steady_region(ctx, lambda i: ctx.qgemm(wg, xbuf, pkg.BF16, yg, pkg.BF16, m, 0, 0, probe, stream), 10, stream)
            return ms, ctx.clock_probe_ghz()

        ms_g, ghz = gemm_figure(xg)
        probe |= pkg.FLAG_PROBE_TILED                     # the tiled kernel (weights dequantised into LDS) beside it
        ms_t, ghz_t = gemm_figure(xg)
        probe &= ~pkg.FLAG_PROBE_TILED
        # the two-dispatch route (dequantise, then the platform's dense GEMM) on the same problem, where the library is there
        ms_l = None
        try:
            ctx.qgemm(wg, xg, pkg.BF16, yg, pkg.BF16, m, 0, 0, pkg.FLAG_FORCE_TWO_STEP, stream)
            ctx.synchronize(stream)
            ms_l, _, _ = steady_region(ctx, lambda i: ctx.qgemm(wg, xg, pkg.BF16, yg, pkg.BF16, m, 0, 0, pkg.FLAG_FORCE_TWO_STEP, stream), 10, stream)
        except pkg.MI355QError as e:
            log(f"  two-dispatch route not available: {e}")
        xc = ctx.upload(np.full((m, 4096), 0x3F80, np.uint16))
        ms_c, ghz_c = gemm_figure(xc)
        xc.free(); xg.free(); yg.free()
        flops = 2.0 * m * 14336 * 4096
        prefill = {"config3": sweep,
                   "fused_kernel_m2048_gate": {"us": round(ms_g * 1e3, 1), "TFLOPs": round(flops / (ms_g * 1e-3) / 1e12, 1),
                                               "shader_clock_GHz": round(ghz, 3),
                                               "kernel": wg.plan_prefill_steps(m, 4096, flags=pkg.FLAG_FORCE_MFMA)[0].device_kernel},
                   "tiled_kernel_m2048_gate": {"us": round(ms_t * 1e3, 1), "TFLOPs": round(flops / (ms_t * 1e-3) / 1e12, 1),
                                               "shader_clock_GHz": round(ghz_t, 3),
                                               "kernel": wg.plan_prefill_steps(m, 4096, flags=pkg.FLAG_FORCE_MFMA | pkg.FLAG_PROBE_TILED)[0].device_kernel},
                   "two_dispatch_route_m2048_gate": (None if ms_l is None else
                                                     {"us": round(ms_l * 1e3, 1), "TFLOPs": round(flops / (ms_l * 1e-3) / 1e12, 1),
                                                      "kernel": "+".join(st.device_kernel for st in wg.plan_prefill_steps(m, 4096, flags=pkg.FLAG_FORCE_TWO_STEP))}),
                   "aside_constant_activations_fused_kernel": {"us": round(ms_c * 1e3, 1), "TFLOPs": round(flops / (ms_c * 1e-3) / 1e12, 1),
                                                               "shader_clock_GHz": round(ghz_c, 3)}}
        log(f"  fused kernel M={m} gate: {prefill['fused_kernel_m2048_gate']}; constant activations (aside): "
            f"{prefill['aside_constant_activations_fused_kernel']}")
        best = sweep["gate 4096->14336 M=2048"]
        roofline_prefill = {"bound": "mfma", "achieved": best["TFLOPs"], "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                            "frac": round(best["TFLOPs"] / MFMA_BF16_PEAK_TFLOPS, 4),
                            "traffic": PREFILL_TRAFFIC_BYTES.get((best["route"], int(wg.plan_prefill_steps(2048, 4096)[0].grid[0]))),
                            "kernel": best["route"], "m": 2048, "shape": "4096->14336", "us": best["us"],
                            "flops": flops, "activations": "N(0,1) bf16",
                            "timing": "sustained load (see config.prefill_gemm_gate.config3.timing)",
                            "first_sample_us": best["first_sample_us"],
                            "gate_m4096": {"TFLOPs": sweep["gate 4096->14336 M=4096"]["TFLOPs"],
                                           "frac": round(sweep["gate 4096->14336 M=4096"]["TFLOPs"] / MFMA_BF16_PEAK_TFLOPS, 4),
                                           "kernel": sweep["gate 4096->14336 M=4096"]["route"]},
                            "down_14336_4096": {"TFLOPs": sweep["down 14336->4096 M=2048"]["TFLOPs"],
                                                "frac": round(sweep["down 14336->4096 M=2048"]["TFLOPs"] / MFMA_BF16_PEAK_TFLOPS, 4),
                                                "kernel": sweep["down 14336->4096 M=2048"]["route"]}}

    cpu = None if a.no_cpu else cpu_baseline(a.cpu_seconds)

    out = {
        "metric": "4-bit decode GEMV GB/s (weight bytes / time, M=1)",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 activations x u4 codes, fp32 accumulate",
        "data": "synthetic: W~N(0,0.02^2) quantised q4 g64 (bf16 scale/bias planes), x~N(0,1) bf16, seeded; "
                f"{a.layers} resident copies of one layer's tensors",
        "config": {"workload": "Llama-3-8B decode layer sweep (benchmark config 1), M=1: q,k,v,o,gate,up,down "
                               "GEMVs per step", "bits": BITS, "group_size": GROUP,
                   "weight_bytes_per_step": layer_bytes, "layers_resident": a.layers,
                   "replay": mode, "replay_GBps": replay_gbps, "step_time_spread": spreads[mode],
                   "step_time_spread_all": spreads, "steps_asked": a.steps, "warmup_asked": a.warmup,
                   "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2), "per_shape": per_shape,
                   "f16_activations_step": f16_step, "batch_sweep": batch_sweep, "other_configs": other, "all_formats": all_formats, "staf_blocks_in_place_step": staf_step, "next_rows": next_rows,
                   "stream_read_probe": stream_read,
                   "prefill_gemm_gate": prefill},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic,
                     "algorithmic_bytes": dom_bytes, "us": per_shape[dom]["us"],
                     "kernel": f"{dom_kernel} grid {dom_grid} x {dom_block}: {dom} launch of the {mode} schedule, 4096->"
                               f"{dom_bytes // weight_bytes(1, 4096)} rows, {dom_bytes} weight bytes/launch"},
    }
    if roofline_prefill is not None:
        out["roofline_prefill"] = roofline_prefill
    if cpu is not None:
        out["cpu_baseline"] = cpu
    print(json.dumps(out), flush=True)
    ctx.close()


if __name__ == "__main__":
    main()
