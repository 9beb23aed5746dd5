"""GPU parity tests of the batched projections (two or three weights sharing their input), through
the C ABI: the decode-time counterpart of the reference's batched q4 prefill kernels
(MetalSourceGenerator+Quantized.swift:166-338: rows routed by cumulative output dimension, every
output with row stride N_i).

Bars as for the single projection: fp32 outputs within relative L2 <= 1e-3 and max-abs <= 2e-2 of
an fp64 accumulation of the same dequantised weights; bf16 outputs equal bf16_rne(fp32 outputs).
"""
import sys

import numpy as np
import pytest

import kat
import oracle
from gpu_util import act_rounded, assert_within_tolerance, out_from_device, seeded_case

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, file=sys.stderr, flush=True)


def _prepare(pkg, ctx, seed, ns, k, bits, group, layout):
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
    ws, wqs = [], []
    for i, n in enumerate(ns):
        words, s, z, wq = seeded_case(seed + i, n, k, bits, group)
        ws.append(ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, layout))
        wqs.append(wq)
    return ws, wqs


def _run_batched(pkg, ctx, ws, ns, x, y_dtype, flags=0, x_stride=0):
    m = x.shape[0]
    xd = ctx.upload(oracle.bf16_from_f32(x).reshape(x.shape))
    esz = 4 if y_dtype == pkg.F32 else 2
    yds = [ctx.alloc(m * n * esz) for n in ns]
    for yd in yds:
        ctx.fill(yd, 0x7FC00000 if y_dtype == pkg.F32 else 0x7FC07FC0)
    ctx.batched_qgemm(ws, xd, pkg.BF16, yds, y_dtype, m, x_stride, flags)
    ctx.synchronize()
    out = [out_from_device(yd, y_dtype, (m, n), pkg) for yd, n in zip(yds, ns)]
    xd.free()
    for yd in yds:
        yd.free()
    return out


@pytest.mark.parametrize("ns,k", [((4096, 1024, 1024), 4096), ((14336, 14336), 4096)])
@pytest.mark.parametrize("m", [1, 2, 8])
def test_batched_llama_projections(pkg, ctx, ns, k, m):
    """q+k+v and gate+up of a Llama-3-8B layer (benchmark config 1 shapes) as one launch each."""
    ws, wqs = _prepare(pkg, ctx, 1300 + len(ns), ns, k, 4, 64, pkg.LAYOUT_PLANES)
    x = act_rounded(kat.seeded_activations(1310 + m, m, k), pkg.BF16, pkg)
    say(f"batched {ns} K={k} M={m}")
    got = _run_batched(pkg, ctx, ws, ns, x, pkg.F32)
    gbf = _run_batched(pkg, ctx, ws, ns, x, pkg.BF16)
    for i, n in enumerate(ns):
        assert_within_tolerance(got[i], oracle.gemm_f64(wqs[i], x), f"projection {i} M={m}")
        assert np.array_equal(oracle.bf16_from_f32(gbf[i]), oracle.bf16_from_f32(got[i]))
    for w in ws:
        w.destroy()


def test_batched_ragged_segments_and_formats(pkg, ctx):
    """Row counts that put segment boundaries inside a wavefront's run of rows and inside a
    workgroup, tiny segments, every fast bit width, odd M."""
    cases = [((5, 1, 3), 256, 4, 64), ((130, 67), 2048 + 64, 4, 64), ((1, 1), 64, 4, 64),
             ((257, 63, 129), 1024, 8, 32), ((70, 200), 1024, 3, 64), ((33, 31, 2), 2048, 2, 64),
             ((100, 100, 100), 512, 6, 64), ((64, 65), 1024, 5, 32)]
    for ci, (ns, k, bits, group) in enumerate(cases):
        ws, wqs = _prepare(pkg, ctx, 1400 + 10 * ci, ns, k, bits, group, pkg.LAYOUT_PLANES)
        for m in (1, 3, 8):
            x = act_rounded(kat.seeded_activations(1500 + ci + m, m, k), pkg.BF16, pkg)
            say(f"ragged batched {ns} K={k} q{bits}g{group} M={m}")
            got = _run_batched(pkg, ctx, ws, ns, x, pkg.F32)
            for i in range(len(ns)):
                assert_within_tolerance(got[i], oracle.gemm_f64(wqs[i], x), f"{ns} seg {i} M={m}")
        for w in ws:
            w.destroy()


def test_batched_equals_separate_launches_on_other_routes(pkg, ctx):
    """STAF blocks (per-code kernel), forced generic, and M > 8 (matrix cores) keep one launch per
    projection; results must match the single-projection entry points exactly."""
    ns, k = (192, 64, 320), 512
    for layout, flags, m in [(pkg.LAYOUT_STAF_BLOCKS, 0, 2), (pkg.LAYOUT_PLANES, pkg.FLAG_FORCE_GENERIC, 3),
                             (pkg.LAYOUT_PLANES, 0, 40)]:
        ws, wqs = _prepare(pkg, ctx, 1600, ns, k, 4, 64, layout)
        x = act_rounded(kat.seeded_activations(1601 + m, m, k), pkg.BF16, pkg)
        say(f"batched route layout={layout} flags={flags} M={m}")
        got = _run_batched(pkg, ctx, ws, ns, x, pkg.F32, flags)
        xd = ctx.upload(oracle.bf16_from_f32(x).reshape(x.shape))
        for i, n in enumerate(ns):
            yd = ctx.alloc(m * n * 4)
            ctx.qgemm(ws[i], xd, pkg.BF16, yd, pkg.F32, m, 0, 0, flags)
            ctx.synchronize()
            assert np.array_equal(yd.download(np.float32, (m, n)), got[i])
            yd.free()
        xd.free()
        for w in ws:
            w.destroy()


def test_batched_argument_errors(pkg, ctx):
    ws, _ = _prepare(pkg, ctx, 1700, (64, 64), 256, 4, 64, pkg.LAYOUT_PLANES)
    other, _ = _prepare(pkg, ctx, 1701, (64,), 512, 4, 64, pkg.LAYOUT_PLANES)
    x = ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(1, 1, 512)))
    y = [ctx.alloc(64 * 4) for _ in range(4)]
    with pytest.raises(pkg.MI355QError):                       # count must be 2 or 3
        ctx.batched_qgemm(ws[:1], x, pkg.BF16, y[:1], pkg.F32, 1)
    with pytest.raises(pkg.MI355QError):
        ctx.batched_qgemm(ws + ws, x, pkg.BF16, y, pkg.F32, 1)
    with pytest.raises(pkg.MI355QError):                       # K differs
        ctx.batched_qgemm([ws[0], other[0]], x, pkg.BF16, y[:2], pkg.F32, 1)
    with pytest.raises(pkg.MI355QError):                       # null output
        ctx.batched_qgemm(ws, x, pkg.BF16, [y[0], None], pkg.F32, 1)
    for b in y + [x]:
        b.free()
    for w in ws + other:
        w.destroy()


def test_plan_with_batched_steps_replays_identically(pkg, ctx):
    """A decode plan of fused steps (q+k+v, o, gate+up, down) replayed on a stream and as a HIP
    graph reproduces the eager batched launches bit for bit on every replay."""
    k = 1024
    ns_qkv, ns_gu = (1024, 256, 256), (2048, 2048)
    qkv, _ = _prepare(pkg, ctx, 1800, ns_qkv, k, 4, 64, pkg.LAYOUT_PLANES)
    gu, _ = _prepare(pkg, ctx, 1810, ns_gu, k, 4, 64, pkg.LAYOUT_PLANES)
    x = ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(1820, 1, k)))
    y_qkv = [ctx.alloc(n * 4) for n in ns_qkv]
    y_gu = [ctx.alloc(n * 4) for n in ns_gu]
    outs = y_qkv + y_gu
    ctx.batched_qgemm(qkv, x, pkg.BF16, y_qkv, pkg.F32, 1)
    ctx.batched_qgemm(gu, x, pkg.BF16, y_gu, pkg.F32, 1)
    ctx.synchronize()
    eager = [o.download(np.float32) for o in outs]
    plan = pkg.DispatchPlan(ctx)
    plan.add_batched_linear(qkv, x, pkg.BF16, y_qkv, pkg.F32, 1, layer_index=0, tensor_name="layers.0.qkv")
    plan.add_batched_linear(gu, x, pkg.BF16, y_gu, pkg.F32, 1, layer_index=0, tensor_name="layers.0.gate_up")
    assert len(plan) == 2
    st, layer, name = plan.step(0)
    assert st.kernel_family == "batched3Q4G64" and name == "layers.0.qkv" and layer == 0
    stream = ctx.stream_create()
    for rep in range(2):
        for o in outs:
            ctx.fill(o, 0x7FC00000, stream)
        plan.encode(stream)
        ctx.synchronize(stream)
        for o, want in zip(outs, eager):
            assert np.array_equal(o.download(np.float32), want), f"stream replay {rep}"
    plan.graph_build(stream)
    for rep in range(3):
        for o in outs:
            ctx.fill(o, 0x7FC00000, stream)
        plan.graph_launch(stream)
        ctx.synchronize(stream)
        for o, want in zip(outs, eager):
            assert np.array_equal(o.download(np.float32), want), f"graph replay {rep}"
    plan.destroy()
    for b in outs + [x]:
        b.free()
    for w in qkv + gu:
        w.destroy()


def test_plan_records_of_shared_steps_name_the_kernel_that_runs(pkg, ctx):
    """The record of a shared step names the kernel of the one launch over all matrices (launcher and planner ask the
    same function): the dot-product, matrix-core, TILE16, in-place and streamed-weight kernels by layout and rows, and
    the replayed step equals the eager call."""
    k, ns = 1024, (1024, 256, 256)
    cases = [(pkg.LAYOUT_PLANES, 1, r"gemv_(rows|planes)_q4_g64"), (pkg.LAYOUT_PLANES, 8, "gemv_mfma_planes_q4_g64"),
             (pkg.LAYOUT_PLANES, 32, "qgemm_stream_q4_g64"), (pkg.LAYOUT_TILE16, 16, "gemv_tile16_q4_g64"),
             (pkg.LAYOUT_STAF_BLOCKS, 2, "gemv_staf_q4_g64"), (pkg.LAYOUT_STAF_BLOCKS, 32, "qgemm_stream_q4_g64")]
    import re
    for layout, m, want in cases:
        ws, _ = _prepare(pkg, ctx, 1900 + m, ns, k, 4, 64, layout)
        fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
        route, planned = pkg.probe_shared_route(fmt, layout, ns, k, pkg.BF16, m)
        x = ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(1910 + m, m, k)))
        ys = [ctx.alloc(m * n * 4) for n in ns]
        ctx.batched_qgemm(ws, x, pkg.BF16, ys, pkg.F32, m)
        ctx.synchronize()
        eager = [y.download(np.float32) for y in ys]
        plan = pkg.DispatchPlan(ctx)
        plan.add_batched_linear(ws, x, pkg.BF16, ys, pkg.F32, m)
        st, _, _ = plan.step(0)
        assert re.fullmatch(want, st.device_kernel) and st.device_kernel == planned and route.startswith("shared/"), (layout, m, st.device_kernel, route)
        for y in ys:
            ctx.fill(y, 0x7FC00000)
        plan.encode(0)
        ctx.synchronize()
        for y, e in zip(ys, eager):
            assert np.array_equal(y.download(np.float32), e), (layout, m)
        plan.destroy()
        for b in ys + [x]:
            b.free()
        for w in ws:
            w.destroy()
