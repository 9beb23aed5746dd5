"""GPU parity tests of the two-dispatch prefill route through the C ABI: dequant_q{b}_g{g}_bf16 into the context's
scratch matrix, then the dense bf16 GEMM of the platform library (the reference's dequant + matmul2d route,
MetalSourceGenerator+Quantized.swift:361-416 then MetalSourceGenerator+Linear.swift:18-81; step builder
MetalPrefillStepBuilder.swift:928-955).  It serves every registered format on every device layout.

Bars: cases whose products and partial sums are exactly representable are compared exactly; seeded cases within
relative L2 <= 1e-3 and max-abs <= 2e-2 of an fp64 accumulation of the bf16-rounded dequantised weights, on the fp32
output; the bf16 output is within one bf16 rounding (2^-8 relative, plus 1e-5 for sums that cancel) of the fp32 output.
"""
import sys

import numpy as np
import pytest

import kat
import oracle
from gpu_util import rel_l2, Case, act_rounded, act_to_device_array, assert_within_tolerance, out_from_device, seeded_case

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, file=sys.stderr, flush=True)


def bf16_round(a):
    a = np.asarray(a, np.float32)
    return oracle.bf16_to_f32(oracle.bf16_from_f32(a)).reshape(a.shape)


def run_qgemm(ctx, pkg, w, x_f32, y_dtype, flags, x_stride=None, y_stride=None, stream=0):
    m, xs = x_f32.shape
    n = int(w.info.n_rows)
    ys = n if y_stride is None else y_stride
    xd = ctx.upload(oracle.bf16_from_f32(x_f32).reshape(x_f32.shape))
    yd = ctx.alloc(m * ys * (4 if y_dtype == pkg.F32 else 2))
    ctx.fill(yd, 0x7FC07FC0 if y_dtype != pkg.F32 else 0x7FC00000)
    ctx.synchronize()
    ctx.qgemm(w, xd, pkg.BF16, yd, y_dtype, m, xs if x_stride is None else x_stride, ys if y_stride else 0, flags, stream)
    ctx.synchronize(stream) if stream else ctx.synchronize()
    y = out_from_device(yd, y_dtype, (m, ys), pkg)
    xd.free(); yd.free()
    return y


@pytest.mark.parametrize("bits,group", kat.ALL_FORMATS)
def test_two_step_exact_small_integers_every_format(pkg, ctx, bits, group):
    """Every registered format from the block layout (and from the planes where the layout exists): codes, scales,
    zeros and activations such that all products and partial sums are multiples of 2^-6 below 2^17, so any order of
    fp32 accumulation gives the same, exact, result."""
    rng = np.random.default_rng(bits * 131 + group)
    blocks_per_row = int(32 // np.gcd(32, group * bits)) * 2
    m, n, k = 45, 88, group * blocks_per_row
    qmax = (1 << bits) - 1
    codes = rng.integers(0, qmax + 1, (n, k), dtype=np.uint8)
    scales = rng.choice([0.125, 0.25, 0.5], (n, k // group))
    zeros = rng.integers(-4, 5, (n, k // group)) * 0.25
    if bits == 8:
        scales = np.full((n, k // group), 0.25)
        zeros = np.zeros((n, k // group))
    case = Case(bits, group, codes, scales, zeros)
    wq = scales.repeat(group, axis=1) * codes + zeros.repeat(group, axis=1)
    assert np.array_equal(bf16_round(wq), wq.astype(np.float32))
    x = rng.integers(-8, 9, (m, k)).astype(np.float32) * 0.125
    want = x.astype(np.float64) @ wq.T
    layouts = [(pkg.LAYOUT_STAF_BLOCKS, None)] + ([(pkg.LAYOUT_PLANES, pkg.BF16)] if case.planes_eligible() else [])
    for layout, sb in layouts:
        w = case.device_weight(ctx, pkg, layout, sb)
        say(f"two-step exact q{bits}g{group} layout {layout}")
        got = run_qgemm(ctx, pkg, w, x, pkg.F32, pkg.FLAG_FORCE_TWO_STEP)
        assert np.array_equal(got.astype(np.float64), want), (bits, group, layout)
        got = run_qgemm(ctx, pkg, w, x, pkg.BF16, pkg.FLAG_FORCE_TWO_STEP)
        assert np.array_equal(got, bf16_round(want.astype(np.float32))), (bits, group, layout)
        w.destroy()


@pytest.mark.parametrize("bits,group,layout_name", [(4, 64, "LAYOUT_STAF_BLOCKS"), (4, 64, "LAYOUT_PLANES"),
                                                    (4, 64, "LAYOUT_TILE16"), (5, 64, "LAYOUT_STAF_BLOCKS"),
                                                    (3, 32, "LAYOUT_STAF_BLOCKS"), (8, 128, "LAYOUT_PLANES")])
def test_two_step_seeded_ragged_shapes_and_strides(pkg, ctx, bits, group, layout_name):
    layout = getattr(pkg, layout_name)
    n, k = 200, 1024
    words, s, z, wq = seeded_case(3100 + bits + group, n, k, bits, group)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
    w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, layout)
    wb = bf16_round(wq)
    for m, xpad, ypad in ((1, 0, 0), (7, 8, 8), (77, 8, 0), (130, 0, 24), (1030, 16, 8)):
        say(f"two-step seeded q{bits}g{group} {layout_name} M={m}")
        x = np.zeros((m, k + xpad), np.float32)
        x[:, :k] = act_rounded(kat.seeded_activations(3200 + m, m, k), pkg.BF16, pkg)
        if xpad:
            x[:, k:] = 1000.0                                  # must never be read into a product
        got = run_qgemm(ctx, pkg, w, x, pkg.F32, pkg.FLAG_FORCE_TWO_STEP, y_stride=(n + ypad) if ypad else None)
        # below sixteen rows the route keeps fp32 weights (the decode kernels' arithmetic), from sixteen bf16 ones
        assert_within_tolerance(got[:, :n], oracle.gemm_f64(wq if m < 16 else wb, x[:, :k]), f"M={m}")
        if ypad:
            assert np.all(np.isnan(got[:, n:]))                # the padding of the output rows stays untouched
        gb = run_qgemm(ctx, pkg, w, x, pkg.BF16, pkg.FLAG_FORCE_TWO_STEP, y_stride=(n + ypad) if ypad else None)
        # one bf16 rounding of a sum that the two launches may have accumulated in different orders
        assert np.all(np.abs(gb[:, :n] - got[:, :n]) <= np.abs(got[:, :n]) * 2.0 ** -8 + 1e-5)
    w.destroy()


def test_two_step_is_chosen_where_measured_faster_and_planned_as_two_steps(pkg, ctx):
    """Without flags: the block layout (no fused matrix-core kernel) takes the route beyond the 96 rows of the
    streamed-weight kernel; the planes keep
    the fused kernel up to 511 rows (wide matrices, N >= 8192, up to 767; shapes with K > N up to 2047).  The planner reports dequant + GEMM as two steps."""
    n, k = 192, 512
    words, s, z, wq = seeded_case(3300, n, k, 4, 64)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    wb = bf16_round(wq)
    ws = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_STAF_BLOCKS)
    words1, s1, z1, _ = seeded_case(3303, 512, 512, 4, 64)               # N >= K
    wp = ctx.weight_prepare_mlx(fmt, words1, s1, z1, pkg.BF16, pkg.LAYOUT_PLANES)
    steps = ws.plan_prefill_steps(100)
    assert [st.kernel_name for st in steps] == ["dequant_q4_g64_bf16", "gemm_bf16_f32s"]
    assert [st.kernel_family for st in steps] == ["dequantToBFloat", "libraryGEMM"]
    assert steps[0].flops == 0 and steps[1].flops == 2 * 100 * n * k and steps[1].weight_bytes == n * k * 2
    assert not steps[0].used_fallback and not steps[1].used_fallback
    assert [st.device_kernel for st in ws.plan_prefill_steps(64)] == ["qgemm_stream_q4_g64"]      # nine to 96 rows
    assert [st.device_kernel for st in ws.plan_prefill_steps(12)] == ["qgemm_stream_q4_g64"]
    assert len(ws.plan_prefill_steps(2)) == 1 and ws.plan_prefill_steps(2)[0].device_kernel == "gemv_staf_q4_g64"
    assert len(ws.plan_prefill_steps(64, flags=pkg.FLAG_FORCE_SMALL_M)) == 1
    assert [st.kernel_family for st in wp.plan_prefill_steps(511)] == ["mfmaGEMM"]
    assert [st.kernel_family for st in wp.plan_prefill_steps(512)] == ["dequantToBFloat", "libraryGEMM"]
    assert [st.kernel_family for st in wp.plan_prefill_steps(1024, flags=pkg.FLAG_FORCE_MFMA)] == ["mfmaGEMM"]
    words3, s3, z3, _ = seeded_case(3304, 8192, 64, 4, 64)                # wide: N >= 8192
    ww = ctx.weight_prepare_mlx(fmt, words3, s3, z3, pkg.BF16, pkg.LAYOUT_PLANES)
    assert [st.kernel_family for st in ww.plan_prefill_steps(767)] == ["mfmaGEMM"]
    assert [st.kernel_family for st in ww.plan_prefill_steps(768)] == ["dequantToBFloat", "libraryGEMM"]
    ww.destroy()
    # K > N: the fused kernel keeps the shape up to 2047 rows
    words2, s2, z2, _ = seeded_case(3301, 128, 1024, 4, 64)
    wl = ctx.weight_prepare_mlx(fmt, words2, s2, z2, pkg.BF16, pkg.LAYOUT_PLANES)
    assert [st.kernel_family for st in wl.plan_prefill_steps(2047)] == ["mfmaGEMM"]
    assert [st.kernel_family for st in wl.plan_prefill_steps(2048)] == ["dequantToBFloat", "libraryGEMM"]
    wl.destroy()
    x = act_rounded(kat.seeded_activations(3302, 64, k), pkg.BF16, pkg)
    want = oracle.gemm_f64(wb, x)
    auto = run_qgemm(ctx, pkg, ws, x, pkg.F32, 0)
    assert_within_tolerance(auto, want, "blocks, no flags")
    slow = run_qgemm(ctx, pkg, ws, x, pkg.F32, pkg.FLAG_FORCE_SMALL_M)       # fp32 weights: close, not the same
    assert_within_tolerance(slow, oracle.gemm_f64(wq, x), "blocks, decode kernels")
    # f16 outputs: the library has no bf16 x bf16 -> f16 product; forced, the route says so; unforced, other kernels serve
    with pytest.raises(pkg.MI355QError) as err:
        run_qgemm(ctx, pkg, ws, x, pkg.F16, pkg.FLAG_FORCE_TWO_STEP)
    assert err.value.status_name == "KERNEL_NOT_FOUND"
    h = run_qgemm(ctx, pkg, ws, x, pkg.F16, 0)                              # 64 rows: the streamed-weight kernel, bf16 weights
    assert_within_tolerance(h, want, "f16 output, no flags")
    for bad in (pkg.FLAG_FORCE_TWO_STEP | pkg.FLAG_FORCE_MFMA, pkg.FLAG_FORCE_TWO_STEP | pkg.FLAG_FORCE_GENERIC):
        with pytest.raises(pkg.MI355QError):
            run_qgemm(ctx, pkg, ws, x, pkg.F32, bad)
    ws.destroy(); wp.destroy()


def test_two_step_in_a_plan_replayed_as_a_graph(pkg, ctx):
    """Two projections on the route inside one plan (they share the context's scratch matrix, in stream order), replayed
    eagerly and as a HIP graph with eager work between the replays: every replay equals the first eager result."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    m = 128                                       # beyond the 96 rows the streamed-weight kernel takes on blocks
    shapes = [(256, 512), (320, 1024)]
    ws, xs, ys = [], [], []
    for i, (n, k) in enumerate(shapes):
        words, s, z, _ = seeded_case(3400 + i, n, k, 4, 64)
        ws.append(ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_STAF_BLOCKS))
        xs.append(ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(3410 + i, m, k))))
        ys.append(ctx.alloc(m * n * 4))
    stream = ctx.stream_create()
    for i in range(2):
        ctx.qgemm(ws[i], xs[i], pkg.BF16, ys[i], pkg.F32, m, 0, 0, 0, stream)
    ctx.synchronize(stream)
    eager = [y.download(np.float32) for y in ys]
    assert all(np.all(np.isfinite(e)) for e in eager)
    plan = pkg.DispatchPlan(ctx)
    for i in range(2):
        plan.add_linear(ws[i], xs[i], pkg.BF16, ys[i], pkg.F32, m)
        assert [st.kernel_family for st in ws[i].plan_prefill_steps(m)] == ["dequantToBFloat", "libraryGEMM"]

    def scrub():
        for y in ys:
            ctx.fill(y, 0x7FC00000, stream)

    for rep in range(2):
        scrub(); plan.encode(stream); ctx.synchronize(stream)
        for y, want in zip(ys, eager):
            assert np.array_equal(y.download(np.float32), want), f"stream replay {rep}"
    plan.graph_build(stream)
    for rep in range(4):
        scrub(); plan.graph_launch(stream); ctx.synchronize(stream)
        for y, want in zip(ys, eager):
            assert np.array_equal(y.download(np.float32), want), f"graph replay {rep}"
        ctx.qgemm(ws[1], xs[1], pkg.BF16, ys[1], pkg.F32, m, 0, 0, 0, stream)      # eager work between the replays
        ctx.synchronize(stream)
    plan.destroy()
    for o in ws:
        o.destroy()
    for b in xs + ys:
        b.free()


def test_dense_entry_point_hands_long_products_to_the_library(pkg, ctx):
    """mi355q_gemm_bf16 (gemm_bf16_f32s of the reference) at 128 rows and more: same bars as the route above."""
    m, n, k = 300, 136, 768
    rng = np.random.default_rng(3500)
    b = bf16_round(rng.standard_normal((n, k)).astype(np.float32) * 0.05)
    x = act_rounded(kat.seeded_activations(3501, m, k), pkg.BF16, pkg)
    bd = ctx.upload(oracle.bf16_from_f32(b).reshape(n, k))
    xd = ctx.upload(oracle.bf16_from_f32(x).reshape(m, k))
    yd = ctx.alloc(m * n * 4)
    ctx.gemm_bf16(xd, pkg.BF16, bd, yd, pkg.F32, m, n, k)
    ctx.synchronize()
    assert_within_tolerance(yd.download(np.float32, (m, n)), oracle.gemm_f64(b, x), "dense entry point")
    for buf in (bd, xd, yd):
        buf.free()


@pytest.mark.parametrize("x_dtype_name,y_dtype_names", [("F16", ("F32", "F16")), ("F32", ("F32",))])
def test_two_step_f16_and_f32_activations(pkg, ctx, x_dtype_name, y_dtype_names):
    """f16 and fp32 activations (the reference's gemm_q*_g* and gemm_q*_g*_f32s signatures).  f16: the matrix is
    dequantised to f16 and the library multiplies in f16 with fp32 accumulation.  fp32 into fp32: bf16 weights, as the
    reference's gemm_bf16_f32s has them, against the activations split into two bf16 matrices (sixteen bits of every
    activation; two library products, the second accumulating).  Unforced, every layout takes the route from sixteen
    rows (the fused kernel reads bf16 only)."""
    x_dtype = getattr(pkg, x_dtype_name)
    n, k = 200, 1024
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    words, s, z, wq = seeded_case(3600, n, k, 4, 64)
    w_round = wq.astype(np.float16).astype(np.float32) if x_dtype == pkg.F16 else bf16_round(wq)
    for layout in (pkg.LAYOUT_PLANES, pkg.LAYOUT_STAF_BLOCKS):
        w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, layout)
        # f16 rows on 4-bit planes and blocks run on the streamed-weight kernel up to 96 rows (f16 weights there too)
        steps = w.plan_prefill_steps(200 if x_dtype == pkg.F16 else 64, x_dtype=x_dtype)
        want_kernels = (["dequant_q4_g64_f16", "hipblaslt_gemm_f16"] if x_dtype == pkg.F16
                        else ["dequant_q4_g64_bf16", "hipblaslt_gemm_bf16_x2"])
        assert [st.device_kernel for st in steps] == want_kernels
        for m in (16, 77, 300):
            x = act_rounded(kat.seeded_activations(3610 + m, m, k), x_dtype, pkg)
            # up to sixteen fp32 rows run on the planes' bf16 decode kernel as three bf16 rows each: unrounded weights
            exact = x_dtype == pkg.F32 and m <= 16 and layout == pkg.LAYOUT_PLANES
            want = oracle.gemm_f64(wq if exact else w_round, x)
            for yname in y_dtype_names:
                y_dtype = getattr(pkg, yname)
                say(f"two-step {x_dtype_name} -> {yname} layout {layout} M={m}")
                xd = ctx.upload(act_to_device_array(x, x_dtype, pkg))
                yd = ctx.alloc(m * n * (4 if y_dtype == pkg.F32 else 2))
                ctx.fill(yd, 0x7FC00000)
                ctx.qgemm(w, xd, x_dtype, yd, y_dtype, m); ctx.synchronize()
                assert_within_tolerance(out_from_device(yd, y_dtype, (m, n), pkg), want, f"{x_dtype_name}->{yname} M={m}")
                xd.free(); yd.free()
        w.destroy()


def test_timed_library_candidates_are_checked_against_the_first(pkg):
    """The first eager call of a problem times the library's ranked algorithms; one of them has returned a wrong matrix
    on a small odd problem (M = N = 17, K = 2176, bf16), so a candidate is kept only if its result agrees with that of
    the heuristic's first algorithm.  Fresh contexts time the candidates anew: every one must give the right product."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(3, 16)
    m, n, k = 17, 17, 2176
    w32 = kat.seeded_weights(3700, n, k)
    words, s, z = oracle.quantize_affine(w32, 3, 16, oracle.F16)
    wq = bf16_round(oracle.dequant_planes_f32(3, 16, n, k, words, s, z, oracle.F16))
    x = act_rounded(kat.seeded_activations(3701, m, k), pkg.BF16, pkg)
    want = oracle.gemm_f64(wq, x)
    for attempt in range(4):
        c = pkg.Context(0)
        w = c.weight_prepare_mlx(fmt, words, s, z, pkg.F16, pkg.LAYOUT_STAF_BLOCKS)
        assert [st.kernel_family for st in w.plan_prefill_steps(m)] == ["dequantToBFloat", "libraryGEMM"]
        xd = c.upload(act_to_device_array(x, pkg.BF16, pkg)); yd = c.alloc(m * n * 4)
        for call in range(2):                       # the call that times the candidates, and one with the algorithm kept
            c.fill(yd, 0x7FC00000)
            c.qgemm(w, xd, pkg.BF16, yd, pkg.F32, m); c.synchronize()
            got = yd.download(np.float32, (m, n))
            assert_within_tolerance(got, want, f"context {attempt}, call {call}")
        xd.free(); yd.free(); w.destroy(); c.close()


@pytest.mark.parametrize("x_dtype_name", ["BF16", "F16", "F32"])
def test_library_route_with_padded_result_rows_and_long_k(pkg, ctx, x_dtype_name):
    """Results whose row stride is not N, with K = 14336: the library has returned wrong matrices into such results
    (the algorithm its heuristic ranks first, strides N + 5 and N + 8 alike), so the route computes a padded result densely in
    scratch and copies it row by row.  All three forms of the route, the dense entry point, canary behind the rows."""
    x_dtype = getattr(pkg, x_dtype_name)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    n, k, m = 72, 14336, 128
    words, s, z, wq = seeded_case(3800, n, k, 4, 64)
    w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
    w_round = wq.astype(np.float16).astype(np.float32) if x_dtype == pkg.F16 else bf16_round(wq)
    x = act_rounded(kat.seeded_activations(3801, m, k), x_dtype, pkg)
    want = oracle.gemm_f64(w_round, x)
    xd = ctx.upload(act_to_device_array(x, x_dtype, pkg))
    for ys in (n, n + 5, n + 8):
        for y_dtype in ((pkg.F32,) if x_dtype == pkg.F32 else (pkg.F32, x_dtype)):
            say(f"padded result rows: x {x_dtype_name} y {y_dtype} stride {ys}")
            ysz = 4 if y_dtype == pkg.F32 else 2
            yd = ctx.alloc((m * ys * ysz + 3) // 4 * 4)
            ctx.fill(yd, 0x7FC00000 if ysz == 4 else 0x7FC07FC0)
            ctx.qgemm(w, xd, x_dtype, yd, y_dtype, m, 0, ys, pkg.FLAG_FORCE_TWO_STEP); ctx.synchronize()
            raw = yd.download(np.float32 if ysz == 4 else np.uint16)[: m * ys].reshape(m, ys)
            got = raw if ysz == 4 else (oracle.bf16_to_f32(raw).reshape(m, ys) if y_dtype == pkg.BF16 else raw.view(np.float16).astype(np.float32))
            assert np.all(np.isnan(got[:, n:])), "padding behind the rows overwritten"
            if ysz == 4:
                assert_within_tolerance(got[:, :n], want, f"x {x_dtype_name} y {y_dtype} stride {ys}")
            else:                                     # a 16-bit result adds its own rounding (2^-9 for bf16)
                assert rel_l2(got[:, :n], want) <= 3e-3, (x_dtype_name, y_dtype, ys)
            yd.free()
    if x_dtype == pkg.BF16:                        # the dense entry point on its own
        dense = ctx.alloc(n * k * 2)
        ctx.dequant_bf16(w, dense)
        for ys in (n + 5, n + 8):
            cd = ctx.alloc(m * ys * 4)
            ctx.fill(cd, 0x7FC00000)
            ctx.gemm_bf16(xd, pkg.BF16, dense, cd, pkg.F32, m, n, k, 0, ys); ctx.synchronize()
            got = cd.download(np.float32, (m, ys))
            assert np.all(np.isnan(got[:, n:]))
            assert_within_tolerance(got[:, :n], want, f"gemm_bf16 stride {ys}")
            cd.free()
        dense.free()
    xd.free(); w.destroy()


def test_one_stream_per_context_is_enforced(pkg):
    """The context's scratch is shared by its launches.  A launch that uses it on a second stream while work that used
    it on a first stream is still running is refused (MI355Q_ERR_INVALID_ARGUMENT) instead of racing; once the first
    stream has finished the second is served, and launches that keep to one stream never notice."""
    c = pkg.Context(0)
    try:
        fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
        n, k, m = 4096, 4096, 2048
        words, s, z = oracle.quantize_affine(kat.seeded_weights(3900, 64, k), 4, 64, oracle.BF16)
        words = np.tile(words, (n // 64, 1)); s = np.tile(s.reshape(64, -1), (n // 64, 1)); z = np.tile(z.reshape(64, -1), (n // 64, 1))
        w = c.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
        x = c.upload(oracle.bf16_from_f32(kat.seeded_activations(3901, m, k)))
        y1 = c.alloc(m * n * 2); y2 = c.alloc(m * n * 2)
        a, b = c.stream_create(), c.stream_create()
        two = pkg.FLAG_FORCE_TWO_STEP                      # the dense copy of the matrix lives in the context's scratch
        c.qgemm(w, x, pkg.BF16, y1, pkg.BF16, m, 0, 0, two, a); c.synchronize(a)      # (first call: timing, synchronous)
        for _ in range(20):
            c.qgemm(w, x, pkg.BF16, y1, pkg.BF16, m, 0, 0, two, a)                     # a few milliseconds of work on a
        with pytest.raises(pkg.MI355QError) as err:
            c.qgemm(w, x, pkg.BF16, y2, pkg.BF16, m, 0, 0, two, b)
        assert "another stream" in str(err.value)
        c.qgemm(w, x, pkg.BF16, y1, pkg.BF16, m, 0, 0, two, a)                         # the same stream goes on
        c.synchronize(a)
        c.qgemm(w, x, pkg.BF16, y2, pkg.BF16, m, 0, 0, two, b); c.synchronize(b)      # the first stream is done: served
        assert np.array_equal(y1.download(np.uint16, (m, n)), y2.download(np.uint16, (m, n)))
        c.stream_destroy(a); c.stream_destroy(b)
        x.free(); y1.free(); y2.free(); w.destroy()
    finally:
        c.close()
