"""GPU parity tests of the gated MLP's first half -- gate_proj + up_proj + swiglu / gelu_gated -- through the C ABI.

Reference: MLPFragment (Sources/MetalCompiler/Compilable/MLPFragment.swift:7-27) = batched gate + up projection, then
the elementwise kernel of Generator/MetalSourceGenerator+NormAndElementwise.swift:196-249, which reads gate and up back
from buffers of the activation type.  Expected values: the oracle's fp64 projections, rounded to the buffer type, through
the oracle's restatement of the elementwise kernel.  Bars: relative L2 <= 1e-3 and max-abs <= 2e-2 on fp32 results; a
16-bit result may differ from the expected one by one step of its type where the fp32 sums differ in their last bits.
"""
import sys

import numpy as np
import pytest

import kat
import oracle
from gpu_util import act_rounded, act_to_device_array, assert_within_tolerance, out_from_device, rel_l2, seeded_case

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, file=sys.stderr, flush=True)


def _o_dtype(pkg, d):
    return {pkg.F32: oracle.F32, pkg.BF16: oracle.BF16, pkg.F16: oracle.F16}[d]


def test_elementwise_kernel_closed_forms_and_oracle(pkg, ctx):
    """The elementwise step alone: closed forms (silu(0) = 0, gelu(0) = 0, large g -> g * u, very negative g -> -0 * u,
    u = 0 -> 0) and seeded values against the oracle, every buffer type, padded rows."""
    g = np.array([0.0, 30.0, -100.0, 1.0, -1.0, 5.0, 0.5, 88.0], np.float32)
    u = np.array([3.0, 2.0, 7.0, 1.0, 1.0, 0.0, -4.0, 0.5], np.float32)
    for kind in (pkg.GATED_SILU, pkg.GATED_GELU_TANH):
        gd, ud, od = ctx.upload(g), ctx.upload(u), ctx.alloc(g.size * 4)
        ctx.gated_activation(gd, ud, od, pkg.F32, g.size, activation=kind)
        ctx.synchronize()
        got = od.download(np.float32)
        assert got[0] == 0.0 and got[1] == 60.0 and got[5] == 0.0 and got[7] == 44.0
        assert got[2] == 0.0                                            # silu(-100) = -100 / (1 + inf) = -0
        want1 = 1.0 / (1.0 + np.exp(-1.0)) if kind == pkg.GATED_SILU else 0.5 * (1.0 + np.tanh(0.7978845608 * 1.044715))
        assert abs(got[3] - want1) < 2e-7
        assert np.allclose(got, oracle.gated_activation_f32(g, u, kind, oracle.F32), rtol=2e-6, atol=2e-6)
        for b in (gd, ud, od):
            b.free()
    rng = np.random.default_rng(5)
    seq, dim, stride = 3, 1000, 1008
    for dt in (pkg.F32, pkg.BF16, pkg.F16):
        gs = act_rounded((rng.standard_normal((seq, stride)) * 3).astype(np.float32), dt, pkg)
        us = act_rounded(rng.standard_normal((seq, stride)).astype(np.float32), dt, pkg)
        for kind in (pkg.GATED_SILU, pkg.GATED_GELU_TANH):
            gd, ud = ctx.upload(act_to_device_array(gs, dt, pkg)), ctx.upload(act_to_device_array(us, dt, pkg))
            od = ctx.alloc(seq * stride * (4 if dt == pkg.F32 else 2))
            ctx.fill(od, 0x7FC07FC0 if dt != pkg.F32 else 0x7FC00000)
            ctx.gated_activation(gd, ud, od, dt, dim, seq, stride, kind)
            ctx.synchronize()
            got = out_from_device(od, dt, (seq, stride), pkg)
            assert np.all(np.isnan(got[:, dim:])), "row padding was written"
            want = oracle.gated_activation_f32(gs[:, :dim], us[:, :dim], kind, _o_dtype(pkg, dt))
            step = {pkg.F32: 2e-6, pkg.BF16: 2.0 ** -7, pkg.F16: 2.0 ** -10}[dt]     # at most one step of the type
            # (1 + tanh cancels for negative g: the device's tanh and the host's differ by a few fp32 steps of |g u|)
            slack = 1e-6 * np.abs(gs[:, :dim] * us[:, :dim])
            assert np.all(np.abs(got[:, :dim] - want) <= step * np.maximum(np.abs(want), 1e-3) + slack), (dt, kind)
            for b in (gd, ud, od):
                b.free()


def _expected(pkg, wq_g, wq_u, x, kind, y_dtype):
    """Expected result and how far one step of the buffer type on the gate and up sums moves it."""
    gate = oracle.gemm_f64(wq_g, x).astype(np.float32)
    up = oracle.gemm_f64(wq_u, x).astype(np.float32)
    od = _o_dtype(pkg, y_dtype)
    want = oracle.gated_activation_f32(gate, up, kind, od)
    step = {pkg.F32: 2.0 ** -22, pkg.BF16: 2.0 ** -8, pkg.F16: 2.0 ** -11}[y_dtype]
    moved = np.zeros_like(want)
    for sg in (1 - step, 1 + step):
        for su in (1 - step, 1 + step):
            moved = np.maximum(moved, np.abs(oracle.gated_activation_f32(gate * np.float32(sg), up * np.float32(su), kind, od) - want))
    # ... and how far an absolute error of a few 1e-5 of the sums themselves (fp32 accumulation order; f16 code pairs with
    # f16 activations) moves it: |d act(g) u| <= 1.13 (|u| dg + |du|)
    moved += np.float32(4e-5) * (1.0 + np.abs(up))
    return want, moved


def _check(pkg, got, expected, y_dtype, what):
    want, moved = expected
    if y_dtype != pkg.F32:
        # the gate and up sums are rounded to the buffer type before the activation: a sum whose last fp32 bits differ
        # from the oracle's may round the other way, one step of the type, and the activation passes that on
        step = 2.0 ** -7 if y_dtype == pkg.BF16 else 2.0 ** -10
        # (a flipped rounding of the gate moves the product by up to two steps of the output, whose own rounding adds one)
        assert np.all(np.abs(got - want) <= moved + 3 * step * np.abs(want)), what
        assert rel_l2(got, want) <= 1e-3, what        # (max-abs 2e-2 is less than one bf16 step from |y| = 4 on)
        return
    assert_within_tolerance(got, want, what)


@pytest.mark.parametrize("bits,group,n,k", [(4, 64, 14336, 4096), (4, 128, 1000, 2048), (8, 32, 520, 4096), (3, 64, 300, 4096),
                                            (4, 64, 333, 8192)])
def test_gated_projection_one_row(pkg, ctx, bits, group, n, k):
    """M = 1 on split planes: one launch (a wavefront owns a gate row and the up row of the same index), every output
    type, bf16 and f16 activations, both activations; Llama-3-8B's gate / up shape among the cases."""
    wg, sg, zg, wq_g = seeded_case(6000 + bits, n, k, bits, group)
    wu, su, zu, wq_u = seeded_case(6100 + bits, n, k, bits, group)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
    g = ctx.weight_prepare_mlx(fmt, wg, sg, zg, pkg.BF16, pkg.LAYOUT_PLANES)
    u = ctx.weight_prepare_mlx(fmt, wu, su, zu, pkg.BF16, pkg.LAYOUT_PLANES)
    for xd in ((pkg.BF16, pkg.F16) if bits in (4, 8) else (pkg.BF16,)):
        x = act_rounded(kat.seeded_activations(6200 + k, 1, k), xd, pkg)
        xdev = ctx.upload(act_to_device_array(x, xd, pkg))
        for yd in (pkg.F32, pkg.BF16, pkg.F16):
            for kind in (pkg.GATED_SILU, pkg.GATED_GELU_TANH):
                say(f"gated q{bits}g{group} {k}->{n} x={xd} y={yd} act={kind}")
                ydev = ctx.alloc(n * (4 if yd == pkg.F32 else 2))
                ctx.gated_qgemm(g, u, xdev, xd, ydev, yd, 1, kind)
                ctx.synchronize()
                got = out_from_device(ydev, yd, (1, n), pkg) if yd != pkg.F32 else ydev.download(np.float32, (1, n))
                _check(pkg, got, _expected(pkg, wq_g, wq_u, x, kind, yd), yd, f"gated q{bits}g{group} y={yd}")
                ydev.free()
        xdev.free()
    g.destroy(); u.destroy()


def test_gated_projection_equals_batched_projection_then_elementwise(pkg, ctx):
    """Every other shape runs the two projections into scratch and then the elementwise kernel: M = 1 on blocks in place
    and on TILE16 records, M = 5, 40 and 300 on planes -- equal, bit for bit, to mi355q_batched_qgemm followed by
    mi355q_gated_activation_apply, and within the bar of the oracle."""
    n, k = 520, 2048
    wg, sg, zg, wq_g = seeded_case(6300, n, k, 4, 64)
    wu, su, zu, wq_u = seeded_case(6301, n, k, 4, 64)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    for layout, ms in ((pkg.LAYOUT_PLANES, (5, 40, 300)), (pkg.LAYOUT_TILE16, (1, 9)), (pkg.LAYOUT_STAF_BLOCKS, (1, 3))):
        sb = pkg.BF16
        if layout == pkg.LAYOUT_STAF_BLOCKS:       # blocks keep f16 headers: quantise with f16 scales
            wg2, sg2, zg2 = oracle.quantize_affine(kat.seeded_weights(6300, n, k), 4, 64, oracle.F16)
            wu2, su2, zu2 = oracle.quantize_affine(kat.seeded_weights(6301, n, k), 4, 64, oracle.F16)
            g = ctx.weight_prepare_mlx(fmt, wg2, sg2, zg2, pkg.F16, layout)
            u = ctx.weight_prepare_mlx(fmt, wu2, su2, zu2, pkg.F16, layout)
            dq_g = oracle.dequant_planes_f32(4, 64, n, k, wg2, sg2, zg2, oracle.F16)
            dq_u = oracle.dequant_planes_f32(4, 64, n, k, wu2, su2, zu2, oracle.F16)
        else:
            g = ctx.weight_prepare_mlx(fmt, wg, sg, zg, sb, layout)
            u = ctx.weight_prepare_mlx(fmt, wu, su, zu, sb, layout)
            dq_g, dq_u = wq_g, wq_u
        for m in ms:
            x = act_rounded(kat.seeded_activations(6400 + m, m, k), pkg.BF16, pkg)
            xdev = ctx.upload(act_to_device_array(x, pkg.BF16, pkg))
            yd = pkg.BF16
            say(f"gated layout={layout} M={m}")
            fused, gate_b, up_b, two = ctx.alloc(m * n * 2), ctx.alloc(m * n * 2), ctx.alloc(m * n * 2), ctx.alloc(m * n * 2)
            ctx.gated_qgemm(g, u, xdev, pkg.BF16, fused, yd, m, pkg.GATED_SILU)
            ctx.batched_qgemm([g, u], xdev, pkg.BF16, [gate_b, up_b], yd, m)
            ctx.gated_activation(gate_b, up_b, two, yd, n, m, 0, pkg.GATED_SILU)
            ctx.synchronize()
            a, b = fused.download(np.uint16, (m, n)), two.download(np.uint16, (m, n))
            assert np.array_equal(a, b), "gated call != batched projection + elementwise kernel"
            got = oracle.bf16_to_f32(a).reshape(m, n)
            if m <= 32:      # few rows: unrounded weights on every route (beyond, the weights are rounded to bf16)
                _check(pkg, got, _expected(pkg, dq_g, dq_u, x, pkg.GATED_SILU, yd), yd, f"layout {layout} M={m}")
            for t in (xdev, fused, gate_b, up_b, two):
                t.free()
        g.destroy(); u.destroy()


def test_gated_projection_rejects_mismatched_weights(pkg, ctx):
    wa, sa, za, _ = seeded_case(6500, 64, 256, 4, 64)
    wb, sb_, zb, _ = seeded_case(6501, 128, 256, 4, 64)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    a = ctx.weight_prepare_mlx(fmt, wa, sa, za, pkg.BF16, pkg.LAYOUT_PLANES)
    b = ctx.weight_prepare_mlx(fmt, wb, sb_, zb, pkg.BF16, pkg.LAYOUT_PLANES)
    x, y = ctx.alloc(256 * 2), ctx.alloc(128 * 4)
    with pytest.raises(pkg.MI355QError):
        ctx.gated_qgemm(a, b, x, pkg.BF16, y, pkg.F32, 1)
    with pytest.raises(pkg.MI355QError):
        ctx.gated_qgemm(a, a, x, pkg.BF16, y, pkg.F32, 1, activation=7)
    a.destroy(); b.destroy(); x.free(); y.free()


def test_gated_step_in_a_plan_replayed_as_a_graph(pkg, ctx):
    """The gated projection as a plan step: the record names the fused launch, and eager replay, a captured graph and
    the direct call give the same bits on every replay."""
    n, k = 2048, 4096
    wg, sg, zg, _ = seeded_case(6600, n, k, 4, 64)
    wu, su, zu, _ = seeded_case(6601, n, k, 4, 64)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    g = ctx.weight_prepare_mlx(fmt, wg, sg, zg, pkg.BF16, pkg.LAYOUT_PLANES)
    u = ctx.weight_prepare_mlx(fmt, wu, su, zu, pkg.BF16, pkg.LAYOUT_PLANES)
    x = act_rounded(kat.seeded_activations(6602, 1, k), pkg.BF16, pkg)
    xdev = ctx.upload(act_to_device_array(x, pkg.BF16, pkg))
    direct, planned = ctx.alloc(n * 2), ctx.alloc(n * 2)
    ctx.gated_qgemm(g, u, xdev, pkg.BF16, direct, pkg.BF16, 1, pkg.GATED_SILU)
    plan = pkg.DispatchPlan(ctx)
    plan.add_gated_mlp(g, u, xdev, pkg.BF16, planned, pkg.BF16, 1, pkg.GATED_SILU, layer_index=3, tensor_name="layers.3.mlp")
    rec, layer, name = plan.step(0)
    assert layer == 3 and name == "layers.3.mlp"
    assert rec.kernel_family == "gatedFusedQ4G64" and rec.device_kernel.endswith("+swiglu"), (rec.kernel_family, rec.device_kernel)
    stream = ctx.stream_create()
    plan.encode(stream)
    ctx.synchronize(stream)
    ctx.synchronize()
    want = direct.download(np.uint16)
    assert np.array_equal(planned.download(np.uint16), want)
    plan.graph_build(stream)
    for _ in range(3):
        ctx.fill(planned, 0x7FC07FC0, stream)
        plan.graph_launch(stream)
        ctx.synchronize(stream)
        assert np.array_equal(planned.download(np.uint16), want)
    plan.destroy()
    for t in (xdev, direct, planned):
        t.free()
    g.destroy(); u.destroy()


@pytest.mark.parametrize("layout_name,x_name", [("LAYOUT_PLANES", "BF16"), ("LAYOUT_STAF_BLOCKS", "BF16"), ("LAYOUT_PLANES", "F16")])
def test_gated_projection_on_the_prefill_kernel(pkg, ctx, layout_name, x_name):
    """Prompts: gate_proj and up_proj as the two column fragments of every wavefront of the wide-tile matrix-core kernel,
    activation(gate) * up in its epilogue, one launch.  Equal, bit for bit, to the two projections on that kernel
    followed by the elementwise kernel (same sums, same roundings), for ragged rows and columns, groups of 64 and 128,
    every output type, both activations and a padded result; the plan record says so."""
    layout, xd = getattr(pkg, layout_name), getattr(pkg, x_name)
    wide_flags = pkg.FLAG_FORCE_MFMA | pkg.FLAG_PROBE_WIDE
    for i, (m, n, k, group) in enumerate([(300, 260, 512, 64), (130, 515, 768, 128), (258, 128, 256, 64)]):
        fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, group)
        sbo, sbp = (oracle.F16, pkg.F16) if layout == pkg.LAYOUT_STAF_BLOCKS else (oracle.BF16, pkg.BF16)
        wg, sg, zg = oracle.quantize_affine(kat.seeded_weights(6500 + i, n, k), 4, group, sbo)
        wu, su, zu = oracle.quantize_affine(kat.seeded_weights(6510 + i, n, k), 4, group, sbo)
        g = ctx.weight_prepare_mlx(fmt, wg, sg, zg, sbp, layout)
        u = ctx.weight_prepare_mlx(fmt, wu, su, zu, sbp, layout)
        x = act_rounded(kat.seeded_activations(6520 + i, m, k), xd, pkg)
        xdev = ctx.upload(act_to_device_array(x, xd, pkg))
        for yd in (pkg.BF16, pkg.F32, pkg.F16):
            esz = 4 if yd == pkg.F32 else 2
            for kind in (pkg.GATED_SILU, pkg.GATED_GELU_TANH):
                for y_pad in (0, 8, 3):
                    say(f"gated wide {layout_name} x={x_name} {m}x{n}x{k} g{group} y={yd} act={kind} pad={y_pad}")
                    ys = n + y_pad
                    fused, gate_b, up_b, two = (ctx.alloc(m * ys * esz) for _ in range(4))
                    ctx.fill(fused, 0x7FC07FC0 if esz == 2 else 0x7FC00000)
                    ctx.fill(two, 0x7FC07FC0 if esz == 2 else 0x7FC00000)
                    ctx.gated_qgemm(g, u, xdev, xd, fused, yd, m, kind, 0, ys if y_pad else 0, pkg.FLAG_PROBE_WIDE)
                    ctx.qgemm(g, xdev, xd, gate_b, yd, m, 0, ys if y_pad else 0, wide_flags)
                    ctx.qgemm(u, xdev, xd, up_b, yd, m, 0, ys if y_pad else 0, wide_flags)
                    ctx.gated_activation(gate_b, up_b, two, yd, n, m, ys if y_pad else 0, kind)
                    ctx.synchronize()
                    dt = np.float32 if esz == 4 else np.uint16
                    a, b = fused.download(dt, (m, ys)), two.download(dt, (m, ys))
                    assert np.array_equal(a[:, :n], b[:, :n]), "one launch != two projections + elementwise kernel"
                    if y_pad:
                        pad = a[:, n:]
                        assert np.all(np.isnan(pad)) if esz == 4 else np.all(pad == 0x7FC0), "padding of the output rows was written"
                    for t in (fused, gate_b, up_b, two):
                        t.free()
        xdev.free(); g.destroy(); u.destroy()


def test_gated_projection_llama_prompt_as_dispatched(pkg, ctx):
    """Llama-3-8B's gate / up pair at 512 rows with no flags: one launch on the wide-tile kernel (the plan record names
    it), equal to the two projections and the elementwise kernel, and within the bar of the oracle on a column sample;
    the plan of 2048 rows names the same launch over 896 tiles."""
    n, k, m = 14336, 4096, 512
    wg, sg, zg, wq_g = seeded_case(6600, n, k, 4, 64)
    wu, su, zu, wq_u = seeded_case(6601, n, k, 4, 64)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    g = ctx.weight_prepare_mlx(fmt, wg, sg, zg, pkg.BF16, pkg.LAYOUT_PLANES)
    u = ctx.weight_prepare_mlx(fmt, wu, su, zu, pkg.BF16, pkg.LAYOUT_PLANES)
    x = act_rounded(kat.seeded_activations(6602, m, k), pkg.BF16, pkg)
    xdev = ctx.upload(act_to_device_array(x, pkg.BF16, pkg))
    fused, gate_b, up_b, two = (ctx.alloc(m * n * 2) for _ in range(4))
    plan = pkg.DispatchPlan(ctx)
    plan.add_gated_mlp(g, u, xdev, pkg.BF16, fused, pkg.BF16, m, activation=pkg.GATED_SILU)
    st, _, _ = plan.step(0)
    assert st.device_kernel == "qgemm_wide_q4_g64+swiglu" and st.kernel_family == "gatedFusedQ4G64", (st.device_kernel, st.kernel_family)
    far = pkg.DispatchPlan(ctx)
    far.add_gated_mlp(g, u, xdev, pkg.BF16, fused, pkg.BF16, 2048, activation=pkg.GATED_SILU)     # (described, not run)
    rec = far.step(0)[0]
    assert rec.kernel_family == "gatedFusedQ4G64" and rec.device_kernel == "qgemm_wide_q4_g64+swiglu" and tuple(rec.grid)[:2] == (896, 1), \
        (rec.kernel_family, rec.device_kernel, tuple(rec.grid))
    far.destroy()
    near = pkg.DispatchPlan(ctx)                  # one row of 128-row tiles: 112 workgroups, K in one part
    near.add_gated_mlp(g, u, xdev, pkg.BF16, fused, pkg.BF16, 128, activation=pkg.GATED_SILU)
    rec = near.step(0)[0]
    assert rec.kernel_family == "gatedFusedQ4G64" and rec.device_kernel == "qgemm_wide_q4_g64+swiglu" and tuple(rec.grid)[:2] == (112, 1), \
        (rec.kernel_family, rec.device_kernel, tuple(rec.grid))
    near.destroy()
    plan.encode(0)
    ctx.qgemm(g, xdev, pkg.BF16, gate_b, pkg.BF16, m)
    ctx.qgemm(u, xdev, pkg.BF16, up_b, pkg.BF16, m)
    ctx.gated_activation(gate_b, up_b, two, pkg.BF16, n, m, 0, pkg.GATED_SILU)
    ctx.synchronize()
    a, b = fused.download(np.uint16, (m, n)), two.download(np.uint16, (m, n))
    assert np.array_equal(a, b)
    cols = np.unique(np.concatenate([np.arange(0, n, n // 16), [1, 127, 128, n - 129, n - 1]]))
    rows = np.unique(np.concatenate([np.arange(0, m, m // 8), [255, 256, m - 1]]))
    bf = lambda w: oracle.bf16_to_f32(oracle.bf16_from_f32(w)).reshape(w.shape)
    want = _expected(pkg, np.ascontiguousarray(bf(wq_g[cols])), np.ascontiguousarray(bf(wq_u[cols])), np.ascontiguousarray(x[rows]),
                     pkg.GATED_SILU, pkg.BF16)
    got = oracle.bf16_to_f32(a).reshape(m, n)[np.ix_(rows, cols)]
    _check(pkg, got, want, pkg.BF16, "gated prompt")
    plan.destroy()
    for t in (xdev, fused, gate_b, up_b, two):
        t.free()
    g.destroy(); u.destroy()


@pytest.mark.parametrize("layout_name,x_name", [("LAYOUT_PLANES", "BF16"), ("LAYOUT_STAF_BLOCKS", "BF16"), ("LAYOUT_PLANES", "F16")])
def test_gated_projection_on_the_streamed_weight_kernel(pkg, ctx, layout_name, x_name):
    """A few dozen rows: gate_proj and up_proj as the two row blocks of every workgroup of the streamed-weight kernel,
    activation(gate) * up in its epilogue, one launch.  Equal, bit for bit, to the two projections on that kernel (K in
    one part there too: K below 2048) followed by the elementwise kernel, for one to three blocks of 32 activation
    rows (the first with unrounded weights), ragged columns, every code width the kernel reads, every output type, both
    activations and a padded result."""
    layout, xd = getattr(pkg, layout_name), getattr(pkg, x_name)
    cases = [(40, 100, 512, 4, 64), (96, 70, 768, 4, 128), (18, 33, 256, 8, 32), (64, 96, 1024, 8, 64),
             (34, 65, 320, 3, 64), (70, 40, 192, 6, 64), (20, 64, 128, 2, 64), (66, 31, 256, 5, 64)]
    for i, (m, n, k, bits, group) in enumerate(cases):
        fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
        sbo, sbp = (oracle.F16, pkg.F16) if layout == pkg.LAYOUT_STAF_BLOCKS else (oracle.BF16, pkg.BF16)
        wg, sg, zg = oracle.quantize_affine(kat.seeded_weights(6700 + i, n, k), bits, group, sbo)
        wu, su, zu = oracle.quantize_affine(kat.seeded_weights(6720 + i, n, k), bits, group, sbo)
        g = ctx.weight_prepare_mlx(fmt, wg, sg, zg, sbp, layout)
        u = ctx.weight_prepare_mlx(fmt, wu, su, zu, sbp, layout)
        x = act_rounded(kat.seeded_activations(6740 + i, m, k), xd, pkg)
        xdev = ctx.upload(act_to_device_array(x, xd, pkg))
        for yd in (pkg.BF16, pkg.F32, pkg.F16):
            esz = 4 if yd == pkg.F32 else 2
            for kind in (pkg.GATED_SILU, pkg.GATED_GELU_TANH):
                for y_pad in (0, 5):
                    say(f"gated stream {layout_name} x={x_name} {m}x{n}x{k} q{bits} g{group} y={yd} act={kind} pad={y_pad}")
                    ys = n + y_pad
                    fused, gate_b, up_b, two = (ctx.alloc(m * ys * esz) for _ in range(4))
                    ctx.fill(fused, 0x7FC07FC0 if esz == 2 else 0x7FC00000)
                    ctx.fill(two, 0x7FC07FC0 if esz == 2 else 0x7FC00000)
                    ctx.gated_qgemm(g, u, xdev, xd, fused, yd, m, kind, 0, ys if y_pad else 0, pkg.FLAG_FORCE_STREAM)
                    ctx.qgemm(g, xdev, xd, gate_b, yd, m, 0, ys if y_pad else 0, pkg.FLAG_FORCE_STREAM)
                    ctx.qgemm(u, xdev, xd, up_b, yd, m, 0, ys if y_pad else 0, pkg.FLAG_FORCE_STREAM)
                    ctx.gated_activation(gate_b, up_b, two, yd, n, m, ys if y_pad else 0, kind)
                    ctx.synchronize()
                    dt = np.float32 if esz == 4 else np.uint16
                    a, b = fused.download(dt, (m, ys)), two.download(dt, (m, ys))
                    assert np.array_equal(a[:, :n], b[:, :n]), "one launch != two projections + elementwise kernel"
                    if y_pad:
                        pad = a[:, n:]
                        assert np.all(np.isnan(pad)) if esz == 4 else np.all(pad == 0x7FC0), "padding of the output rows was written"
                    for t in (fused, gate_b, up_b, two):
                        t.free()
        plan = pkg.DispatchPlan(ctx)
        out = ctx.alloc(m * n * 2)
        plan.add_gated_mlp(g, u, xdev, xd, out, pkg.BF16, m, activation=pkg.GATED_SILU, flags=pkg.FLAG_FORCE_STREAM)
        st = plan.step(0)[0]
        assert st.device_kernel == f"qgemm_stream_q{bits}_g{group}+swiglu" and st.kernel_family == f"gatedFusedQ{bits}G{group}", \
            (st.device_kernel, st.kernel_family)
        assert tuple(st.grid)[:2] == ((n + 31) // 32, 1) and st.rows_per_workgroup == 32
        plan.destroy()
        out.free(); xdev.free(); g.destroy(); u.destroy()


def test_gated_projection_llama_64_rows_as_dispatched(pkg, ctx):
    """Llama-3-8B's gate / up pair at 64 rows with no flags: one launch of the streamed-weight kernel (the plan record
    names it, a graph replays it), equal to the two projections on that kernel and the elementwise kernel, and within the
    bar of the oracle on a column sample."""
    n, k, m = 14336, 4096, 64
    wg, sg, zg, wq_g = seeded_case(6800, n, k, 4, 64)
    wu, su, zu, wq_u = seeded_case(6801, n, k, 4, 64)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    g = ctx.weight_prepare_mlx(fmt, wg, sg, zg, pkg.BF16, pkg.LAYOUT_PLANES)
    u = ctx.weight_prepare_mlx(fmt, wu, su, zu, pkg.BF16, pkg.LAYOUT_PLANES)
    x = act_rounded(kat.seeded_activations(6802, m, k), pkg.BF16, pkg)
    xdev = ctx.upload(act_to_device_array(x, pkg.BF16, pkg))
    fused, gate_b, up_b, two = (ctx.alloc(m * n * 2) for _ in range(4))
    stream = ctx.stream_create()
    plan = pkg.DispatchPlan(ctx)
    plan.add_gated_mlp(g, u, xdev, pkg.BF16, fused, pkg.BF16, m, activation=pkg.GATED_SILU)
    st, _, _ = plan.step(0)
    assert st.device_kernel == "qgemm_stream_q4_g64+swiglu" and st.kernel_family == "gatedFusedQ4G64", (st.device_kernel, st.kernel_family)
    assert tuple(st.grid)[:2] == (448, 1)
    ctx.qgemm(g, xdev, pkg.BF16, gate_b, pkg.BF16, m, flags=pkg.FLAG_FORCE_STREAM)
    ctx.qgemm(u, xdev, pkg.BF16, up_b, pkg.BF16, m, flags=pkg.FLAG_FORCE_STREAM)
    ctx.gated_activation(gate_b, up_b, two, pkg.BF16, n, m, 0, pkg.GATED_SILU)
    ctx.synchronize()
    b = two.download(np.uint16, (m, n))
    plan.graph_build(stream)
    for _ in range(3):
        ctx.fill(fused, 0x7FC07FC0, stream)
        plan.graph_launch(stream)
        ctx.synchronize(stream)
        assert np.array_equal(fused.download(np.uint16, (m, n)), b)
    a = fused.download(np.uint16, (m, n))
    cols = np.unique(np.concatenate([np.arange(0, n, n // 16), [1, 31, 32, 63, 64, n - 33, n - 1]]))
    rows = np.unique(np.concatenate([np.arange(0, m, m // 8), [31, 32, m - 1]]))
    bf = lambda w: oracle.bf16_to_f32(oracle.bf16_from_f32(w)).reshape(w.shape)
    want = _expected(pkg, np.ascontiguousarray(bf(wq_g[cols])), np.ascontiguousarray(bf(wq_u[cols])), np.ascontiguousarray(x[rows]),
                     pkg.GATED_SILU, pkg.BF16)
    got = oracle.bf16_to_f32(a).reshape(m, n)[np.ix_(rows, cols)]
    _check(pkg, got, want, pkg.BF16, "gated 64 rows")
    plan.destroy()
    ctx.stream_destroy(stream)
    for t in (xdev, fused, gate_b, up_b, two):
        t.free()
    g.destroy(); u.destroy()


def test_gated_projection_forced_onto_the_streamed_weight_kernel_keeps_k_in_one_part(pkg, ctx):
    """Few outputs and a long K, where a projection alone splits K over workgroups: forced onto the streamed-weight kernel
    the gated launch walks K in one part (a partial sum cannot be gated) and agrees with the two projections (K in
    parts, another order of the fp32 sums) followed by the elementwise kernel to 1e-5 of the largest output."""
    m, n, k = 48, 96, 4096
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    wg, sg, zg = oracle.quantize_affine(kat.seeded_weights(6900, n, k), 4, 64, oracle.BF16)
    wu, su, zu = oracle.quantize_affine(kat.seeded_weights(6901, n, k), 4, 64, oracle.BF16)
    g = ctx.weight_prepare_mlx(fmt, wg, sg, zg, pkg.BF16, pkg.LAYOUT_PLANES)
    u = ctx.weight_prepare_mlx(fmt, wu, su, zu, pkg.BF16, pkg.LAYOUT_PLANES)
    assert g.plan_prefill_steps(m, 0, pkg.BF16, flags=pkg.FLAG_FORCE_STREAM)[0].grid[1] > 1, "the projection alone is meant to split K"
    x = act_rounded(kat.seeded_activations(6902, m, k), pkg.BF16, pkg)
    xdev = ctx.upload(act_to_device_array(x, pkg.BF16, pkg))
    fused, gate_b, up_b, two = (ctx.alloc(m * n * 4) for _ in range(4))
    ctx.gated_qgemm(g, u, xdev, pkg.BF16, fused, pkg.F32, m, pkg.GATED_SILU, 0, 0, pkg.FLAG_FORCE_STREAM)
    ctx.qgemm(g, xdev, pkg.BF16, gate_b, pkg.F32, m, 0, 0, pkg.FLAG_FORCE_STREAM)
    ctx.qgemm(u, xdev, pkg.BF16, up_b, pkg.F32, m, 0, 0, pkg.FLAG_FORCE_STREAM)
    ctx.gated_activation(gate_b, up_b, two, pkg.F32, n, m, 0, pkg.GATED_SILU)
    ctx.synchronize()
    a, b = fused.download(np.float32, (m, n)), two.download(np.float32, (m, n))
    assert np.all(np.isfinite(a)) and float(np.max(np.abs(a - b))) <= 1e-5 * float(np.max(np.abs(b))), float(np.max(np.abs(a - b)))
    plan = pkg.DispatchPlan(ctx)
    plan.add_gated_mlp(g, u, xdev, pkg.BF16, fused, pkg.F32, m, activation=pkg.GATED_SILU, flags=pkg.FLAG_FORCE_STREAM)
    st = plan.step(0)[0]
    assert st.device_kernel == "qgemm_stream_q4_g64+swiglu" and tuple(st.grid)[:2] == (3, 1), (st.device_kernel, tuple(st.grid))
    plan.destroy()
    for t in (xdev, fused, gate_b, up_b, two):
        t.free()
    g.destroy(); u.destroy()
