"""GPU parity tests of fp32 and f16 activations at a few rows on the kernels that compute in bf16 (the f32s and f16
signatures of gemv_q{b}_g{g} / gemm_q{b}_g{g}, Sources/MetalCompiler/Generator/MetalSourceGenerator+Quantized.swift:496-575,
:22-156) through the C ABI.  Every fp32 row is split on the device into three bf16 rows whose sum is the row exactly;
the bf16 decode kernel of the layout runs on those rows and the partial results of a row are added.  f16 rows are
split into two bf16 rows inside the matrix-core kernels themselves.  Either way the matrix is read once per launch and
every product is exact.

Bars: against an fp64 accumulation of the dequantised weights and the UNROUNDED fp32 activations, relative L2 <= 1e-5
(rounding the activations to bf16 would give 1e-3); a case that needs all three parts and is exactly representable is
compared exactly; padding of activation and output rows is neither read into the result nor written.
"""
import sys

import numpy as np
import pytest

import kat
import oracle
from gpu_util import Case, out_from_device, rel_l2, seeded_case

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, file=sys.stderr, flush=True)


def run_f32(ctx, pkg, w, x, y_dtype=None, flags=0, xpad=0, ypad=0, use_qgemm=False, x_dtype=None):
    y_dtype = pkg.F32 if y_dtype is None else y_dtype
    x_dtype = pkg.F32 if x_dtype is None else x_dtype
    m, k = x.shape
    n = int(w.info.n_rows)
    xh = np.full((m, k + xpad), 6e4, np.float32); xh[:, :k] = x
    xd = ctx.upload(xh if x_dtype == pkg.F32 else xh.astype(np.float16).view(np.uint16))
    yd = ctx.alloc(m * (n + ypad) * (4 if y_dtype == pkg.F32 else 2))
    ctx.fill(yd, 0x7FC07FC0 if y_dtype != pkg.F32 else 0x7FC00000)
    (ctx.qgemm if use_qgemm else ctx.qgemv)(w, xd, x_dtype, yd, y_dtype, m, k + xpad, (n + ypad) if ypad else 0, flags)
    ctx.synchronize()
    y = out_from_device(yd, y_dtype, (m, n + ypad), pkg)
    xd.free(); yd.free()
    assert np.all(np.isnan(y[:, n:]))
    return y[:, :n]


LAYOUTS = [("planes", 4, 64, 16), ("planes", 4, 128, 16), ("planes", 8, 32, 16), ("planes", 3, 64, 2), ("planes", 6, 64, 2),
           ("tile16", 4, 64, 16), ("staf", 4, 64, 2), ("staf", 5, 32, 2)]


@pytest.mark.parametrize("layout,bits,group,most", LAYOUTS, ids=lambda v: str(v))
def test_f32_rows_full_mantissas(pkg, ctx, layout, bits, group, most):
    """Seeded weights, activations with all 24 significant bits in use, every row count the route takes for the layout
    (up to three launches of sixteen rows on TILE16 records and 4- / 8-bit planes, one launch of eight rows
    elsewhere); one more row takes another route (or the streamed-weight kernel on the split rows) and still meets the
    common bar."""
    lay = {"planes": pkg.LAYOUT_PLANES, "tile16": pkg.LAYOUT_TILE16, "staf": pkg.LAYOUT_STAF_BLOCKS}[layout]
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
    for i, (n, k) in enumerate([(200, 1024), (70, 4096 + 256)]):
        words, s, z, wq = seeded_case(5100 + i + bits + group, n, k, bits, group)
        w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, lay)
        for m in ([1, 2, 3] if most == 2 else [1, 2, 5, 6, 11, 16, 17]):
            say(f"f32 rows {layout} q{bits} g{group} {k}->{n} M={m}")
            x = kat.seeded_activations(5200 + m, m, k).astype(np.float32)
            x *= np.float32(1.0) + np.float32(2.0 ** -23) * (np.arange(k, dtype=np.float32) % 7)   # low mantissa bits in use
            want = oracle.gemm_f64(wq, x)
            st = w.plan_prefill_steps(m, x_dtype=pkg.F32)[0]
            got = run_f32(ctx, pkg, w, x, use_qgemm=True)
            if m <= most:
                assert st.device_kernel.startswith("split_f32_bf16x3+"), st.device_kernel
                assert rel_l2(got, want) <= 1e-5, (m, rel_l2(got, want))
                if m <= 8:
                    assert w.plan_decode_step(m, pkg.F32).device_kernel == st.device_kernel
                    assert np.array_equal(run_f32(ctx, pkg, w, x), got)
            else:
                # beyond the small-batch launches: the split rows on the streamed-weight kernel where it reads the weight
                # (planes and blocks of the widths it takes: unrounded weights up to 32 bf16 rows, bf16 weights beyond), else another route
                streams = layout != "tile16" and (bits in (4, 8) or group == 64)     # what the streamed-weight kernel reads
                assert st.device_kernel.startswith("split_f32_bf16x3+qgemm_stream") == streams, st.device_kernel
                if streams and 3 * m <= 32:
                    assert rel_l2(got, want) <= 1e-5, (m, rel_l2(got, want))
                assert rel_l2(got, want) <= 3e-3        # from sixteen rows the weights are rounded to bf16 once
        w.destroy()


def test_f32_rows_exact_values_padding_and_output_types(pkg, ctx):
    """Exact case: one activation per row is non-zero, v = (2^16 + odd) / 2^17, a value of 17 significant bits that
    needs all three bf16 parts (8 + 8 + 1); with power-of-two scales and small integer zeros every product is exact and
    y = (s q + z) v has at most 23 significant bits, so the fp32 result must equal it bit for bit.  Then seeded rows with
    padded activation rows (poison behind K) and padded output rows (canary kept); bf16 and f16 outputs are the rounded
    fp32 ones; forced, the per-code kernel agrees."""
    rng = np.random.default_rng(5300)
    n, k = 50, 512
    codes = rng.integers(0, 16, (n, k), dtype=np.uint8)
    scales = rng.choice([0.5, 1.0, 2.0], (n, k // 64)); zeros = rng.integers(-4, 5, (n, k // 64)).astype(np.float64)
    case = Case(4, 64, codes, scales, zeros)
    wq = scales.repeat(64, axis=1) * codes + zeros.repeat(64, axis=1)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    for layout in (pkg.LAYOUT_PLANES, pkg.LAYOUT_TILE16, pkg.LAYOUT_STAF_BLOCKS):
        w = ctx.weight_prepare_mlx(fmt, *case.planes(pkg.BF16, pkg), pkg.BF16, layout)
        for m, xpad, ypad in ((1, 0, 0), (2, 8, 3), (5, 4, 0)):
            if 3 * m > 8 and layout == pkg.LAYOUT_STAF_BLOCKS:
                continue
            x = np.zeros((m, k), np.float32)
            pos = rng.choice(k, m, replace=False)
            for r in range(m):
                x[r, pos[r]] = np.float32(((1 << 16) + 2 * int(rng.integers(0, 1 << 15)) + 1) / float(1 << 17)) * (-1) ** r
            want = x.astype(np.float64) @ wq.T
            assert np.array_equal(want.astype(np.float32).astype(np.float64), want)
            got = run_f32(ctx, pkg, w, x, xpad=xpad, ypad=ypad)
            assert np.array_equal(got.astype(np.float64), want), (layout, m)
            x = kat.seeded_activations(5310 + m, m, k)
            want = oracle.gemm_f64(wq, x)
            got = run_f32(ctx, pkg, w, x, xpad=xpad, ypad=ypad)
            assert rel_l2(got, want) <= 1e-5, (layout, m, rel_l2(got, want))
            for yd in (pkg.BF16, pkg.F16):
                low = run_f32(ctx, pkg, w, x, y_dtype=yd, xpad=xpad, ypad=ypad)
                ref = oracle.bf16_to_f32(oracle.bf16_from_f32(got)).reshape(got.shape) if yd == pkg.BF16 \
                    else got.astype(np.float16).astype(np.float32)
                assert np.array_equal(low, ref), (layout, m, yd)
            slow = run_f32(ctx, pkg, w, x, flags=pkg.FLAG_FORCE_GENERIC, xpad=xpad, ypad=ypad)
            assert rel_l2(slow, want) <= 1e-5
        w.destroy()


def test_f32_rows_non_finite_activation_and_graph_replay(pkg, ctx):
    """An infinite activation stays in the first bf16 part (the output row is non-finite where its weight is not zero,
    finite rows are untouched); a finite one above the largest bf16 (its rounding to bf16 is infinite) takes the largest
    bf16 as its first part and a remainder, so its parts never cancel into NaN (the row overflows to infinity inside the
    bf16 kernels, whose code values carry an offset of 128); a plan with fp32 rows replays as a HIP graph with the same
    result every time."""
    n, k, m = 64, 1024, 4
    words, s, z, wq = seeded_case(5400, n, k, 4, 64)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
    x = kat.seeded_activations(5401, m, k).astype(np.float32)
    x[1, 17] = np.inf
    x[3, 29] = 3.4e38
    got = run_f32(ctx, pkg, w, x)
    assert not np.any(np.isfinite(got[1][wq[:, 17] != 0]))
    assert not np.any(np.isnan(got[3]))
    fin = oracle.gemm_f64(wq, x[[0, 2]])
    assert rel_l2(got[[0, 2]], fin) <= 1e-5
    x[1, 17] = 0.25
    x[3, 29] = 0.5
    xd = ctx.upload(x); yd = ctx.alloc(m * n * 4)
    plan = pkg.DispatchPlan(ctx)
    plan.add_linear(w, xd, pkg.F32, yd, pkg.F32, m)
    stream = ctx.stream_create()
    plan.encode(stream); ctx.synchronize(stream)
    eager = yd.download(np.float32, (m, n)).copy()
    assert rel_l2(eager, oracle.gemm_f64(wq, x)) <= 1e-5
    plan.graph_build(stream)
    for _ in range(3):
        ctx.fill(yd, 0x7FC00000, stream)
        plan.graph_launch(stream); ctx.synchronize(stream)
        assert np.array_equal(yd.download(np.float32, (m, n)), eager)
    plan.destroy(); ctx.stream_destroy(stream)
    xd.free(); yd.free(); w.destroy()


@pytest.mark.parametrize("layout", ["tile16", "planes"])
def test_f16_rows_on_the_matrix_core_kernels(pkg, ctx, layout):
    """f16 activations (the reference's decode type) on the kernels that compute in bf16 on the matrix cores: a row is
    staged inside the kernel as two bf16 rows (the upper eight significant bits, the remaining three) and the two
    partial results are added before the store -- up to eight f16 rows a launch on TILE16 records, three to eight on
    4-bit planes (below, the f16 dot-product kernels), more rows in steps of eight on the records and on the
    streamed-weight kernel on the planes.  One-hot rows with an 11-bit value
    (1024 + odd) / 2048, which needs both parts, must come out bit for bit; seeded f16 rows to 1e-5 of the fp64
    reference on the same f16 values; padded rows; all output types."""
    lay = {"planes": pkg.LAYOUT_PLANES, "tile16": pkg.LAYOUT_TILE16}[layout]
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    rng = np.random.default_rng(5500)
    n, k = 130, 1024
    codes = rng.integers(0, 16, (n, k), dtype=np.uint8)
    scales = rng.choice([0.5, 1.0, 2.0], (n, k // 64)); zeros = rng.integers(-4, 5, (n, k // 64)).astype(np.float64)
    case = Case(4, 64, codes, scales, zeros)
    wq = scales.repeat(64, axis=1) * codes + zeros.repeat(64, axis=1)
    w = ctx.weight_prepare_mlx(fmt, *case.planes(pkg.BF16, pkg), pkg.BF16, lay)
    fast = "gemv_tile16_q4_g64" if layout == "tile16" else "gemv_mfma_planes_q4_g64"
    for m in (1, 2, 3, 4, 5, 7, 8, 9, 13, 15):
        say(f"f16 rows {layout} M={m}")
        st = w.plan_prefill_steps(m, x_dtype=pkg.F16)[0]
        if layout == "planes" and m > 8:        # beyond one launch of eight f16 rows: the streamed-weight kernel (f16 weights)
            assert st.device_kernel == "qgemm_stream_q4_g64", (m, st.device_kernel)
        else:
            assert (st.device_kernel == fast) == (layout == "tile16" or m >= 3), (m, st.device_kernel)
        assert m > 8 or not st.used_fallback
        x = np.zeros((m, k), np.float32)
        pos = rng.choice(k, m, replace=False)
        for r in range(m):
            x[r, pos[r]] = np.float32((1024 + 2 * int(rng.integers(0, 512)) + 1) / 2048.0) * (-1) ** r
        want = x.astype(np.float64) @ wq.T
        got = run_f32(ctx, pkg, w, x, use_qgemm=True, x_dtype=pkg.F16, xpad=8 if m % 2 else 0, ypad=3 if m % 3 == 0 else 0)
        assert np.array_equal(got.astype(np.float64), want), (layout, m)
        x = kat.seeded_activations(5510 + m, m, k).astype(np.float16).astype(np.float32)
        got = run_f32(ctx, pkg, w, x, use_qgemm=True, x_dtype=pkg.F16)
        assert rel_l2(got, oracle.gemm_f64(wq, x)) <= 1e-5, (layout, m)
        if m <= 8:
            assert np.array_equal(run_f32(ctx, pkg, w, x, x_dtype=pkg.F16), got)
            for yd in (pkg.BF16, pkg.F16):
                low = run_f32(ctx, pkg, w, x, y_dtype=yd, x_dtype=pkg.F16)
                ref = oracle.bf16_to_f32(oracle.bf16_from_f32(got)).reshape(got.shape) if yd == pkg.BF16 \
                    else got.astype(np.float16).astype(np.float32)
                assert np.array_equal(low, ref), (layout, m, yd)
    w.destroy()


def test_f16_rows_long_k_parts_and_eight_bit_planes(pkg, ctx):
    """Rows of 14336 codes at eight f16 rows (sixteen staged rows) overflow the staged copy: K parts with folded
    partial results; 8-bit planes in groups of 32 take f16 rows on the same kernel."""
    for lay, bits, group, n, k, ms in ((pkg.LAYOUT_TILE16, 4, 64, 48, 14336, (4, 8)), (pkg.LAYOUT_PLANES, 4, 64, 48, 14336, (4, 8)),
                                       (pkg.LAYOUT_PLANES, 8, 32, 100, 2048, (3, 8)), (pkg.LAYOUT_PLANES, 4, 128, 100, 2048, (3, 6))):
        fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
        words, s, z, wq = seeded_case(5700 + bits + group, n, k, bits, group)
        w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, lay)
        for m in ms:
            say(f"f16 rows layout {lay} q{bits} g{group} {k}->{n} M={m}")
            x = kat.seeded_activations(5710 + m, m, k).astype(np.float16).astype(np.float32)
            got = run_f32(ctx, pkg, w, x, x_dtype=pkg.F16)
            assert rel_l2(got, oracle.gemm_f64(wq, x)) <= 1e-5, (lay, bits, m, rel_l2(got, oracle.gemm_f64(wq, x)))
        w.destroy()


def test_batched_projections_other_activation_types(pkg, ctx):
    """q+k+v / gate+up with f16 rows on TILE16 records (one shared launch that stages the f16 rows itself) and fp32 rows
    on planes and blocks (split once into bf16 rows, one shared bf16 launch, one sum per projection): the same bits as
    the separate calls."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    for layout, x_dtype, npdt, ms in ((pkg.LAYOUT_TILE16, pkg.F16, np.float16, (1, 3, 8)),
                                      (pkg.LAYOUT_PLANES, pkg.F32, np.float32, (1, 2, 5)),
                                      (pkg.LAYOUT_STAF_BLOCKS, pkg.F32, np.float32, (1, 2))):
        ns, k = (384, 96, 96), 1024
        ws, wqs = [], []
        for i, n in enumerate(ns):
            words, s, z, wq = seeded_case(5600 + i, n, k, 4, 64)
            ws.append(ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, layout)); wqs.append(wq)
        for m in ms:
            say(f"batched split layout {layout} dtype {x_dtype} M={m}")
            x = kat.seeded_activations(5610 + m, m, k).astype(npdt)
            xd = ctx.upload(x.view(np.uint16) if npdt == np.float16 else x)
            yds = [ctx.alloc(m * n * 4) for n in ns]
            ctx.batched_qgemm(ws, xd, x_dtype, yds, pkg.F32, m); ctx.synchronize()
            for j, n in enumerate(ns):
                fused = yds[j].download(np.float32, (m, n))
                alone = run_f32(ctx, pkg, ws[j], x.astype(np.float32), x_dtype=x_dtype, use_qgemm=True)
                if layout == pkg.LAYOUT_STAF_BLOCKS:
                    # the streamed-weight kernel: the K parts follow the launch's workgroup count, so the order of the
                    # fp32 sums may differ between the shared launch and a launch alone
                    assert rel_l2(fused, alone) <= 2e-6, (layout, m, j)
                else:
                    assert np.array_equal(fused, alone), (layout, m, j)
                assert rel_l2(fused, oracle.gemm_f64(wqs[j], x.astype(np.float32))) <= 1e-5
            xd.free()
            for b in yds:
                b.free()
        for w in ws:
            w.destroy()


def test_output_head_with_fp32_and_f16_rows(pkg, ctx):
    """The output head with activation types the fused head kernels do not read (fp32 anywhere, f16 on TILE16 records):
    the projection takes its fast route to fp32 logits, an arg-max launch picks the token.  Logits to 1e-5 of the fp64
    reference on the unrounded activations, token = lowest-index argmax of the device's logits and of the reference."""
    n, k = 8192, 2048
    words, s, z, wq = seeded_case(5800, n, k, 4, 64)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    for layout, x_dtype in ((pkg.LAYOUT_PLANES, pkg.F32), (pkg.LAYOUT_TILE16, pkg.F32), (pkg.LAYOUT_TILE16, pkg.F16),
                            (pkg.LAYOUT_STAF_BLOCKS, pkg.F32)):
        w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, layout)
        x = kat.seeded_activations(5801, 1, k)
        if x_dtype == pkg.F16:
            x = x.astype(np.float16).astype(np.float32)
        want = oracle.gemm_f64(wq, x)[0]
        top2 = np.sort(want)[-2:]
        assert top2[1] - top2[0] > 1e-3, "seed gives a near-tie; pick another"
        xd = ctx.upload(x if x_dtype == pkg.F32 else x.astype(np.float16).view(np.uint16))
        logits = ctx.alloc(n * 4); ctx.fill(logits, 0x7FC00000)
        tok = ctx.upload(np.array([-7], np.int32))
        for _ in range(2):
            ctx.lmhead_argmax(w, xd, x_dtype, logits, tok); ctx.synchronize()
            got = logits.download(np.float32)
            assert rel_l2(got, want) <= 1e-5, (layout, x_dtype, rel_l2(got, want))
            token = int(tok.download(np.int32)[0])
            assert token == oracle.argmax_lowest(got) == int(np.argmax(want))
        w.destroy(); xd.free(); logits.free(); tok.free()
