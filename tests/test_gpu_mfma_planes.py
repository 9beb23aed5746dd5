"""GPU parity tests of the small-batch matrix-core kernel over the split planes (4-bit codes in groups of 64 and 128,
8-bit codes in groups of 32, 64 and 128), through the C ABI: the projections of gemv_q4_g64 / gemm_q4_g64 and
gemv_q8_g32 / gemm_q8_g32 of the reference
(MetalSourceGenerator+Quantized.swift:496-575, :22-156) for 4 <= M <= 16 rows per launch on the layout that serves M = 1
(up to eight rows the two quantisation groups of a block are kept apart in the M dimension, above with two products).

Bars: fp32 outputs within relative L2 <= 1e-3 and max-abs <= 2e-2 of an fp64 accumulation of the dequantised weights
(exact codes, no rounding of the weights); bf16 outputs equal bf16_rne(fp32 outputs); exactly representable cases are
compared exactly; a fused launch of two or three projections equals the separate launches bit for bit.
"""
import sys

import numpy as np
import pytest

import kat
import oracle
from gpu_util import Case, act_rounded, assert_within_tolerance, out_from_device, run_gemv, seeded_case

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, file=sys.stderr, flush=True)


def _fmt(pkg, group=64, bits=4):
    return pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)


@pytest.mark.parametrize("bits,group", [(4, 64), (4, 128), (8, 32), (8, 64), (8, 128)])
def test_mfma_planes_seeded_shapes(pkg, ctx, bits, group):
    """Ragged row counts (tiles of sixteen rows end inside the matrix), one block (64 bytes of a row) up to rows of
    14336 codes (sixteen wavefronts a tile), every M the kernel takes; the plan record names it."""
    for i, (n, k) in enumerate([(96, 512), (200, 1024), (33, 128), (17, 256), (64, 14336), (4100, 4096), (40, max(group, 512 // bits) * 3)]):
        words, s, z, wq = seeded_case(4100 + i + group + bits, n, k, bits, group)
        w = ctx.weight_prepare_mlx(_fmt(pkg, group, bits), words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
        for m in ((3, 4, 5, 6, 7, 8, 9, 11, 13, 16) if n < 4000 else (3, 4, 8, 16)):
            say(f"mfma planes q{bits} g{group} {k}->{n} M={m}")
            x = act_rounded(kat.seeded_activations(4200 + m, m, k), pkg.BF16, pkg)
            st = w.plan_decode_step(m) if m <= 8 else w.plan_prefill_steps(m)[0]
            # small 4-bit matrices with rows of 2049 to 4096 codes keep three rows (below 12 MB: four) on the dot-product
            # rows kernel
            rows_kernel = bits == 4 and 2048 < k <= 4096 and m in (3, 4) and n * (k // group) * (4 + group // 2) < (24 if m == 3 else 12) << 20
            want_kernel = f"gemv_rows_q{bits}_g{group}" if rows_kernel else f"gemv_mfma_planes_q{bits}_g{group}"
            assert st.device_kernel == want_kernel and not st.used_fallback, st.device_kernel
            y32 = run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.F32, use_qgemm=m > 8)
            assert_within_tolerance(y32, oracle.gemm_f64(wq, x), f"q{bits} g{group} {k}->{n} M={m}")
            ybf = run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.BF16, use_qgemm=m > 8)
            assert np.array_equal(oracle.bf16_from_f32(ybf), oracle.bf16_from_f32(y32))
        for m in (2,):                                          # below the threshold: the dot-product kernels
            assert w.plan_decode_step(m).device_kernel != f"gemv_mfma_planes_q{bits}_g{group}"
        w.destroy()


@pytest.mark.parametrize("bits,group", [(4, 64), (8, 32), (8, 64), (8, 128)])
def test_mfma_planes_exact_small_integers_f16_scales_and_strides(pkg, ctx, bits, group):
    """Exactly representable case: every product and partial sum (those of the offset codes included: 128 + q, and for
    8 bits 128 + l and 16 (128 + h)) is a multiple of 2^-6 that fits 24 bits, so the result is exact whatever the order
    of the sums; planes made from STAF blocks (f16 scale words) and from MLX planes (bf16); padded activation and
    output rows."""
    rng = np.random.default_rng(4300 + bits + group)
    n, k = 100, 1024
    codes = rng.integers(0, 1 << bits, (n, k), dtype=np.uint8)
    scales = rng.choice([0.125, 0.25, 0.5], (n, k // group)); zeros = rng.integers(-4, 5, (n, k // group)) * 0.25
    case = Case(bits, group, codes, scales, zeros)
    wq = scales.repeat(group, axis=1) * codes + zeros.repeat(group, axis=1)
    fmt = _fmt(pkg, group, bits)
    for name, w in (("f16", ctx.weight_prepare_staf(fmt, n, k, case.staf_blocks(), pkg.LAYOUT_PLANES)),
                    ("bf16", ctx.weight_prepare_mlx(fmt, *case.planes(pkg.BF16, pkg), pkg.BF16, pkg.LAYOUT_PLANES))):
        for m, xpad, ypad in ((4, 0, 0), (5, 8, 0), (8, 16, 12), (12, 8, 4), (16, 0, 0)):
            x = np.full((m, k + xpad), 512.0, np.float32)
            x[:, :k] = rng.integers(-8, 9, (m, k)).astype(np.float32) * 0.125
            xd = ctx.upload(oracle.bf16_from_f32(x).reshape(x.shape))
            yd = ctx.alloc(m * (n + ypad) * 4); ctx.fill(yd, 0x7FC00000)
            (ctx.qgemv if m <= 8 else ctx.qgemm)(w, xd, pkg.BF16, yd, pkg.F32, m, k + xpad, (n + ypad) if ypad else 0)
            ctx.synchronize()
            got = yd.download(np.float32, (m, n + ypad))
            assert np.array_equal(got[:, :n].astype(np.float64), x[:, :k].astype(np.float64) @ wq.T), (name, m)
            assert np.all(np.isnan(got[:, n:]))
            xd.free(); yd.free()
        w.destroy()


def test_mfma_planes_batched_projections_one_launch(pkg, ctx):
    """q+k+v and gate+up at 4 <= M <= 8 share one launch on the planes: identical bits to the separate launches."""
    for ns, k, bits, group in [((1024, 256, 256), 1024, 4, 64), ((1400, 1400), 512, 4, 64), ((5, 17, 130), 256, 4, 64),
                               ((1024, 256, 256), 1024, 8, 32), ((300, 700), 448, 8, 64)]:
        ws, wqs = [], []
        for i, n in enumerate(ns):
            words, s, z, wq = seeded_case(4400 + i + n % 13, n, k, bits, group)
            ws.append(ctx.weight_prepare_mlx(_fmt(pkg, group, bits), words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)); wqs.append(wq)
        for m in (4, 7, 8, 10, 16):
            x = act_rounded(kat.seeded_activations(4500 + m, m, k), pkg.BF16, pkg)
            xd = ctx.upload(oracle.bf16_from_f32(x).reshape(x.shape))
            yds = [ctx.alloc(m * n * 4) for n in ns]
            ctx.batched_qgemm(ws, xd, pkg.BF16, yds, pkg.F32, m); ctx.synchronize()
            for j, n in enumerate(ns):
                fused = yds[j].download(np.float32, (m, n))
                alone = run_gemv(ctx, pkg, ws[j], x, pkg.BF16, pkg.F32, use_qgemm=m > 8)
                assert np.array_equal(fused, alone), (ns, m, j)
                assert_within_tolerance(fused, oracle.gemm_f64(wqs[j], x), f"batched {ns} M={m} #{j}")
            xd.free()
            for b in yds:
                b.free()
        for w in ws:
            w.destroy()


def test_mfma_planes_long_rows_in_k_parts_and_linearity(pkg, ctx):
    """Rows of 28672 codes at eight activation rows overflow the staged copy: K is split over workgroup parts and a
    second launch adds the partial results.  At full projection size y(2x) == 2 y(x) bit for bit."""
    n, k, m = 48, 28672, 8
    words, s, z, wq = seeded_case(4600, n, k, 4, 64)
    w = ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
    x = act_rounded(kat.seeded_activations(4601, m, k), pkg.BF16, pkg)
    st = w.plan_decode_step(m)
    assert st.device_kernel == "gemv_mfma_planes_q4_g64" and st.grid[1] > 1
    assert_within_tolerance(run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.F32), oracle.gemm_f64(wq, x), "K parts")
    w.destroy()
    n, k = 14336, 4096
    words, s, z, _ = seeded_case(4602, n, k, 4, 64)
    w = ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
    x = act_rounded(kat.seeded_activations(4603, 6, k), pkg.BF16, pkg)
    y1, y2 = run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.F32), run_gemv(ctx, pkg, w, 2.0 * x, pkg.BF16, pkg.F32)
    assert np.array_equal(2.0 * y1, y2)
    w.destroy()
