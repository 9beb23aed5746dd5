"""GPU parity tests of the wide-tile prefill GEMM (4-bit planes, weights dequantised in registers), through the C ABI.

Numerics are those of the reference's dequant -> bf16 -> GEMM route
(MetalSourceGenerator+Quantized.swift:361-416, MetalSourceGenerator+Linear.swift:18-81): the expected values are an
fp64 accumulation of the bf16-rounded dequantised weights from the CPU oracle.  Bars as for the tiled kernel:
relative L2 <= 1e-3 and max-abs <= 2e-2 on the fp32 output, 16-bit outputs equal to the rounding of the fp32 output,
exactly representable cases compared exactly.  The kernel is forced with the probe flag where the shape is smaller
than what the dispatcher gives it; benchmark config 3 runs as dispatched.
"""
import itertools
import sys

import numpy as np
import pytest

import kat
import oracle
from gpu_util import Case, act_rounded, assert_within_tolerance, seeded_case
from test_gpu_gemm import _tile_edge_sample, bf16_round, run_qgemm

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, file=sys.stderr, flush=True)


def wide(pkg):
    return pkg.FLAG_FORCE_MFMA | pkg.FLAG_PROBE_WIDE


@pytest.mark.parametrize("group", [64, 128])
def test_wide_gemm_exact_small_integers(pkg, ctx, group):
    """Every product and partial sum an integer multiple of 2^-6 below 2^17: any summation order is exact.  Rows
    and columns off the tile grid (300 rows: a 256-row tile and a cut one; 530 columns: two whole column tiles and
    one that ends inside a group of four), both scale types, all three output types, wide and narrow stores."""
    rng = np.random.default_rng(4000 + group)
    m, n, k = 300, 530, 3 * 256
    codes = rng.integers(0, 16, (n, k), dtype=np.uint8)
    scales = rng.choice([0.125, 0.25, 0.5], (n, k // group))
    zeros = rng.integers(-4, 5, (n, k // group)) * 0.25
    case = Case(4, group, codes, scales, zeros)
    wq = scales.repeat(group, axis=1) * codes + zeros.repeat(group, axis=1)
    assert np.array_equal(bf16_round(wq), wq.astype(np.float32))
    x = rng.integers(-8, 9, (m, k)).astype(np.float32) * 0.125
    want = x.astype(np.float64) @ wq.T
    for sb in (pkg.F16, pkg.BF16):
        w = case.device_weight(ctx, pkg, pkg.LAYOUT_PLANES, sb)
        step = w.plan_prefill_steps(m, flags=wide(pkg))[0]
        assert step.device_kernel == f"qgemm_wide_q4_g{group}" and step.block[0] == 256, step.device_kernel
        for yd in (pkg.F32, pkg.BF16, pkg.F16):
            for y_pad in (0, 2, 3):               # 532 columns a row: 16-byte rows; 533: the narrow stores
                say(f"wide exact g{group} sb={sb} y={yd} pad={y_pad}")
                got = run_qgemm(ctx, pkg, w, x, yd, wide(pkg), y_stride=(n + y_pad) if y_pad else None)
                if y_pad:
                    assert np.all(np.isnan(got[:, n:])), "padding of the output rows was written"
                    got = got[:, :n]
                if yd == pkg.F32:
                    assert np.array_equal(got.astype(np.float64), want)
                elif yd == pkg.BF16:
                    assert np.array_equal(got, bf16_round(want.astype(np.float32)))
                else:
                    assert np.array_equal(got, want.astype(np.float16).astype(np.float32))
        w.destroy()


def _seeded(pkg, ctx, seed, m, n, k, group, flags, sample=None, x_pad=0, y_pad=0, layout=None, x_dtype=None):
    """Seeded weights and activations through the kernel: fp32 result against the fp64 product of the weights rounded
    to the activation type (bf16 or f16), and the 16-bit result against the rounding of the fp32 one."""
    layout = pkg.LAYOUT_PLANES if layout is None else layout
    x_dtype = pkg.BF16 if x_dtype is None else x_dtype
    words, s, z, wq = seeded_case(seed, n, k, 4, group)
    # fp32 activations meet bf16 weights, as in the reference's gemm_bf16_f32s
    wb = wq.astype(np.float16).astype(np.float32) if x_dtype == pkg.F16 else bf16_round(wq)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, group)
    w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, layout)
    x = np.zeros((m, k + x_pad), np.float32)
    x[:, :k] = act_rounded(kat.seeded_activations(seed + 1, m, k), x_dtype, pkg)
    if x_pad:
        x[:, k:] = 3.0e4
    say(f"wide seeded g{group} M={m} {k}->{n} pads=({x_pad},{y_pad}) flags={flags} layout={layout} x={x_dtype}")
    got = run_qgemm(ctx, pkg, w, x, pkg.F32, flags, y_stride=(n + y_pad) if y_pad else None, x_dtype=x_dtype)
    if y_pad:
        assert np.all(np.isnan(got[:, n:])), "padding of the output rows was written"
        got = got[:, :n]
    cols = np.arange(n) if sample is None else sample
    want = oracle.gemm_f64(np.ascontiguousarray(wb[cols]), np.ascontiguousarray(x[:, :k]))
    r = assert_within_tolerance(got[:, cols], want, f"wide g{group} M={m} {k}->{n}")
    assert np.all(np.isfinite(got))
    gb = run_qgemm(ctx, pkg, w, x, pkg.BF16, flags, x_dtype=x_dtype)
    assert np.array_equal(oracle.bf16_from_f32(gb), oracle.bf16_from_f32(got)), "bf16 out != rne(fp32 out)"
    return w, x, got, r


def test_wide_gemm_ragged_shapes_against_the_oracle(pkg, ctx):
    """One row, rows just past a tile, one column, columns off every grid, one group of four K-tiles and several, padded
    rows on both sides; and the same weights through the tiled kernel: equal up to the order of the fp32 sums."""
    for i, (m, n, k, group, x_pad, y_pad) in enumerate([(1, 1, 256, 64, 0, 0), (129, 257, 512, 64, 0, 0),
                                                         (257, 70, 256, 128, 0, 0), (130, 515, 1024, 64, 64, 5),
                                                         (600, 300, 768, 128, 8, 4), (33, 1030, 256, 64, 0, 1)]):
        w, x, got, _ = _seeded(pkg, ctx, 4100 + i, m, n, k, group, wide(pkg), x_pad=x_pad, y_pad=y_pad)
        tiled = run_qgemm(ctx, pkg, w, x, pkg.F32, pkg.FLAG_FORCE_MFMA | pkg.FLAG_PROBE_TILED)
        assert np.max(np.abs(tiled - got)) <= 2e-5 * max(1.0, float(np.max(np.abs(got)))), "wide vs tiled kernel"
        w.destroy()


@pytest.mark.parametrize("group", [64, 128])
@pytest.mark.parametrize("blocks,f16", [(True, False), (False, True), (True, True)])
def test_wide_gemm_blocks_in_place_and_f16_activations_exact(pkg, ctx, group, blocks, f16):
    """The reference's interleaved blocks read in place (a lane's code bytes at 4-byte aligned addresses, scale and zero
    from the block headers) and f16 activations (weights rounded to f16, f16 matrix instruction): small integers, so
    every result is exact whatever the order of the sums; all three output types."""
    rng = np.random.default_rng(4500 + group + 7 * blocks + 13 * f16)
    m, n, k = 290, 300, 2 * 256
    codes = rng.integers(0, 16, (n, k), dtype=np.uint8)
    scales = rng.choice([0.125, 0.25, 0.5], (n, k // group))
    zeros = rng.integers(-4, 5, (n, k // group)) * 0.25
    case = Case(4, group, codes, scales, zeros)
    wq = scales.repeat(group, axis=1) * codes + zeros.repeat(group, axis=1)
    x = rng.integers(-8, 9, (m, k)).astype(np.float32) * 0.125
    want = x.astype(np.float64) @ wq.T
    x_dtype = pkg.F16 if f16 else pkg.BF16
    w = case.device_weight(ctx, pkg, pkg.LAYOUT_STAF_BLOCKS if blocks else pkg.LAYOUT_PLANES, pkg.BF16)
    step = w.plan_prefill_steps(m, x_dtype=x_dtype, flags=wide(pkg))[0]
    assert step.device_kernel == f"qgemm_wide_q4_g{group}" and step.kernel_family == "mfmaGEMM", step.device_kernel
    for yd in (pkg.F32, pkg.BF16, pkg.F16):
        say(f"wide exact g{group} blocks={blocks} f16={f16} y={yd}")
        got = run_qgemm(ctx, pkg, w, x, yd, wide(pkg), x_dtype=x_dtype)
        if yd == pkg.F32:
            assert np.array_equal(got.astype(np.float64), want)
        elif yd == pkg.BF16:
            assert np.array_equal(got, bf16_round(want.astype(np.float32)))
        else:
            assert np.array_equal(got, want.astype(np.float16).astype(np.float32))
    w.destroy()


def test_wide_gemm_blocks_and_f16_seeded_against_the_oracle(pkg, ctx):
    """Seeded weights: blocks in place give the bits of the planes kernel (same codes, same f16 scales); f16
    activations hold the bar against the fp64 product of f16-rounded weights."""
    for i, (m, n, k, group) in enumerate([(257, 300, 512, 64), (130, 515, 768, 128)]):
        wp, x, got_p, _ = _seeded(pkg, ctx, 4600 + i, m, n, k, group, wide(pkg))
        wb, _, got_b, _ = _seeded(pkg, ctx, 4600 + i, m, n, k, group, wide(pkg), layout=pkg.LAYOUT_STAF_BLOCKS)
        assert np.array_equal(got_p, got_b), "blocks in place and planes differ"
        wp.destroy(); wb.destroy()
        for layout in (pkg.LAYOUT_PLANES, pkg.LAYOUT_STAF_BLOCKS):
            w, _, _, _ = _seeded(pkg, ctx, 4610 + i, m, n, k, group, wide(pkg), layout=layout, x_dtype=pkg.F16)
            w.destroy()


def test_wide_gemm_fp32_activations(pkg, ctx):
    """fp32 activations (the reference's prefill type, gemm_q4_g*_f32s): every row is split into [hi | lo] bf16 halves
    that carry sixteen bits of it, and the kernel walks 2 K against the weights twice; planes and blocks in place, K in
    parts, against the fp64 product of bf16 weights and the fp32 activations."""
    for i, (m, n, k, group, layout) in enumerate([(257, 300, 512, 64, pkg.LAYOUT_PLANES), (130, 515, 768, 128, pkg.LAYOUT_STAF_BLOCKS),
                                                   (300, 264, 2304, 64, pkg.LAYOUT_PLANES)]):
        w, x, got, _ = _seeded(pkg, ctx, 4800 + i, m, n, k, group, wide(pkg), layout=layout, x_dtype=pkg.F32)
        step = w.plan_prefill_steps(m, x_dtype=pkg.F32, flags=wide(pkg))[0]
        assert step.device_kernel == f"split_f32_bf16x2+qgemm_wide_q4_g{group}" and step.kernel_family == "mfmaGEMM"
        if i == 2:
            pkg.Context.probe_wide_shape(256, 3)
            try:
                parts = run_qgemm(ctx, pkg, w, x, pkg.F32, wide(pkg), x_dtype=pkg.F32)
            finally:
                pkg.Context.probe_wide_shape(0, 0)
            assert np.max(np.abs(parts - got)) <= 2e-5 * max(1.0, float(np.max(np.abs(got))))
        w.destroy()


@pytest.mark.parametrize("layout_name,x_name", [("LAYOUT_STAF_BLOCKS", "BF16"), ("LAYOUT_PLANES", "F16"), ("LAYOUT_STAF_BLOCKS", "F16"),
                                                ("LAYOUT_PLANES", "F32")])
@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336)])
def test_config3_on_blocks_and_f16_as_dispatched(pkg, ctx, layout_name, x_name, n, k):
    """benchmark config 3 at M = 2048 on the reference's block layout and with its f16 and fp32 activations, no flags:
    the plan names this library's matrix-core kernel, and the result holds the bar on the tile-edge column sample."""
    m = 2048
    layout, x_dtype = getattr(pkg, layout_name), getattr(pkg, x_name)
    sample = _tile_edge_sample(n, 31 * m + n, tile=256)
    w, _, _, (rel, _) = _seeded(pkg, ctx, 4700, m, n, k, 64, 0, sample=sample, layout=layout, x_dtype=x_dtype)
    steps = w.plan_prefill_steps(m, x_dtype=x_dtype)
    say("as dispatched:", [s.device_kernel for s in steps])
    assert len(steps) == 1 and steps[0].device_kernel.endswith("qgemm_wide_q4_g64") and steps[0].kernel_family == "mfmaGEMM"
    assert steps[0].device_kernel.startswith("split_f32_bf16x2+") == (x_dtype == pkg.F32)
    assert not steps[0].used_fallback
    assert rel < 5e-4
    w.destroy()


@pytest.mark.parametrize("tile_rows,parts", [(256, 2), (256, 4), (128, 3), (128, 4)])
def test_wide_gemm_with_k_in_parts(pkg, ctx, tile_rows, parts):
    """K split over workgroups (fp32 partial results, summed in part order by a second launch): exact on small integers
    for every output type and a padded result; seeded values against the oracle; the forced shape shows in the plan."""
    rng = np.random.default_rng(4400 + parts)
    m, n, k = 300, 264, 64 * 16 * parts + 256           # the last part is shorter than the others
    codes = rng.integers(0, 16, (n, k), dtype=np.uint8)
    scales = rng.choice([0.125, 0.25, 0.5], (n, k // 64))
    zeros = rng.integers(-4, 5, (n, k // 64)) * 0.25
    case = Case(4, 64, codes, scales, zeros)
    wq = scales.repeat(64, axis=1) * codes + zeros.repeat(64, axis=1)
    x = rng.integers(-8, 9, (m, k)).astype(np.float32) * 0.125
    want = x.astype(np.float64) @ wq.T
    pkg.Context.probe_wide_shape(tile_rows, parts)
    try:
        w = case.device_weight(ctx, pkg, pkg.LAYOUT_PLANES, pkg.BF16)
        step = w.plan_prefill_steps(m, flags=wide(pkg))[0]
        tiles = -(-m // tile_rows) * -(-n // 256)
        assert step.device_kernel == "qgemm_wide_q4_g64" and step.grid[0] == -(-tiles * parts // 8) * 8, (step.grid, tiles)
        for yd in (pkg.F32, pkg.BF16, pkg.F16):
            for y_pad in (0, 3):
                say(f"wide K parts {tile_rows}x{parts} y={yd} pad={y_pad}")
                got = run_qgemm(ctx, pkg, w, x, yd, wide(pkg), y_stride=(n + y_pad) if y_pad else None)
                if y_pad:
                    assert np.all(np.isnan(got[:, n:])), "padding of the output rows was written"
                    got = got[:, :n]
                if yd == pkg.F32:
                    assert np.array_equal(got.astype(np.float64), want)
                elif yd == pkg.BF16:
                    assert np.array_equal(got, bf16_round(want.astype(np.float32)))
                else:
                    assert np.array_equal(got, want.astype(np.float16).astype(np.float32))
        w.destroy()
        w, x, got, _ = _seeded(pkg, ctx, 4410 + parts, 257, 520, k, 64, wide(pkg))
        pkg.Context.probe_wide_shape(0, 0)
        whole = run_qgemm(ctx, pkg, w, x, pkg.F32, pkg.FLAG_FORCE_MFMA | pkg.FLAG_PROBE_TILED)
        assert np.max(np.abs(whole - got)) <= 2e-5 * max(1.0, float(np.max(np.abs(got))))
        w.destroy()
    finally:
        pkg.Context.probe_wide_shape(0, 0)


@pytest.mark.parametrize("m", [128, 512, 2048])
@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336)])
def test_config3_prefill_as_dispatched(pkg, ctx, m, n, k):
    """benchmark config 3 at full size with no flags: whatever route the library picks for the shape (the plan record
    names it) is checked against the oracle on every row and the tile-edge column sample."""
    sample = _tile_edge_sample(n, 17 * m + n, tile=256)
    w, _, _, (rel, _) = _seeded(pkg, ctx, 4200 + m % 83, m, n, k, 64, 0, sample=sample)
    steps = w.plan_prefill_steps(m)
    say("as dispatched:", [s.device_kernel for s in steps])
    if m == 2048:
        # long prompts stay on this library's own kernel
        assert len(steps) == 1 and steps[0].device_kernel == "qgemm_wide_q4_g64" and not steps[0].used_fallback
    assert rel < 5e-4
    w.destroy()


def test_context_without_the_dense_library_keeps_in_tree_kernels(pkg):
    """mi355q_context_set_library_use(ctx, 0): a long prompt on blocks in place, which the two-dispatch route would
    serve, stays on this library's kernels, and the result holds the bar."""
    c = pkg.Context(0)
    try:
        c.set_library_use(False)
        m, n, k = 130, 96, 512
        words, s, z = oracle.quantize_affine(kat.seeded_weights(4300, n, k), 4, 64, oracle.F16)
        wq = oracle.dequant_planes_f32(4, 64, n, k, words, s, z, oracle.F16)
        fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
        w = c.weight_prepare_mlx(fmt, words, s, z, pkg.F16, pkg.LAYOUT_STAF_BLOCKS)
        x = act_rounded(kat.seeded_activations(4301, m, k), pkg.BF16, pkg)
        assert all(s.kernel_family != "libraryGEMM" for s in w.plan_prefill_steps(m)), "the plan names the library"
        got = run_qgemm(c, pkg, w, x, pkg.F32, 0)
        assert_within_tolerance(got, oracle.gemm_f64(wq, x), "blocks in place, library forbidden")
        w.destroy()
    finally:
        c.close()


@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336)])
def test_config3_full_size_properties_every_output(pkg, ctx, n, k):
    """benchmark config 3 at M = 2048, as dispatched, every one of the M x N outputs through properties that need no
    oracle pass over the matrix: y(2x) == 2 y(x) bit for bit (doubling is exact in bf16 and in every fp32 sum), rows of
    x that are equal give rows of y that are equal, a zero row gives the zero row, and the fp32 and bf16 results agree
    to one rounding."""
    m = 2048
    words, s, z, _ = seeded_case(4700 + n % 7, n, k, 4, 64)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
    assert w.plan_prefill_steps(m)[0].device_kernel == "qgemm_wide_q4_g64"
    x = act_rounded(kat.seeded_activations(4710, m, k), pkg.BF16, pkg)
    x[5] = x[1900]                     # equal rows in different row tiles
    x[300] = 0.0
    y1 = run_qgemm(ctx, pkg, w, x, pkg.F32, 0)
    y2 = run_qgemm(ctx, pkg, w, 2.0 * x, pkg.F32, 0)
    assert np.all(np.isfinite(y1))
    assert np.array_equal(2.0 * y1, y2)
    assert np.array_equal(y1[5], y1[1900]) and not np.any(y1[300])
    yb = run_qgemm(ctx, pkg, w, x, pkg.BF16, 0)
    assert np.array_equal(oracle.bf16_from_f32(yb), oracle.bf16_from_f32(y1))
    w.destroy()


@pytest.mark.parametrize("layout_name,x_name", [("LAYOUT_PLANES", "BF16"), ("LAYOUT_STAF_BLOCKS", "BF16"), ("LAYOUT_PLANES", "F16"),
                                                ("LAYOUT_PLANES", "F32")])
def test_shared_launch_of_the_wide_kernel_equals_one_matrix_of_all_rows(pkg, ctx, layout_name, x_name):
    """Two or three projections that share their activations (q+k+v, gate+up) as one launch of the wide-tile kernel: every
    column tile belongs to one matrix.  Bit for bit the result of one matrix made of the rows of all of them (same
    tiles, same K parts, same sums), for 128- and 256-row tiles, K in one part and in several, a ragged last matrix,
    every output type, results whose rows are and are not 16-byte multiples, fp32 activations (split once into bf16
    halves for all the matrices); the plan record names the launch."""
    layout, xd = getattr(pkg, layout_name), getattr(pkg, x_name)
    sbo, sbp = (oracle.F16, pkg.F16) if layout == pkg.LAYOUT_STAF_BLOCKS else (oracle.BF16, pkg.BF16)
    cases = [(100, (512, 256, 200), 1024, 64), (300, (768, 260), 512, 128), (700, (256, 256, 256), 2048, 64)]
    for i, (m, ns, k, group) in enumerate(cases):
        fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, group)
        parts = [oracle.quantize_affine(kat.seeded_weights(7300 + 10 * i + j, n, k), 4, group, sbo) for j, n in enumerate(ns)]
        ws = [ctx.weight_prepare_mlx(fmt, w_, s_, z_, sbp, layout) for (w_, s_, z_) in parts]
        whole = ctx.weight_prepare_mlx(fmt, np.concatenate([p[0] for p in parts]), np.concatenate([p[1].reshape(n, -1) for p, n in zip(parts, ns)]),
                                       np.concatenate([p[2].reshape(n, -1) for p, n in zip(parts, ns)]), sbp, layout)
        x = act_rounded(kat.seeded_activations(7350 + i, m, k), xd, pkg)
        xdev = ctx.upload(x.astype(np.float16).view(np.uint16) if xd == pkg.F16 else x.astype(np.float32) if xd == pkg.F32
                          else oracle.bf16_from_f32(x))
        total = sum(ns)
        shapes = [(0, 0)] + ([(128, 2), (256, 2)] if k >= 2048 else [])       # as chosen; K forced into two parts
        for yd, (tile_rows, k_parts) in itertools.product((pkg.BF16, pkg.F32, pkg.F16), shapes):
            esz = 4 if yd == pkg.F32 else 2
            dt = np.float32 if esz == 4 else np.uint16
            say(f"shared wide launch {layout_name} x={x_name} m={m} ns={ns} k={k} g{group} y={yd} tile {tile_rows} parts {k_parts}")
            outs = [ctx.alloc(m * n * esz) for n in ns]
            ref = ctx.alloc(m * total * esz)
            pkg.Context.probe_wide_shape(tile_rows, k_parts)
            try:
                ctx.batched_qgemm(ws, xdev, xd, outs, yd, m, flags=pkg.FLAG_PROBE_WIDE)
                ctx.qgemm(whole, xdev, xd, ref, yd, m, flags=pkg.FLAG_FORCE_MFMA | pkg.FLAG_PROBE_WIDE)
            finally:
                pkg.Context.probe_wide_shape(0, 0)
            ctx.synchronize()
            want = ref.download(dt, (m, total))
            col = 0
            for o, n in zip(outs, ns):
                assert np.array_equal(o.download(dt, (m, n)), want[:, col:col + n]), (m, ns, k, yd, col)
                col += n
            for t in outs + [ref]:
                t.free()
        launcher, plan = pkg.probe_shared_route(fmt, layout, ns, k, xd, m, flags=pkg.FLAG_PROBE_WIDE, sb_dtype=sbp)
        assert launcher == "shared/wide" and plan == ("split_f32_bf16x2+" if xd == pkg.F32 else "") + f"qgemm_wide_q4_g{group}", (launcher, plan)
        xdev.free(); whole.destroy()
        for w in ws:
            w.destroy()
