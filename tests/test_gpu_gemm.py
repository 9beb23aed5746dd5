"""GPU parity tests of the prefill (sequence) GEMM on the matrix cores, through the C ABI.

The matrix-core kernel follows the numerics of the reference's dequant -> bf16 -> GEMM route
(MetalSourceGenerator+Quantized.swift:361-416 then MetalSourceGenerator+Linear.swift:18-81):
every weight is dequantised in fp32 (scale*q + zero), rounded once to bf16, multiplied with
bf16 activations and accumulated in fp32.  The expected values are therefore an fp64
accumulation of the bf16-rounded dequantised weights from the CPU oracle.

Bars: relative L2 <= 1e-3 and max-abs <= 2e-2 on the fp32 output; bf16 / f16 outputs equal the
rounding of the fp32 output bit for bit; exactly representable cases are compared exactly.
"""
import sys

import numpy as np
import pytest

import kat
import oracle
from gpu_util import act_to_device_array, Case, act_rounded, assert_within_tolerance, out_from_device, seeded_case

pytestmark = pytest.mark.gpu
KATS = kat.load_kats()

MFMA_FORMATS = [(4, 64), (4, 128), (8, 32), (8, 64), (6, 64), (3, 64), (2, 64)]


def say(*a):
    print(*a, file=sys.stderr, flush=True)


def bf16_round(a):
    a = np.asarray(a, np.float32)
    return oracle.bf16_to_f32(oracle.bf16_from_f32(a)).reshape(a.shape)


def run_qgemm(ctx, pkg, w, x_f32, y_dtype, flags, x_stride=None, y_stride=None, x_dtype=None):
    """x_f32 [M, x_stride] (representable in the activation type, bf16 unless given) -> device result [M, y_stride] as float32."""
    m, xs = x_f32.shape
    n = int(w.info.n_rows)
    ys = n if y_stride is None else y_stride
    x_dtype = pkg.BF16 if x_dtype is None else x_dtype
    xd = ctx.upload(act_to_device_array(x_f32, x_dtype, pkg))
    yd = ctx.alloc(m * ys * (4 if y_dtype == pkg.F32 else 2))
    ctx.fill(yd, 0x7FC07FC0 if y_dtype != pkg.F32 else 0x7FC00000)      # NaN canary
    ctx.qgemm(w, xd, x_dtype, yd, y_dtype, m, xs if x_stride is None else x_stride, ys if y_stride else 0, flags)
    ctx.synchronize()
    y = out_from_device(yd, y_dtype, (m, ys), pkg)
    xd.free(); yd.free()
    return y


# ------------------------------------------------------------------ exactly representable cases
@pytest.mark.parametrize("bits,group", MFMA_FORMATS)
def test_mfma_gemm_exact_small_integers(pkg, ctx, bits, group):
    """Codes, scales, zeros and activations chosen so that every product and every partial sum is
    an integer multiple of 2^-6 below 2^17: fp32 accumulation in any order is exact, and so is the
    bf16 rounding of the dequantised weights (|w| needs at most 8 significant bits)."""
    rng = np.random.default_rng(bits * 100 + group)
    m, n, k = 77, 150, 3 * 128
    qmax = (1 << bits) - 1
    codes = rng.integers(0, qmax + 1, (n, k), dtype=np.uint8)
    scales = rng.choice([0.125, 0.25, 0.5], (n, k // group))
    zeros = rng.integers(-4, 5, (n, k // group)) * 0.25
    if bits == 8:            # keep scale*q + zero within 8 significant bits
        scales = np.full((n, k // group), 0.25)
        zeros = np.zeros((n, k // group))
    case = Case(bits, group, codes, scales, zeros)
    wq = scales.repeat(group, axis=1) * codes + zeros.repeat(group, axis=1)
    assert np.array_equal(bf16_round(wq), wq.astype(np.float32))
    x = rng.integers(-8, 9, (m, k)).astype(np.float32) * 0.125
    want = x.astype(np.float64) @ wq.T
    for sb in (pkg.F16, pkg.BF16):
        w = case.device_weight(ctx, pkg, pkg.LAYOUT_PLANES, sb)
        for yd in (pkg.F32, pkg.BF16, pkg.F16):
            say(f"exact q{bits}g{group} sb={sb} y={yd}")
            got = run_qgemm(ctx, pkg, w, x, yd, pkg.FLAG_FORCE_MFMA)
            if yd == pkg.F32:
                assert np.array_equal(got.astype(np.float64), want)
            elif yd == pkg.BF16:
                assert np.array_equal(got, bf16_round(want.astype(np.float32)))
            else:
                assert np.array_equal(got, want.astype(np.float16).astype(np.float32))
        w.destroy()


def test_q3_dequant_then_gemm_reference_vector(pkg, ctx):
    """The reference's q3 g64 prefill check (dequant to bf16, then bf16 GEMM, bar < 0.02), on both
    routes this library offers: two dispatches through a bf16 scratch, and the fused kernel."""
    v = KATS["q3_dequant_then_gemm"]
    k, n, m, group = v["k"], v["n"], v["m"], v["group"]
    nb = k // group
    codes = np.array([[(e + 3 * b + 5 * r) % 8 for b in range(nb) for e in range(group)] for r in range(n)], np.uint8)
    s = np.array([[0.03125 * (b + 1) + 0.0078125 * r for b in range(nb)] for r in range(n)])
    z = np.array([[-0.125 + 0.0625 * r - 0.015625 * b for b in range(nb)] for r in range(n)])
    x = np.array([((i % 17) - 8) * 0.0625 for i in range(m * k)], np.float32).reshape(m, k)
    want = kat.exact_gemv(codes, s, z, x, group)
    case = Case(3, group, codes, s, z)
    wb = oracle.bf16_to_f32(oracle.dequant_staf_bf16(3, group, n, k, case.staf_blocks())).reshape(n, k)
    want_bf = oracle.gemm_f64(wb, x)
    for layout in (pkg.LAYOUT_STAF_BLOCKS, pkg.LAYOUT_PLANES):
        w = case.device_weight(ctx, pkg, layout, pkg.F16)
        scratch = ctx.alloc(n * k * 2)
        ctx.dequant_bf16(w, scratch)
        xd = ctx.upload(oracle.bf16_from_f32(x).reshape(m, k))
        yd = ctx.alloc(m * n * 4)
        say(f"q3 reference vector, two dispatches, layout {layout}")
        ctx.gemm_bf16(xd, pkg.BF16, scratch, yd, pkg.F32, m, n, k)
        ctx.synchronize()
        got = yd.download(np.float32, (m, n))
        assert np.max(np.abs(got - want)) < 0.02                       # the reference's own bar
        assert np.max(np.abs(got - want_bf)) < 1e-5
        if layout == pkg.LAYOUT_PLANES:
            say("q3 reference vector, fused")
            fused = run_qgemm(ctx, pkg, w, x, pkg.F32, pkg.FLAG_FORCE_MFMA)
            assert np.array_equal(fused, got)
        for b in (scratch, xd, yd):
            b.free()
        w.destroy()


def test_q4_gemm_padded_stride_on_matrix_cores(pkg, ctx):
    """The reference's padded-inputRowStride GEMM vector (poisoned padding must not be read)."""
    v = KATS["q4_gemm_padded_stride"]
    k, n, m, stride = v["k"], v["n"], v["m"], v["stride"]
    x = np.full((m, stride), v["poison"], np.float32)
    for mi in range(m):
        for c in range(k):
            x[mi, c] = (mi + 3) * ((c % 7) - 3) * 0.125
    case = Case(4, 64, [[r + 1] * k for r in range(n)], np.full((n, 1), v["scale"]), np.full((n, 1), v["zero"]))
    want = np.array([[0.25 * (r + 1) * x[mi, :k].astype(np.float64).sum() for r in range(n)] for mi in range(m)])
    w = case.device_weight(ctx, pkg, pkg.LAYOUT_PLANES, pkg.F16)
    say("padded stride vector")
    got = run_qgemm(ctx, pkg, w, x, pkg.F32, pkg.FLAG_FORCE_MFMA)
    assert np.max(np.abs(got - want)) < 1e-3
    w.destroy()


# ------------------------------------------------------------------ seeded, against the oracle
def _seeded_gemm(pkg, ctx, seed, m, n, k, bits, group, sample=None, x_pad=0, y_pad=0, flags=None):
    words, s, z, wq = seeded_case(seed, n, k, bits, group)
    wb = bf16_round(wq)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
    w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
    x = np.zeros((m, k + x_pad), np.float32)
    x[:, :k] = act_rounded(kat.seeded_activations(seed + 1, m, k), pkg.BF16, pkg)
    if x_pad:
        x[:, k:] = 3.0e4
    fl = pkg.FLAG_FORCE_MFMA if flags is None else flags
    say(f"seeded q{bits}g{group} M={m} {k}->{n} pads=({x_pad},{y_pad})")
    got = run_qgemm(ctx, pkg, w, x, pkg.F32, fl, y_stride=(n + y_pad) if y_pad else None)
    if y_pad:
        assert np.all(np.isnan(got[:, n:])), "padding of the output rows was written"
        got = got[:, :n]
    cols = np.arange(n) if sample is None else sample
    want = oracle.gemm_f64(np.ascontiguousarray(wb[cols]), np.ascontiguousarray(x[:, :k]))
    r = assert_within_tolerance(got[:, cols], want, f"q{bits}g{group} M={m} {k}->{n}")
    assert np.all(np.isfinite(got))
    gb = run_qgemm(ctx, pkg, w, x, pkg.BF16, fl)
    assert np.array_equal(oracle.bf16_from_f32(gb), oracle.bf16_from_f32(got)), "bf16 out != rne(fp32 out)"
    w.destroy()
    return got, r


def _tile_edge_sample(n, seed, per_tile=2, tile=128):
    rng = np.random.default_rng(seed)
    cols = {0, n - 1}
    for t0 in range(0, n, tile):
        hi = min(t0 + tile, n)
        cols.update([t0, hi - 1])
        cols.update(int(c) for c in rng.integers(t0, hi, per_tile))
    return np.array(sorted(cols))


@pytest.mark.parametrize("m", [128, 512, 2048])
@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336)])
def test_config3_prefill_gate_up_and_down(pkg, ctx, m, n, k):
    """benchmark config 3 at full size.  Every one of the M output rows is checked, on a sample of
    output columns that holds the first and last column of every 128-wide column tile plus two
    random ones (the CPU oracle on all 14336 columns would take minutes)."""
    sample = _tile_edge_sample(n, 31 * m + n)
    _, (rel, _) = _seeded_gemm(pkg, ctx, 700 + m % 89, m, n, k, 4, 64, sample=sample)
    assert rel < 5e-4


def test_mfma_gemm_wide_tiles_with_k_split_ragged(pkg, ctx):
    """Shapes whose 256 x 256 tiles alone leave CUs idle run with K split over workgroups (fp32 partials, then a sum
    launch): M and N off the tile grid, padded output rows, 4- and 8-bit codes."""
    for i, (m, n, k, bits, group, y_pad) in enumerate([(333, 14330, 4096, 4, 64, 0), (300, 7001, 4096, 8, 32, 3),
                                                       (1000, 4100, 4096, 4, 64, 0)]):
        sample = _tile_edge_sample(n, 990 + i, per_tile=1, tile=256)
        _seeded_gemm(pkg, ctx, 970 + i, m, n, k, bits, group, sample=sample, y_pad=y_pad)


def test_mfma_gemm_many_tiles_ragged_last_column_tile(pkg, ctx):
    """2048 x 14286: more 256 x 256 tiles than CUs (two rounds), the last column tile cut at column 14286,
    padded output rows."""
    m, n, k = 2048, 14286, 128
    sample = _tile_edge_sample(n, 77)
    _seeded_gemm(pkg, ctx, 960, m, n, k, 4, 64, sample=sample)
    _seeded_gemm(pkg, ctx, 961, m, n, k, 8, 32, sample=sample, y_pad=2)


@pytest.mark.parametrize("bits,group", [f for f in MFMA_FORMATS if f != (4, 64)])
def test_mfma_gemm_other_formats_seeded(pkg, ctx, bits, group):
    _seeded_gemm(pkg, ctx, 800 + bits + group, 200, 384, 1024, bits, group)


def test_mfma_gemm_ragged_shapes(pkg, ctx):
    """M and N off the tile grid (including a single row / a single column), one K-tile, padded strides."""
    for i, (m, n, k) in enumerate([(9, 1, 64), (1, 130, 128), (129, 257, 192), (300, 100, 64), (257, 513, 320),
                                   (31, 4099, 256)]):
        _seeded_gemm(pkg, ctx, 900 + i, m, n, k, 4, 64)
    _seeded_gemm(pkg, ctx, 910, 70, 200, 256, 4, 64, x_pad=64, y_pad=8)
    _seeded_gemm(pkg, ctx, 911, 270, 300, 512, 8, 32, x_pad=8, y_pad=1)


def test_qgemm_selects_matrix_cores_above_eight_rows(pkg, ctx):
    """Without flags, M > 8 goes to the matrix-core kernel when the weight is eligible and to the
    per-row kernel otherwise; both agree within the tolerance, and the plan record names the choice."""
    m, n, k = 200, 256, 512
    got_auto, _ = _seeded_gemm(pkg, ctx, 920, m, n, k, 4, 64, flags=0)
    got_mfma, _ = _seeded_gemm(pkg, ctx, 920, m, n, k, 4, 64)
    assert np.array_equal(got_auto, got_mfma)
    words, s, z, wq = seeded_case(920, n, k, 4, 64)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
    step = w.plan_prefill_steps(m)[0]
    assert step.kernel_family == "mfmaGEMM" and not step.used_fallback and step.device_kernel == "qgemm_mfma_q4_g64"
    assert step.block[0] in (256, 512) and step.grid[0] >= 1
    m = 64
    ws = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_STAF_BLOCKS)
    step = ws.plan_prefill_steps(m, flags=pkg.FLAG_FORCE_SMALL_M)[0]       # unforced, the two-dispatch route serves it
    assert step.kernel_family != "mfmaGEMM"
    step = ws.plan_prefill_steps(12)[0]                  # nine to 96 rows: the streamed-weight kernel reads the blocks
    assert step.device_kernel == "qgemm_stream_q4_g64" and not step.used_fallback
    step = ws.plan_prefill_steps(2)[0]
    assert step.kernel_family != "mfmaGEMM"
    with pytest.raises(pkg.MI355QError):
        x = act_rounded(kat.seeded_activations(1, m, k), pkg.BF16, pkg)
        run_qgemm(ctx, pkg, ws, x, pkg.F32, pkg.FLAG_FORCE_MFMA)
    # the per-row kernel keeps fp32 weights: close to, but not the same numbers as, the bf16 route
    x = act_rounded(kat.seeded_activations(921, m, k), pkg.BF16, pkg)
    slow = run_qgemm(ctx, pkg, ws, x, pkg.F32, pkg.FLAG_FORCE_SMALL_M)
    assert_within_tolerance(slow, oracle.gemm_f64(wq, x), "per-row kernel")
    w.destroy(); ws.destroy()


def test_dense_bf16_gemm(pkg, ctx):
    """mi355q_gemm_bf16 (the second dispatch of the two-step prefill route) against fp64."""
    rng = np.random.default_rng(77)
    for m, n, k in [(1, 1, 64), (130, 70, 128), (256, 512, 1024), (1000, 300, 192)]:
        a = bf16_round(rng.standard_normal((m, k)).astype(np.float32))
        b = bf16_round((rng.standard_normal((n, k)) * 0.05).astype(np.float32))
        ad, bd = ctx.upload(oracle.bf16_from_f32(a).reshape(m, k)), ctx.upload(oracle.bf16_from_f32(b).reshape(n, k))
        cd = ctx.alloc(m * n * 4)
        say(f"dense {m}x{n}x{k}")
        ctx.gemm_bf16(ad, pkg.BF16, bd, cd, pkg.F32, m, n, k)
        ctx.synchronize()
        got = cd.download(np.float32, (m, n))
        assert_within_tolerance(got, oracle.gemm_f64(b, a), f"dense {m}x{n}x{k}")
        for t in (ad, bd, cd):
            t.free()


def test_two_dispatch_route_equals_fused_kernel(pkg, ctx):
    """dequant_bf16 + gemm_bf16 (the library's product at this length), the two-dispatch route of qgemm and the fused
    kernel feed the same bf16 weights to an fp32 accumulation: equal up to the order of the sums, at a full projection
    shape (max difference a few fp32 steps of the largest partial sums)."""
    m, n, k = 512, 4096, 4096
    words, s, z, _ = seeded_case(930, n, k, 4, 64)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
    x = act_rounded(kat.seeded_activations(931, m, k), pkg.BF16, pkg)
    say("two-dispatch vs fused 512x4096x4096")
    fused = run_qgemm(ctx, pkg, w, x, pkg.F32, pkg.FLAG_FORCE_MFMA)
    scratch, yd = ctx.alloc(n * k * 2), ctx.alloc(m * n * 4)
    xd = ctx.upload(oracle.bf16_from_f32(x).reshape(m, k))
    ctx.dequant_bf16(w, scratch)
    ctx.gemm_bf16(xd, pkg.BF16, scratch, yd, pkg.F32, m, n, k)
    ctx.synchronize()
    two = yd.download(np.float32, (m, n))
    routed = run_qgemm(ctx, pkg, w, x, pkg.F32, pkg.FLAG_FORCE_TWO_STEP)
    for other, name in ((two, "dequant + dense entry"), (routed, "two-dispatch route")):
        assert np.max(np.abs(other - fused)) <= 2e-5 * max(1.0, float(np.max(np.abs(fused)))), name
    for t in (scratch, yd, xd):
        t.free()
    w.destroy()
