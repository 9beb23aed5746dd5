"""GPU parity tests of the matrix-core decode kernel over the TILE16 layout (4-bit, group 64), through
the C ABI: the same projections as gemv_q4_g64 / gemm_q4_g64 of the reference
(MetalSourceGenerator+Quantized.swift:496-575, :22-156) for 1 <= M <= 16 rows per launch.

Bars: unpacked codes and dequantised bf16 bit patterns of the re-tiled weight are bit-exact against
the CPU oracle; fp32 outputs within relative L2 <= 1e-3 and max-abs <= 2e-2 of an fp64 accumulation
of the same dequantised weights; bf16 outputs equal bf16_rne(fp32 outputs); token indices exact.
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


def _fmt(pkg):
    return pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)


def _run(ctx, pkg, w, x, y_dtype, use_qgemm=False, flags=0):
    m, k = x.shape
    n = int(w.info.n_rows)
    xd = ctx.upload(oracle.bf16_from_f32(x).reshape(x.shape))
    yd = ctx.alloc(m * n * (4 if y_dtype == pkg.F32 else 2))
    ctx.fill(yd, 0x7FC00000 if y_dtype == pkg.F32 else 0x7FC07FC0)
    (ctx.qgemm if use_qgemm else ctx.qgemv)(w, xd, pkg.BF16, yd, y_dtype, m, 0, 0, flags)
    ctx.synchronize()
    y = out_from_device(yd, y_dtype, (m, n), pkg)
    xd.free(); yd.free()
    return y


@pytest.mark.parametrize("n,k", [(16, 128), (37, 256), (1, 128), (130, 1024 + 128), (512, 4096)])
def test_retiled_weight_unpacks_and_dequantises_bit_exactly(pkg, ctx, n, k):
    """The device re-tiling (rows -> TILE16 records, nibble permutation included) loses nothing:
    unpack_codes and dequant_bf16 on the re-tiled weight equal the CPU oracle on the source planes,
    for both sources (MLX planes with bf16 scales, STAF blocks with f16 scales)."""
    words, s, z, wq = seeded_case(2000 + n, n, k, 4, 64)
    want_codes = oracle.unpack_plane_codes(4, n, k, words)
    w = ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)
    assert w.info.layout == pkg.LAYOUT_TILE16 and w.info.weight_bytes == n * (k // 64) * 36
    out = ctx.alloc(n * k); ctx.unpack_codes(w, out); ctx.synchronize()
    assert np.array_equal(out.download(np.uint8, (n, k)), want_codes)
    deq = ctx.alloc(n * k * 2); ctx.dequant_bf16(w, deq); ctx.synchronize()
    assert np.array_equal(deq.download(np.uint16, (n, k)), oracle.bf16_from_f32(wq).reshape(n, k))
    out.free(); deq.free(); w.destroy()
    # from STAF blocks (f16 headers)
    rng = np.random.default_rng(n * 7 + k)
    codes = rng.integers(0, 16, (n, k), dtype=np.uint8)
    case = Case(4, 64, codes, rng.choice([0.0625, 0.125, 0.5], (n, k // 64)), rng.integers(-8, 8, (n, k // 64)) * 0.125)
    blocks = case.staf_blocks()
    w = ctx.weight_prepare_staf(_fmt(pkg), n, k, blocks, pkg.LAYOUT_TILE16)
    out = ctx.alloc(n * k); ctx.unpack_codes(w, out); ctx.synchronize()
    assert np.array_equal(out.download(np.uint8, (n, k)), codes)
    deq = ctx.alloc(n * k * 2); ctx.dequant_bf16(w, deq); ctx.synchronize()
    assert np.array_equal(deq.download(np.uint16, (n, k)), oracle.dequant_staf_bf16(4, 64, n, k, blocks).reshape(n, k))
    out.free(); deq.free(); w.destroy()


LLAMA = {"q_o": (4096, 4096), "k_v": (1024, 4096), "gate_up": (14336, 4096), "down": (4096, 14336)}


@pytest.mark.parametrize("name", list(LLAMA))
def test_tile16_llama_shapes_all_batch_sizes(pkg, ctx, name):
    """benchmark config 1 shapes, M = 1, 2, 4, 8 (and the sizes in between up to 16)."""
    n, k = LLAMA[name]
    words, s, z, wq = seeded_case(2100 + n % 89, n, k, 4, 64)
    w = ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)
    for m in (1, 2, 3, 4, 5, 8, 13, 16):
        x = act_rounded(kat.seeded_activations(2200 + m, m, k), pkg.BF16, pkg)
        say(f"tile16 {name} M={m}")
        want = oracle.gemm_f64(wq, x)
        use_qgemm = m > 8
        y32 = _run(ctx, pkg, w, x, pkg.F32, use_qgemm)
        rel, _ = assert_within_tolerance(y32, want, f"{name} M={m}")
        assert rel < 1e-4
        ybf = _run(ctx, pkg, w, x, pkg.BF16, use_qgemm)
        assert np.array_equal(oracle.bf16_from_f32(ybf), oracle.bf16_from_f32(y32))
    w.destroy()


def test_tile16_ragged_shapes_and_long_batches(pkg, ctx):
    """N off the 16-row tile, single row, short and long K, f16 scales, M beyond one launch."""
    for i, (n, k) in enumerate([(1, 128), (5, 256), (17, 128), (130, 2048 + 128), (4099, 384), (33, 14336)]):
        words, s, z, wq = seeded_case(2300 + i, n, k, 4, 64)
        w = ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)
        for m in (1, 3, 7, 16, 21, 40):
            x = act_rounded(kat.seeded_activations(2400 + i + m, m, k), pkg.BF16, pkg)
            say(f"tile16 ragged {k}->{n} M={m}")
            got = _run(ctx, pkg, w, x, pkg.F32, use_qgemm=m > 8)
            # beyond 32 rows (two launches) the projection runs on the prefill kernel, whose weights are rounded to bf16
            ref_w = wq if m <= 32 else oracle.bf16_to_f32(oracle.bf16_from_f32(wq)).reshape(wq.shape)
            assert_within_tolerance(got, oracle.gemm_f64(ref_w, x), f"{k}->{n} M={m}")
        w.destroy()
    # f16 scale words (STAF source)
    rng = np.random.default_rng(5)
    n, k = 70, 512
    codes = rng.integers(0, 16, (n, k), dtype=np.uint8)
    scales = rng.choice([0.0625, 0.125, 0.25], (n, k // 64)); zeros = rng.integers(-8, 8, (n, k // 64)) * 0.0625
    case = Case(4, 64, codes, scales, zeros)
    w = ctx.weight_prepare_staf(_fmt(pkg), n, k, case.staf_blocks(), pkg.LAYOUT_TILE16)
    wq = (scales.repeat(64, axis=1) * codes + zeros.repeat(64, axis=1)).astype(np.float32)
    for m in (1, 6):
        x = act_rounded(kat.seeded_activations(2500 + m, m, k), pkg.BF16, pkg)
        assert_within_tolerance(_run(ctx, pkg, w, x, pkg.F32), oracle.gemm_f64(wq, x), f"f16 scales M={m}")
    w.destroy()


@pytest.mark.parametrize("tiles_per_cu", [3, 5, 6, 7, 8])
def test_tile16_one_round_workgroup_shapes(pkg, ctx, tiles_per_cu):
    """From three activation rows on, a matrix with three to eight row tiles per CU runs as one round of workgroups that
    each take their CU's share of row tiles (4 x 3, 2 x 5 ... 2 x 8 wavefronts): every such shape, ragged last tile,
    K of one and of several blocks per wavefront, single and fused launches."""
    cus = ctx.device_info().compute_units
    # just past (tiles_per_cu - 1) tiles per CU with a ragged last tile; three per CU exist only as exactly 3 x CUs tiles
    n = 16 * cus * 3 if tiles_per_cu == 3 else 16 * (cus * (tiles_per_cu - 1) + 3) + 5
    for k in (128, 1280):
        words, s, z, wq = seeded_case(2800 + tiles_per_cu + k, n, k, 4, 64)
        w = ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)
        for m in (3, 8, 16):
            st = w.plan_prefill_steps(m)[0]
            assert st.device_kernel == "gemv_tile16_q4_g64" and st.grid[0] <= cus, (st.grid[0], cus)
            assert st.block[0] == 64 * tiles_per_cu * (4 if tiles_per_cu <= 4 else 2), st.block[0]
            x = act_rounded(kat.seeded_activations(2850 + m, m, k), pkg.BF16, pkg)
            say(f"tile16 one round, {tiles_per_cu} tiles per CU, K={k} M={m}")
            assert_within_tolerance(_run(ctx, pkg, w, x, pkg.F32, use_qgemm=True), oracle.gemm_f64(wq, x), f"{tiles_per_cu} K={k} M={m}")
        w.destroy()


def test_tile16_large_batch_few_tiles_per_cu(pkg, ctx):
    """Sixteen activation rows of 4096 (131 KB staged, one workgroup per CU) over matrices with one, two and three row
    tiles per CU: sixteen wavefronts on one row tile, 8 x 2 and 4 x 3."""
    cus = ctx.device_info().compute_units
    k, m = 4096, 16
    for i, tiles in enumerate((cus - 3, cus + cus // 2, 2 * cus + 9)):
        n = 16 * tiles - 7
        words, s, z, wq = seeded_case(2880 + i, n, k, 4, 64)
        w = ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)
        st = w.plan_prefill_steps(m)[0]
        assert st.device_kernel == "gemv_tile16_q4_g64" and st.grid[0] <= cus and st.block[0] == (1024, 1024, 768)[i], (st.grid[0], st.block[0])
        x = act_rounded(kat.seeded_activations(2885 + i, m, k), pkg.BF16, pkg)
        say(f"tile16 M=16, {tiles} row tiles on {cus} CUs")
        assert_within_tolerance(_run(ctx, pkg, w, x, pkg.F32, use_qgemm=True), oracle.gemm_f64(wq, x), f"{tiles} tiles")
        w.destroy()


def test_tile16_long_rows_split_over_k_parts(pkg, ctx):
    """Rows too long for M staged activation rows in LDS (14336 codes from M = 5, 65536 codes at M = 1) run as one
    launch whose workgroups each take a part of K, plus a launch that adds the parts: every output type, strided
    rows, ragged N, agreement with the per-code kernel, the plan record, and replay from a HIP graph."""
    for i, (n, k) in enumerate([(4096, 14336), (50, 14336), (33, 65536)]):
        words, s, z, wq = seeded_case(2600 + i, n, k, 4, 64)
        w = ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)
        for m in ((5, 8, 13, 16) if k == 14336 else (1, 2, 16)):
            x = act_rounded(kat.seeded_activations(2650 + i + m, m, k), pkg.BF16, pkg)
            say(f"tile16 K parts {k}->{n} M={m}")
            st = w.plan_prefill_steps(m)[0] if m > 1 else w.plan_decode_step(1)
            assert st.device_kernel == "gemv_tile16_q4_g64" and not st.used_fallback and st.lds_bytes <= 144 * 1024
            want = oracle.gemm_f64(wq, x)
            y32 = _run(ctx, pkg, w, x, pkg.F32, use_qgemm=True)
            rel, _ = assert_within_tolerance(y32, want, f"{k}->{n} M={m}")
            assert rel < 1e-4
            assert np.array_equal(oracle.bf16_from_f32(_run(ctx, pkg, w, x, pkg.BF16, use_qgemm=True)), oracle.bf16_from_f32(y32))
            if n <= 50:
                y16 = _run(ctx, pkg, w, x, pkg.F16, use_qgemm=True)
                assert np.array_equal(y16.astype(np.float16), y32.astype(np.float16))
                assert_within_tolerance(_run(ctx, pkg, w, x, pkg.F32, True, pkg.FLAG_FORCE_GENERIC), want, "per-code kernel")
        w.destroy()
    # strided activation and output rows, then the same projection from a plan and its graph, three replays; on a
    # context of its own, so that the scratch buffer of partial results starts small and a later, larger user of it
    # (a split-K prefill projection) makes it grow while the graph still holds the address it was captured with
    c2 = pkg.Context(0)
    n, k, m, xs, ys = 200, 14336, 16, 14336 + 64, 200 + 24
    words, s, z, wq = seeded_case(2690, n, k, 4, 64)
    w = c2.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)
    x = act_rounded(kat.seeded_activations(2691, m, k), pkg.BF16, pkg)
    xh = np.zeros((m, xs), np.uint16); xh[:, :k] = oracle.bf16_from_f32(x).reshape(m, k)
    xd = c2.upload(xh); yd = c2.alloc(m * ys * 4)
    c2.fill(yd, 0x7FC00000)
    c2.qgemm(w, xd, pkg.BF16, yd, pkg.F32, m, xs, ys); c2.synchronize()
    got = yd.download(np.float32, (m, ys))
    assert_within_tolerance(got[:, :n], oracle.gemm_f64(wq, x), "strided rows")
    assert np.isnan(got[:, n:]).all()                         # nothing written between the rows
    plan = pkg.DispatchPlan(c2)
    plan.add_linear(w, xd, pkg.BF16, yd, pkg.F32, m, xs, ys)
    stream = c2.stream_create()
    plan.graph_build(stream)
    rng = np.random.default_rng(2692)
    for rep in range(4):
        if rep == 3:
            nb, mb = 4096, 2048
            wb = c2.weight_prepare_mlx(_fmt(pkg), rng.integers(0, 2**32, (nb, k // 8), dtype=np.uint32),
                                       np.full((nb, k // 64), 0x3C00, np.uint16), np.zeros((nb, k // 64), np.uint16), pkg.F16)
            xb = c2.alloc(mb * k * 2); yb = c2.alloc(mb * nb * 2)
            c2.fill(xb, 0x3C003C00)
            say("tile16 K parts: a split-K prefill projection grows the scratch buffer")
            c2.qgemm(wb, xb, pkg.BF16, yb, pkg.BF16, mb); c2.synchronize()
            xb.free(); yb.free(); wb.destroy()
        c2.fill(yd, 0x7FC00000, stream)
        plan.graph_launch(stream) if rep else plan.encode(stream)
        c2.synchronize(stream)
        again = yd.download(np.float32, (m, ys))
        assert np.array_equal(again[:, :n], got[:, :n]) and np.isnan(again[:, n:]).all(), rep
    plan.destroy(); xd.free(); yd.free(); w.destroy(); c2.close()
    # two long-row projections of one activation batch: no fused launch, each runs split, results as above
    ws, wqs = [], []
    for j, n2 in enumerate((48, 130)):
        words, s, z, wq = seeded_case(2695 + j, n2, 14336, 4, 64)
        ws.append(ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)); wqs.append(wq)
    x = act_rounded(kat.seeded_activations(2697, 8, 14336), pkg.BF16, pkg)
    xd = ctx.upload(oracle.bf16_from_f32(x).reshape(x.shape)); yds = [ctx.alloc(8 * n2 * 4) for n2 in (48, 130)]
    ctx.batched_qgemm(ws, xd, pkg.BF16, yds, pkg.F32, 8); ctx.synchronize()
    for j, n2 in enumerate((48, 130)):
        assert_within_tolerance(yds[j].download(np.float32, (8, n2)), oracle.gemm_f64(wqs[j], x), f"batched long rows {j}")
    xd.free()
    for b in yds:
        b.free()
    for w2 in ws:
        w2.destroy()


def test_tile16_exact_small_integers_and_scaling(pkg, ctx):
    """Exactly representable case (every partial sum an integer multiple of 2^-6 below 2^20): the
    result must be exact whatever the summation order; and y(2x) == 2*y(x) bit for bit at full size."""
    rng = np.random.default_rng(11)
    n, k = 100, 1024
    codes = rng.integers(0, 16, (n, k), dtype=np.uint8)
    scales = rng.choice([0.125, 0.25, 0.5], (n, k // 64)); zeros = rng.integers(-4, 5, (n, k // 64)) * 0.25
    case = Case(4, 64, codes, scales, zeros)
    wq = scales.repeat(64, axis=1) * codes + zeros.repeat(64, axis=1)
    for sb, w in ((pkg.F16, ctx.weight_prepare_staf(_fmt(pkg), n, k, case.staf_blocks(), pkg.LAYOUT_TILE16)),
                  (pkg.BF16, ctx.weight_prepare_mlx(_fmt(pkg), *case.planes(pkg.BF16, pkg), pkg.BF16, pkg.LAYOUT_TILE16))):
        for m in (1, 2, 4, 9):
            x = rng.integers(-8, 9, (m, k)).astype(np.float32) * 0.125
            got = _run(ctx, pkg, w, x, pkg.F32, use_qgemm=m > 8)
            assert np.array_equal(got.astype(np.float64), x.astype(np.float64) @ wq.T), (sb, m)
        w.destroy()
    n, k = 14336, 4096
    words, s, z, _ = seeded_case(2600, n, k, 4, 64)
    w = ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)
    x = act_rounded(kat.seeded_activations(2601, 2, k), pkg.BF16, pkg)
    y1, y2 = _run(ctx, pkg, w, x, pkg.F32), _run(ctx, pkg, w, 2.0 * x, pkg.F32)
    assert np.array_equal(2.0 * y1, y2)
    w.destroy()


def test_tile16_batched_projections_one_launch(pkg, ctx):
    for ns, k in [((4096, 1024, 1024), 4096), ((14336, 14336), 4096), ((5, 17, 130), 256)]:
        ws, wqs = [], []
        for i, n in enumerate(ns):
            words, s, z, wq = seeded_case(2700 + i + n % 13, n, k, 4, 64)
            ws.append(ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)); wqs.append(wq)
        for m in (1, 4, 11):
            x = act_rounded(kat.seeded_activations(2750 + m, m, k), pkg.BF16, pkg)
            xd = ctx.upload(oracle.bf16_from_f32(x).reshape(x.shape))
            yds = [ctx.alloc(m * n * 4) for n in ns]
            say(f"tile16 batched {ns} M={m}")
            ctx.batched_qgemm(ws, xd, pkg.BF16, yds, pkg.F32, m)
            ctx.synchronize()
            for i, n in enumerate(ns):
                assert_within_tolerance(yds[i].download(np.float32, (m, n)), oracle.gemm_f64(wqs[i], x), f"{ns} seg {i}")
            xd.free()
            for b in yds:
                b.free()
        for w in ws:
            w.destroy()


def test_tile16_lm_head_fused_argmax(pkg, ctx):
    """benchmark config 4 (2048 -> 65536): token == lowest-index argmax of the GPU's own fp32 logits and
    of the CPU reference logits; ties resolve to the lowest index."""
    n, k = 65536, 2048
    words, s, z, wq = seeded_case(2800, n, k, 4, 64)
    w = ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)
    x = act_rounded(kat.seeded_activations(2801, 1, k), pkg.BF16, pkg)
    xd = ctx.upload(oracle.bf16_from_f32(x)); logits = ctx.alloc(n * 4); tok = ctx.upload(np.array([-7], np.int32))
    for rep in range(3):                                     # the scratch cells reset themselves
        ctx.lmhead_argmax(w, xd, pkg.BF16, logits, tok)
        ctx.synchronize()
        got = logits.download(np.float32)
        assert int(tok.download(np.int32)[0]) == oracle.argmax_lowest(got)
    want = oracle.gemm_f64(wq, x)[0]
    assert_within_tolerance(got, want, "lm head logits")
    assert int(tok.download(np.int32)[0]) == int(np.argmax(want))
    ctx.lmhead_argmax(w, xd, pkg.BF16, None, tok)            # token only
    ctx.synchronize()
    assert int(tok.download(np.int32)[0]) == int(np.argmax(want))
    w.destroy()
    # ties: identical rows placed across tile and workgroup boundaries
    n, k = 4096, 256
    codes = np.zeros((n, k), np.uint8); codes[[7, 15, 16, 1000, 4095]] = 9
    case = Case(4, 64, codes, np.full((n, k // 64), 0.25), np.full((n, k // 64), -0.5))
    w = ctx.weight_prepare_staf(_fmt(pkg), n, k, case.staf_blocks(), pkg.LAYOUT_TILE16)
    x = np.full((1, k), 0.5, np.float32)
    xd2 = ctx.upload(oracle.bf16_from_f32(x)); lg2 = ctx.alloc(n * 4)
    ctx.lmhead_argmax(w, xd2, pkg.BF16, lg2, tok); ctx.synchronize()
    assert int(tok.download(np.int32)[0]) == 7
    w.destroy()
    for b in (xd, logits, tok, xd2, lg2):
        b.free()


def test_tile16_prefill_runs_on_the_matrix_cores(pkg, ctx):
    """Above 32 rows (two launches of the small-batch kernel) a TILE16 weight feeds the prefill GEMM directly from its
    records.  The arithmetic is that of the same kernel on the split planes (same bf16 weights, same contraction
    order): identical bits; the plan record names the matrix-core kernel."""
    for i, (m, n, k) in enumerate([(17, 130, 2048 + 128), (64, 4099, 384), (300, 257, 128), (512, 4096, 4096),
                                   (2048, 1024, 512)]):
        words, s, z, wq = seeded_case(2700 + i, n, k, 4, 64)
        wt = ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)
        wp = ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
        x = act_rounded(kat.seeded_activations(2750 + i, m, k), pkg.BF16, pkg)
        say(f"tile16 prefill {k}->{n} M={m}")
        two_step_from = 2048 if k > n else 768 if n >= 8192 else 512       # rows from which dequantise once + dense GEMM
        got = _run(ctx, pkg, wt, x, pkg.F32, use_qgemm=True, flags=0 if 32 < m < two_step_from else pkg.FLAG_FORCE_MFMA)
        same = _run(ctx, pkg, wp, x, pkg.F32, use_qgemm=True, flags=pkg.FLAG_FORCE_MFMA | pkg.FLAG_PROBE_TILED)   # the same tiled kernel (long prompts on planes would take the wide-tile one)
        assert np.array_equal(got, same), f"{k}->{n} M={m}: records and planes disagree"
        if m * n * k <= 2 ** 28:
            wb = oracle.bf16_to_f32(oracle.bf16_from_f32(wq)).reshape(wq.shape)
            assert_within_tolerance(got, oracle.gemm_f64(wb, x), f"{k}->{n} M={m}")
        st = wt.plan_prefill_steps(m, flags=pkg.FLAG_FORCE_MFMA)[0]
        assert st.device_kernel == "qgemm_mfma_q4_g64" and not st.used_fallback
        unforced = [s.device_kernel for s in wt.plan_prefill_steps(m)]     # long prompts: dequantise once + dense GEMM
        assert unforced == (["dequant_q4_g64_bf16", "hipblaslt_gemm_bf16"] if m >= two_step_from else
                            ["qgemm_mfma_q4_g64"] if m > 32 else ["gemv_tile16_q4_g64"])
        if m <= 32:                                          # two launches of the small-batch kernel: unrounded weights
            assert_within_tolerance(_run(ctx, pkg, wt, x, pkg.F32, use_qgemm=True), oracle.gemm_f64(wq, x), f"M={m} in steps")
        wt.destroy(); wp.destroy()
    # f16 scale words (a STAF source)
    rng = np.random.default_rng(6)
    n, k, m = 96, 256, 40
    case = Case(4, 64, rng.integers(0, 16, (n, k), dtype=np.uint8), rng.choice([0.0625, 0.125], (n, k // 64)),
                rng.integers(-8, 8, (n, k // 64)) * 0.0625)
    wt = ctx.weight_prepare_staf(_fmt(pkg), n, k, case.staf_blocks(), pkg.LAYOUT_TILE16)
    x = act_rounded(kat.seeded_activations(2790, m, k), pkg.BF16, pkg)
    wq = (case.scales.repeat(64, axis=1) * case.codes + case.zeros.repeat(64, axis=1)).astype(np.float32)
    assert_within_tolerance(_run(ctx, pkg, wt, x, pkg.F32, use_qgemm=True), oracle.gemm_f64(wq, x), "f16 scales")   # exact in bf16
    wt.destroy()


def test_tile16_errors_and_plan_records(pkg, ctx):
    fmt8 = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(8, 32)
    words, s, z, _ = seeded_case(2900, 16, 128, 8, 32)
    with pytest.raises(pkg.MI355QError):                      # only q4 g64
        ctx.weight_prepare_mlx(fmt8, words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)
    words, s, z, _ = seeded_case(2901, 16, 192, 4, 64)
    with pytest.raises(pkg.MI355QError):                      # K % 128
        ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)
    words, s, z, wq = seeded_case(2902, 256, 512, 4, 64)
    w = ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)
    st = w.plan_decode_step(4)
    assert st.device_kernel == "gemv_tile16_q4_g64" and not st.used_fallback and st.grid[0] == 16
    # f32 activations are not served by the tile kernel: the per-code kernel runs and agrees
    x = act_rounded(kat.seeded_activations(2903, 2, 512), pkg.BF16, pkg)
    xd = ctx.upload(x.astype(np.float32)); yd = ctx.alloc(2 * 256 * 4)
    ctx.qgemv(w, xd, pkg.F32, yd, pkg.F32, 2); ctx.synchronize()
    assert_within_tolerance(yd.download(np.float32, (2, 256)), oracle.gemm_f64(wq, x), "f32 activations")
    got_generic = _run(ctx, pkg, w, x, pkg.F32, flags=pkg.FLAG_FORCE_GENERIC)
    assert_within_tolerance(got_generic, oracle.gemm_f64(wq, x), "forced generic")
    xd.free(); yd.free(); w.destroy()


def test_tile16_plan_replay_and_graph(pkg, ctx):
    k = 1024
    ns = (512, 256, 2048)
    ws = []
    for i, n in enumerate(ns):
        words, s, z, _ = seeded_case(3000 + i, n, k, 4, 64)
        ws.append(ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_TILE16))
    x = ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(3010, 1, k)))
    ys = [ctx.alloc(n * 4) for n in ns]
    tok = ctx.upload(np.array([-3], np.int32))
    ctx.batched_qgemm(ws[:2], x, pkg.BF16, ys[:2], pkg.F32, 1)
    ctx.lmhead_argmax(ws[2], x, pkg.BF16, ys[2], tok)
    ctx.synchronize()
    eager = [y.download(np.float32) for y in ys]; etok = int(tok.download(np.int32)[0])
    assert etok == oracle.argmax_lowest(eager[2])
    plan = pkg.DispatchPlan(ctx)
    plan.add_batched_linear(ws[:2], x, pkg.BF16, ys[:2], pkg.F32, 1)
    plan.add_output_head(ws[2], x, pkg.BF16, ys[2], tok)
    stream = ctx.stream_create()
    plan.graph_build(stream)
    for rep in range(3):
        for y in ys:
            ctx.fill(y, 0x7FC00000, stream)
        tok.upload(np.array([-3], np.int32))
        plan.graph_launch(stream) if rep else plan.encode(stream)
        ctx.synchronize(stream)
        for y, want in zip(ys, eager):
            assert np.array_equal(y.download(np.float32), want), rep
        assert int(tok.download(np.int32)[0]) == etok
    plan.destroy()
    for b in ys + [x, tok]:
        b.free()
    for w in ws:
        w.destroy()


@pytest.mark.parametrize("x_dtype_name", ["F16", "F32"])
def test_tile16_other_activation_types(pkg, ctx, x_dtype_name):
    """The tile kernel computes in bf16.  f16 rows are staged inside it as two bf16 rows each (eight rows a launch), up to
    sixteen fp32 rows run on it as three bf16 rows each; from sixteen rows both take the two-dispatch route
    (the matrix dequantised to the activations' type, then the dense library GEMM; fp32 from sixteen rows: bf16
    weights against split activations); forced, the per-code kernel takes all rows in one launch (no walk in steps
    of sixteen, eight ... one row)."""
    x_dtype = getattr(pkg, x_dtype_name)
    n, k = 96, 512
    words, s, z, wq = seeded_case(2931, n, k, 4, 64)
    w = ctx.weight_prepare_mlx(_fmt(pkg), words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)
    for m in (1, 13, 200):
        x = act_rounded(kat.seeded_activations(2932 + m, m, k), x_dtype, pkg)
        got = run_gemv(ctx, pkg, w, x, x_dtype, pkg.F32, 0, use_qgemm=True)
        # from sixteen rows fp32 activations meet bf16 weights (the reference's gemm_bf16_f32s); f16 ones f16 weights
        weights = wq if m < 16 or x_dtype == pkg.F16 else oracle.bf16_to_f32(oracle.bf16_from_f32(wq)).reshape(wq.shape)
        assert_within_tolerance(got, oracle.gemm_f64(weights, x), f"{x_dtype_name} M={m}")
        if m <= 15:
            want_kernel = "split_f32_bf16x3+gemv_tile16_q4_g64" if x_dtype == pkg.F32 else "gemv_tile16_q4_g64"
            assert w.plan_prefill_steps(m, x_dtype=x_dtype)[0].device_kernel == want_kernel
        elif m > 1:
            assert w.plan_prefill_steps(m, x_dtype=x_dtype)[0].kernel_family in ("libraryGEMM", "dequantToBFloat")
        slow = run_gemv(ctx, pkg, w, x, x_dtype, pkg.F32, pkg.FLAG_FORCE_GENERIC, use_qgemm=True)
        assert_within_tolerance(slow, oracle.gemm_f64(wq, x), f"{x_dtype_name} M={m}, per-code kernel")
    w.destroy()
