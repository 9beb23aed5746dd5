"""Streamed-weight matrix-core kernel (gemm_stream.hip): 17 to 96 activation rows (bf16, or f16 from nine rows) on 4- and
8-bit planes, the weights
dequantised in registers straight into the matrix cores' operand, the activations alone staged through LDS.

The kernel rounds every weight to bf16 exactly as the tiled prefill kernel does
(Sources/MetalCompiler/Generator/MetalSourceGenerator+Quantized.swift:361-416 writes bf16 weights for gemm_bf16_f32s), so
its results equal the tiled kernel's up to the order of the fp32 sums; both are checked against the fp64 oracle."""
import numpy as np
import pytest

import kat
import oracle
import sys

from gpu_util import act_rounded, act_to_device_array, out_from_device, rel_l2

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, file=sys.stderr, flush=True)


def _case(seed, n, k, group, sb, bits=4):
    w = kat.seeded_weights(seed, n, k)
    words, s, z = oracle.quantize_affine(w, bits, group, sb)
    return words, s, z, oracle.dequant_planes_f32(bits, group, n, k, words, s, z, sb)


def _run(ctx, pkg, w, x, m, n, y_dtype, flags, ypad=0, xpad=0, x_dtype=None):
    x_dtype = pkg.BF16 if x_dtype is None else x_dtype
    k = x.shape[1]
    xh = np.zeros((m, k + xpad), dtype=np.float32)
    xh[:, :k] = x
    xd = ctx.upload(act_to_device_array(xh, x_dtype, pkg))
    ysz = 4 if y_dtype == pkg.F32 else 2
    if (m * (n + ypad) * ysz) % 4:
        ypad += 1
    yd = ctx.alloc(m * (n + ypad) * ysz)
    ctx.fill(yd, 0x7FC07FC0 if ysz == 2 else 0x7FC00000)
    ctx.qgemm(w, xd, x_dtype, yd, y_dtype, m, k + xpad, n + ypad, flags)
    ctx.synchronize()
    got = out_from_device(yd, y_dtype, (m, n + ypad), pkg)
    xd.free(); yd.free()
    assert np.isnan(got[:, n:]).all(), "output padding overwritten"
    return got[:, :n]


@pytest.mark.parametrize("group,sb", [(64, "bf16"), (64, "f16"), (128, "bf16"), (128, "f16")])
def test_stream_kernel_against_oracle_and_tiled_kernel(pkg, ctx, group, sb):
    """Row counts across the three block counts, N off the 64-row workgroups and the 32-row blocks, K with and
    without whole 256-column iterations and split into parts (few rows, long K), padded strides."""
    sbo, sbp = (oracle.BF16, pkg.BF16) if sb == "bf16" else (oracle.F16, pkg.F16)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, group)
    shapes = [(17, 64, 128), (32, 1000, 320), (33, 130, 2112), (64, 4096, 1024), (65, 31, 4096), (96, 200, 8192 + 128),
              (90, 257, 256), (48, 64, 14336)]
    for i, (m, n, k) in enumerate(shapes):
        k += 64 if k % group else 0                      # 320 and 2112 columns: whole groups of 128 take 64 more
        say(f"stream q4 g{group} {sb} M={m} {k}->{n}")
        words, s, z, wq = _case(1300 + i, n, k, group, sbo)
        w = ctx.weight_prepare_mlx(fmt, words, s, z, sbp, pkg.LAYOUT_PLANES)
        x = act_rounded(kat.seeded_activations(1400 + i, m, k), pkg.BF16, pkg)
        want = oracle.gemm_f64(wq, x)
        got = _run(ctx, pkg, w, x, m, n, pkg.F32, pkg.FLAG_FORCE_STREAM, ypad=i % 3, xpad=8 * (i % 2))
        tiled = _run(ctx, pkg, w, x, m, n, pkg.F32, pkg.FLAG_FORCE_MFMA)
        if m <= 32:
            # one block of rows: the codes themselves in the operand, scale and bias applied to each K-tile's fp32 sums
            assert rel_l2(got, want) < 1e-5, (m, n, k, rel_l2(got, want))
            assert rel_l2(got, tiled) < 2.5e-3
        else:
            # bf16-rounded weights: 2^-9 relative per weight, 1.5e-3 in the L2 norm at most
            assert rel_l2(got, want) < 2.5e-3, (m, n, k, rel_l2(got, want))
            # the same rounded weights as the tiled kernel: only the order of the fp32 sums differs
            assert rel_l2(got, tiled) < 2e-6, (m, n, k, rel_l2(got, tiled))
        auto = _run(ctx, pkg, w, x, m, n, pkg.F32, 0)
        assert np.array_equal(auto, got), "rows 17 to 96 on eligible planes take the streamed-weight kernel unforced"
        step = w.plan_prefill_steps(m)[0]
        assert step.device_kernel == f"qgemm_stream_q4_g{group}" and step.kernel_family == "mfmaGEMM"
        assert not step.used_fallback and step.block[0] == 768
        for y_dtype in (pkg.BF16, pkg.F16):
            low = _run(ctx, pkg, w, x, m, n, y_dtype, pkg.FLAG_FORCE_STREAM, ypad=1)
            ref = act_rounded(got, y_dtype, pkg)
            assert np.array_equal(low, ref), "16-bit outputs are the fp32 results rounded once"
        w.destroy()


def test_stream_kernel_exact_on_integer_weights(pkg, ctx):
    """Weights and activations that bf16 holds exactly and sums that fp32 holds exactly: the result is the integer
    sum, whatever the order -- a dropped K-tile, a swapped word or a wrong row would show as a whole number off."""
    rng = np.random.default_rng(31)
    m, n, k = 70, 192, 1280
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    q = rng.integers(0, 16, size=(n, k)).astype(np.uint32)
    scales = np.ones((n, k // 64), dtype=np.float32) * 2.0
    biases = -rng.integers(0, 8, size=(n, k // 64)).astype(np.float32)
    words = (q.reshape(n, k // 8, 8) << (4 * np.arange(8, dtype=np.uint32))).sum(axis=2).astype(np.uint32)
    w = ctx.weight_prepare_mlx(fmt, words, oracle.bf16_from_f32(scales), oracle.bf16_from_f32(biases), pkg.BF16,
                               pkg.LAYOUT_PLANES)
    x = rng.integers(-3, 4, size=(m, k)).astype(np.float32)
    wq = 2.0 * q.astype(np.float64) + np.repeat(biases.astype(np.float64), 64, axis=1)
    want = x.astype(np.float64) @ wq.T
    got = _run(ctx, pkg, w, x, m, n, pkg.F32, pkg.FLAG_FORCE_STREAM)
    assert np.array_equal(got.astype(np.float64), want)
    w.destroy()


def test_stream_kernel_refuses_what_it_does_not_read(pkg, ctx):
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    words, s, z, _ = _case(1500, 64, 128, 64, oracle.BF16)
    w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
    x = act_rounded(kat.seeded_activations(1, 97, 128), pkg.BF16, pkg)
    with pytest.raises(pkg.MI355QError):
        _run(ctx, pkg, w, x, 97, 64, pkg.F32, pkg.FLAG_FORCE_STREAM)           # more than 96 rows
    with pytest.raises(pkg.MI355QError):
        _run(ctx, pkg, w, x[:20], 20, 64, pkg.F32, pkg.FLAG_FORCE_STREAM | pkg.FLAG_FORCE_MFMA)
    ws = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_TILE16)
    with pytest.raises(pkg.MI355QError):
        _run(ctx, pkg, ws, x[:20], 20, 64, pkg.F32, pkg.FLAG_FORCE_STREAM)     # tile records
    fmt8 = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(6, 16)
    words8, s8, z8 = oracle.quantize_affine(kat.seeded_weights(1501, 64, 128), 6, 16, oracle.BF16)
    w8 = ctx.weight_prepare_mlx(fmt8, words8, s8, z8, pkg.BF16, pkg.LAYOUT_PLANES)
    with pytest.raises(pkg.MI355QError):
        _run(ctx, pkg, w8, x[:20], 20, 64, pkg.F32, pkg.FLAG_FORCE_STREAM)     # groups of 16: two in a lane's 32 codes
    for t in (w, ws, w8):
        t.destroy()


@pytest.mark.parametrize("count,m", [(2, 40), (3, 24), (3, 96), (2, 70)])
def test_stream_kernel_shared_launch_equals_separate_launches(pkg, ctx, count, m):
    """Two or three matrices that share the activations (gate+up, q+k+v) as one launch of the streamed-weight kernel:
    every output has the bits of its own launch; row counts off the 64-row workgroups, one and several K parts."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    k = 1024 if count == 2 else 4096
    ns = [300, 64, 130][:count] if count == 3 else [2048 + 40, 1000]
    ws, wqs = [], []
    for i, n in enumerate(ns):
        words, s, z, wq = _case(1600 + 10 * count + i, n, k, 64, oracle.BF16)
        ws.append(ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES))
        wqs.append(wq)
    x = act_rounded(kat.seeded_activations(1700 + count, m, k), pkg.BF16, pkg)
    xd = ctx.upload(act_to_device_array(x, pkg.BF16, pkg))
    for y_dtype in (pkg.F32, pkg.BF16):
        ysz = 4 if y_dtype == pkg.F32 else 2
        say(f"shared launch of {count} M={m} K={k} N={ns} y {y_dtype}")
        dense = [ctx.alloc(m * n * ysz) for n in ns]               # batched outputs are dense: row stride N_i
        ctx.batched_qgemm(ws, xd, pkg.BF16, dense, y_dtype, m, 0, 0)
        ctx.synchronize()
        for w, wq, n, yd in zip(ws, wqs, ns, dense):
            got = out_from_device(yd, y_dtype, (m, n), pkg)
            alone = _run(ctx, pkg, w, x, m, n, y_dtype, pkg.FLAG_FORCE_STREAM)
            # the K parts follow the launch's workgroup count, so the order of the fp32 sums may differ from a launch alone
            assert rel_l2(got, alone) < (2e-6 if y_dtype == pkg.F32 else 1e-3), (count, m, n)
            assert rel_l2(got, oracle.gemm_f64(wq, x)) < (2.5e-3 if y_dtype == pkg.F32 else 5e-3)
        for b in dense:
            b.free()
    xd.free()
    for w in ws:
        w.destroy()


@pytest.mark.parametrize("bits,group", [(8, 32), (8, 64), (8, 128)])
def test_stream_kernel_eight_bit_codes(pkg, ctx, bits, group):
    """8-bit codes: a lane's 32 codes are eight words, two per k-step; groups of 32 give the two halves of a K-tile
    their own (scale, bias) word.  Against the oracle, the tiled kernel (which reads q8 g32 / g64) and the plan record."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
    for i, (m, n, k) in enumerate([(17, 64, 128), (40, 1000, 384), (96, 130, 2176), (64, 4096, 1024), (33, 64, 14336)]):
        for sbo, sbp in ((oracle.BF16, pkg.BF16), (oracle.F16, pkg.F16)):
            say(f"stream q8 g{group} M={m} {k}->{n} sb {sbp}")
            words, s, z, wq = _case(1800 + i, n, k, group, sbo, bits=8)
            w = ctx.weight_prepare_mlx(fmt, words, s, z, sbp, pkg.LAYOUT_PLANES)
            x = act_rounded(kat.seeded_activations(1900 + i, m, k), pkg.BF16, pkg)
            got = _run(ctx, pkg, w, x, m, n, pkg.F32, pkg.FLAG_FORCE_STREAM, ypad=i % 2, xpad=8 * (i % 2))
            exact = m <= 32 and group % 64 == 0              # groups of 32 keep the rounded weights at every M
            assert rel_l2(got, oracle.gemm_f64(wq, x)) < (1e-5 if exact else 2.5e-3)
            if group != 128:
                tiled = _run(ctx, pkg, w, x, m, n, pkg.F32, pkg.FLAG_FORCE_MFMA)
                assert rel_l2(got, tiled) < (2.5e-3 if exact else 2e-6)
            auto = _run(ctx, pkg, w, x, m, n, pkg.F32, 0)
            assert np.array_equal(auto, got)
            assert w.plan_prefill_steps(m)[0].device_kernel == f"qgemm_stream_q8_g{group}"
            w.destroy()


@pytest.mark.parametrize("bits,group", [(4, 64), (4, 128), (8, 32), (8, 64)])
def test_stream_kernel_f16_activations(pkg, ctx, bits, group):
    """f16 activations (the reference's decode type): the weights are rounded to f16 instead of bf16 and the f16 matrix
    instruction multiplies; taken unforced from nine rows (one small-batch launch takes eight f16 rows)."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
    for i, (m, n, k) in enumerate([(9, 64, 128), (16, 300, 1024), (31, 1000, 384), (64, 130, 4096), (96, 257, 2176)]):
        say(f"stream f16 q{bits} g{group} M={m} {k}->{n}")
        words, s, z, wq = _case(2000 + i, n, k, group, oracle.BF16, bits=bits)
        w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
        x = act_rounded(kat.seeded_activations(2100 + i, m, k), pkg.F16, pkg)
        want = oracle.gemm_f64(wq, x)
        got = _run(ctx, pkg, w, x, m, n, pkg.F32, pkg.FLAG_FORCE_STREAM, ypad=i % 2, x_dtype=pkg.F16)
        exact = m <= 32 and group % 64 == 0
        # f16-rounded weights: 2^-12 relative per weight; unrounded in the one-block variant
        assert rel_l2(got, want) < (1e-5 if exact else 4e-4), rel_l2(got, want)
        two = _run(ctx, pkg, w, x, m, n, pkg.F32, pkg.FLAG_FORCE_TWO_STEP, x_dtype=pkg.F16) if m >= 16 else None
        if two is not None:
            assert rel_l2(got, two) < (4e-4 if exact else 2e-6)     # rounded: the same f16 weights, another order of the sums
        auto = _run(ctx, pkg, w, x, m, n, pkg.F32, 0, x_dtype=pkg.F16)
        assert np.array_equal(auto, got), "nine to 96 f16 rows on eligible planes take the streamed-weight kernel"
        low = _run(ctx, pkg, w, x, m, n, pkg.F16, pkg.FLAG_FORCE_STREAM, x_dtype=pkg.F16)
        assert np.array_equal(low, act_rounded(got, pkg.F16, pkg))
        step = w.plan_prefill_steps(m, x_dtype=pkg.F16)[0]
        assert step.device_kernel == f"qgemm_stream_q{bits}_g{group}"
        w.destroy()


@pytest.mark.parametrize("bits,group", [(4, 64), (4, 128), (8, 32), (8, 64), (8, 128)])
def test_stream_kernel_reads_staf_blocks_in_place(pkg, ctx, bits, group):
    """Weights left in the reference's interleaved blocks (a model.staf payload, zero copy): the lane's 32 codes lie in
    one block behind its (scale, zero) header, at a 4-byte aligned address.  Same results as from the planes bit for
    bit (the same f16 scales), against the oracle, unforced from nine rows (from three or five on large matrices, see the
    test below), bf16 and f16 activations, shared launch."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
    for i, (m, n, k) in enumerate([(3, 64, 128), (8, 300, 1024), (17, 300, 1024), (40, 1000, 384), (96, 130, 2176), (64, 200, 14336)]):
        if m < 9 and group % 64:
            continue                                     # groups of 32: from nine rows (rounded weights only)
        words, s, z, wq = _case(2200 + i, n, k, group, oracle.F16, bits=bits)
        wb = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.F16, pkg.LAYOUT_STAF_BLOCKS)
        wp = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.F16, pkg.LAYOUT_PLANES)
        for x_dtype in (pkg.BF16, pkg.F16):
            say(f"stream from blocks q{bits} g{group} M={m} {k}->{n} x {x_dtype}")
            x = act_rounded(kat.seeded_activations(2300 + i, m, k), x_dtype, pkg)
            got = _run(ctx, pkg, wb, x, m, n, pkg.F32, pkg.FLAG_FORCE_STREAM, ypad=i % 2, xpad=8 * (i % 2), x_dtype=x_dtype)
            ref = _run(ctx, pkg, wp, x, m, n, pkg.F32, pkg.FLAG_FORCE_STREAM, x_dtype=x_dtype)
            assert np.array_equal(got, ref), "blocks and planes hold the same codes and f16 scales"
            assert rel_l2(got, oracle.gemm_f64(wq, x)) < (1e-5 if m <= 32 and group % 64 == 0 else 2.5e-3 if x_dtype == pkg.BF16 else 4e-4)
            if m >= 9:                                   # matrices this small keep the in-place decode kernel up to eight rows
                auto = _run(ctx, pkg, wb, x, m, n, pkg.F32, 0, x_dtype=x_dtype)
                assert np.array_equal(auto, got), "nine to 96 rows on blocks take the streamed-weight kernel unforced"
                step = wb.plan_prefill_steps(m, x_dtype=x_dtype)[0]
                assert step.device_kernel == f"qgemm_stream_q{bits}_g{group}" and not step.used_fallback
        wb.destroy(); wp.destroy()
    # two matrices in blocks sharing the activations: one launch, the bits of separate launches
    m, k, ns = 33, 1024, [200, 1000]
    ws, alone = [], []
    x = act_rounded(kat.seeded_activations(2400, m, k), pkg.BF16, pkg)
    for j, n in enumerate(ns):
        words, s, z, _ = _case(2410 + j, n, k, group, oracle.F16, bits=bits)
        ws.append(ctx.weight_prepare_mlx(fmt, words, s, z, pkg.F16, pkg.LAYOUT_STAF_BLOCKS))
        alone.append(_run(ctx, pkg, ws[-1], x, m, n, pkg.F32, pkg.FLAG_FORCE_STREAM))
    xd = ctx.upload(act_to_device_array(x, pkg.BF16, pkg))
    yds = [ctx.alloc(m * n * 4) for n in ns]
    ctx.batched_qgemm(ws, xd, pkg.BF16, yds, pkg.F32, m, 0, 0)
    ctx.synchronize()
    for yd, n, want in zip(yds, ns, alone):
        assert rel_l2(out_from_device(yd, pkg.F32, (m, n), pkg), want) < 2e-6
        yd.free()
    xd.free()
    for w in ws:
        w.destroy()


def test_blocks_in_place_change_over_to_the_stream_kernel_by_size(pkg, ctx):
    """Blocks in place at a few rows: the in-place decode kernel re-reads the matrix for every four rows, the
    streamed-weight kernel (unrounded weights up to 32 rows) costs the same whatever the rows but has a floor of about
    10 us; matrices of 2^25 codes and more change over at three rows, of 2^23 at five, smaller ones at nine.  qgemv and
    qgemm agree, the result holds the decode tolerance, and a shared launch decides on the matrices together."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    for n, k, first in ((4096, 8192, 3), (2048, 4096, 5), (1024, 4096, 9)):
        words, s, z, wq = _case(2500 + first, n, k, 64, oracle.F16)
        w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.F16, pkg.LAYOUT_STAF_BLOCKS)
        for m in (first - 1, first):
            want = "qgemm_stream_q4_g64" if m >= first else "gemv_staf_q4_g64"
            if m <= 8:
                assert w.plan_decode_step(m).device_kernel == want, (n, k, m)
            assert w.plan_prefill_steps(m)[0].device_kernel == want, (n, k, m)
            for x_dtype in (pkg.BF16, pkg.F16):
                say(f"blocks {k}->{n} M={m} x {x_dtype}")
                x = act_rounded(kat.seeded_activations(2600 + m, m, k), x_dtype, pkg)
                got = _run(ctx, pkg, w, x, m, n, pkg.F32, 0, x_dtype=x_dtype)
                # unrounded weights on either kernel (the in-place kernel's f16 dot products: pairs summed in fp32)
                assert rel_l2(got, oracle.gemm_f64(wq, x)) < (1e-5 if m >= first else 1e-4)
                if m <= 8:
                    xd = ctx.upload(act_to_device_array(x, x_dtype, pkg)); yd = ctx.alloc(m * n * 4)
                    ctx.qgemv(w, xd, x_dtype, yd, pkg.F32, m); ctx.synchronize()
                    assert np.array_equal(out_from_device(yd, pkg.F32, (m, n), pkg), got)
                    xd.free(); yd.free()
        w.destroy()
    # q + k + v of 2^23 + 2^21 + 2^21 codes at five rows: together 1.5 * 2^23, one shared launch of the stream kernel
    ns, k, m = (2048, 512, 512), 4096, 5
    ws, wqs = [], []
    for j, n in enumerate(ns):
        words, s, z, wq = _case(2700 + j, n, k, 64, oracle.F16)
        ws.append(ctx.weight_prepare_mlx(fmt, words, s, z, pkg.F16, pkg.LAYOUT_STAF_BLOCKS)); wqs.append(wq)
    x = act_rounded(kat.seeded_activations(2710, m, k), pkg.BF16, pkg)
    xd = ctx.upload(act_to_device_array(x, pkg.BF16, pkg))
    yds = [ctx.alloc(m * n * 4) for n in ns]
    ctx.batched_qgemm(ws, xd, pkg.BF16, yds, pkg.F32, m); ctx.synchronize()
    for yd, n, wq, w in zip(yds, ns, wqs, ws):
        got = out_from_device(yd, pkg.F32, (m, n), pkg)
        assert rel_l2(got, oracle.gemm_f64(wq, x)) < 1e-5
        assert rel_l2(got, _run(ctx, pkg, w, x, m, n, pkg.F32, pkg.FLAG_FORCE_STREAM)) < 2e-6
        yd.free()
    xd.free()
    for w in ws:
        w.destroy()


def test_stream_kernel_in_a_plan_replayed_as_a_graph(pkg, ctx):
    """A shared launch (K split into parts: partial results in the context's scratch, a sum launch) and a single
    projection on the kernel inside one plan, replayed eagerly and as a HIP graph with eager work between the replays:
    every replay equals the first eager result bit for bit."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    m, k = 40, 2048
    ns = (192, 64, 64, 320)
    ws = []
    for i, n in enumerate(ns):
        words, s, z, _ = _case(2800 + i, n, k, 64, oracle.BF16)
        ws.append(ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES))
    xd = ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(2810, m, k)))
    ys = [ctx.alloc(m * n * 4) for n in ns]
    stream = ctx.stream_create()
    plan = pkg.DispatchPlan(ctx)
    plan.add_batched_linear(ws[:3], xd, pkg.BF16, ys[:3], pkg.F32, m)
    plan.add_linear(ws[3], xd, pkg.BF16, ys[3], pkg.F32, m)
    assert ws[3].plan_prefill_steps(m)[0].device_kernel == "qgemm_stream_q4_g64"
    plan.encode(stream); ctx.synchronize(stream)
    eager = [y.download(np.float32) for y in ys]
    assert all(np.all(np.isfinite(e)) for e in eager)

    def scrub():
        for y in ys:
            ctx.fill(y, 0x7FC00000, stream)

    plan.graph_build(stream)
    for rep in range(4):
        scrub(); plan.graph_launch(stream); ctx.synchronize(stream)
        for y, want in zip(ys, eager):
            assert np.array_equal(y.download(np.float32), want), f"graph replay {rep}"
        ctx.qgemm(ws[0], xd, pkg.BF16, ys[0], pkg.F32, m, 0, 0, 0, stream)          # eager work between the replays
        ctx.synchronize(stream)
    plan.destroy()
    for w in ws:
        w.destroy()
    xd.free()
    for y in ys:
        y.free()


@pytest.mark.parametrize("layout_name", ["planes", "blocks"])
def test_fp32_rows_ride_on_the_stream_kernel(pkg, ctx, layout_name):
    """fp32 activations (the reference's prefill type) split exactly into three bf16 rows each: up to ten fp32 rows (32
    bf16 rows) the streamed-weight kernel keeps the weights unrounded; from sixteen fp32 rows, where the rows would
    otherwise take the dequantise-once route with bf16 weights, it takes up to 32 of them with bf16 weights.  Eleven
    to fifteen rows keep their earlier routes (unrounded weights)."""
    layout = pkg.LAYOUT_PLANES if layout_name == "planes" else pkg.LAYOUT_STAF_BLOCKS
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    n, k = 300, 2048
    words, s, z, wq = _case(2900, n, k, 64, oracle.F16)
    w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.F16, layout)
    wb = oracle.bf16_to_f32(oracle.bf16_from_f32(wq)).reshape(wq.shape)
    for m in (3, 6, 10, 13, 16, 25, 32):
        say(f"fp32 rows {layout_name} M={m}")
        x = kat.seeded_activations(2910 + m, m, k)
        xd = ctx.upload(x)
        yd = ctx.alloc(m * n * 4)
        ctx.qgemm(w, xd, pkg.F32, yd, pkg.F32, m); ctx.synchronize()
        got = yd.download(np.float32, (m, n))
        kernel = w.plan_prefill_steps(m, x_dtype=pkg.F32)[0].device_kernel
        on_stream = kernel == "split_f32_bf16x3+qgemm_stream_q4_g64"
        if m <= 10:
            assert on_stream == (layout_name == "blocks" or m >= 6), (m, kernel)
        elif m >= 16:
            assert on_stream == (layout_name == "blocks" or m > 16), (m, kernel)
        else:
            assert not on_stream, (m, kernel)
        rounded = on_stream and 3 * m > 32
        want = oracle.gemm_f64(wb if rounded else wq, x)
        assert rel_l2(got, want) < (2e-6 if not rounded else 1e-5), (m, kernel, rel_l2(got, want))
        xd.free(); yd.free()
    w.destroy()


@pytest.mark.parametrize("bits", [2, 3, 5, 6])
def test_stream_kernel_other_widths(pkg, ctx, bits):
    """2-, 3-, 5- and 6-bit codes in groups of 64 (fields that straddle words included): planes and blocks, bf16 and f16
    rows; unrounded weights up to 32 rows, rounded to the activations' type beyond; the same bits from both layouts."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, 64)
    for i, (m, n, k) in enumerate([(5, 64, 128), (20, 300, 1024), (40, 1000, 384), (96, 130, 2176), (33, 70, 14336)]):
        words, s, z, wq = _case(3000 + 10 * bits + i, n, k, 64, oracle.F16, bits=bits)
        wp = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.F16, pkg.LAYOUT_PLANES)
        wb = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.F16, pkg.LAYOUT_STAF_BLOCKS)
        for x_dtype in (pkg.BF16, pkg.F16):
            say(f"stream q{bits} g64 M={m} {k}->{n} x {x_dtype}")
            x = act_rounded(kat.seeded_activations(3100 + i, m, k), x_dtype, pkg)
            got = _run(ctx, pkg, wp, x, m, n, pkg.F32, pkg.FLAG_FORCE_STREAM, ypad=i % 2, xpad=8 * (i % 2), x_dtype=x_dtype)
            bar = 1e-5 if m <= 32 else 2.5e-3 if x_dtype == pkg.BF16 else 4e-4
            assert rel_l2(got, oracle.gemm_f64(wq, x)) < bar, (m, rel_l2(got, oracle.gemm_f64(wq, x)))
            from_blocks = _run(ctx, pkg, wb, x, m, n, pkg.F32, pkg.FLAG_FORCE_STREAM, x_dtype=x_dtype)
            assert np.array_equal(from_blocks, got)
            if m >= 17:
                assert wp.plan_prefill_steps(m, x_dtype=x_dtype)[0].device_kernel == f"qgemm_stream_q{bits}_g64"
                assert np.array_equal(_run(ctx, pkg, wp, x, m, n, pkg.F32, 0, x_dtype=x_dtype), got)
        wp.destroy(); wb.destroy()
