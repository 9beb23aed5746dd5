"""GPU parity tests of the decode GEMV that reads STAF interleaved blocks in place (no repacking),
through the C ABI: the kernel a weight wrapped or uploaded straight from a model file runs
(reference kernels gemv_q{b}_g{g}: MetalSourceGenerator+Quantized.swift:496-575, reading the block
layout of QuantizationFormat.swift:1284-1312).

Bars: fp32 outputs within relative L2 <= 1e-3 and max-abs <= 2e-2 of an fp64 accumulation of the
same dequantised weights; bf16/f16 outputs equal the rounding of the fp32 outputs; the result of
the per-code kernel (FLAG_FORCE_GENERIC) on the same buffers within the same bars.
"""
import sys

import numpy as np
import pytest

import kat
import oracle
from gpu_util import Case, act_rounded, assert_within_tolerance, run_gemv

pytestmark = pytest.mark.gpu

# formats whose blocks are whole 32-bit words and that the in-place kernel is built for
FORMATS = [(4, 64), (4, 128), (8, 32), (8, 64), (8, 128), (2, 16), (2, 32), (2, 64), (3, 32), (3, 64), (5, 32), (5, 64),
           (6, 16), (6, 32), (6, 64)]


def say(*a):
    print(*a, file=sys.stderr, flush=True)


def _case(seed, n, k, bits, group):
    rng = np.random.default_rng(seed)
    codes = kat.random_codes(seed, n, k, bits)
    scales = rng.integers(1, 400, size=(n, k // group)) / 16384.0       # exact in f16
    zeros = rng.integers(-300, 300, size=(n, k // group)) / 8192.0
    return Case(bits, group, codes, scales, zeros)


def _row_alignment_k(bits, group):
    """Smallest K whose row of blocks is a multiple of 16 bytes."""
    bpb = 4 + group * bits // 8
    blocks = 16 // int(np.gcd(16, bpb))
    return blocks * group


def _q4_blocks(case):
    """STAF q4 blocks [N, row bytes] of a Case, vectorised (kat.staf_blocks walks every block in Python)."""
    n, k, g = case.n, case.k, case.group
    codes = case.codes.reshape(n, k // g, g // 2, 2)
    packed = (codes[..., 0] | (codes[..., 1] << 4)).astype(np.uint8)                 # LSB-first: even code in the low nibble
    hdr = np.stack([case.scales.astype(np.float16).view(np.uint16), case.zeros.astype(np.float16).view(np.uint16)], -1)
    hdr = np.ascontiguousarray(hdr.astype("<u2")).view(np.uint8).reshape(n, k // g, 4)
    return np.ascontiguousarray(np.concatenate([hdr, packed], axis=2).reshape(n, -1))


def _device_and_reference(pkg, ctx, case):
    """(STAF-layout device weight, dequantised fp32 reference weights); 4-bit cases use the vectorised block builder."""
    blocks = _q4_blocks(case).reshape(-1) if case.bits == 4 else case.staf_blocks()
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(case.bits, case.group)
    w = ctx.weight_prepare_staf(fmt, case.n, case.k, blocks, pkg.LAYOUT_STAF_BLOCKS)
    return w, oracle.dequant_staf_f32(case.bits, case.group, case.n, case.k, blocks)


@pytest.mark.parametrize("bits,group", FORMATS)
def test_in_place_gemv_formats_and_tails(pkg, ctx, bits, group):
    """Rows shorter than one span of 64 blocks, exactly one span, one span plus a tail, several spans;
    row counts that leave wavefronts partly or wholly past the end."""
    unit = _row_alignment_k(bits, group)
    ks = sorted({unit, 64 * group, 64 * group + unit, 3 * 64 * group + 2 * unit})
    for ci, k in enumerate(ks):
        for n in (1, 37, 700):
            case = _case(3000 + bits * 7 + group + ci, n, k, bits, group)
            w = case.device_weight(ctx, pkg, pkg.LAYOUT_STAF_BLOCKS)
            assert w.plan_decode_step(1).device_kernel == f"gemv_staf_q{bits}_g{group}"
            wq = oracle.dequant_staf_f32(bits, group, n, k, case.staf_blocks())
            for m in (1, 2, 3, 5, 8):
                x = act_rounded(kat.seeded_activations(3100 + m + ci, m, k), pkg.BF16, pkg)
                say(f"in-place q{bits}g{group} N={n} K={k} M={m}")
                got = run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.F32)
                assert_within_tolerance(got, oracle.gemm_f64(wq, x), f"q{bits}g{group} N={n} K={k} M={m}")
            # f16 activations (the reference's decode type): the same kernel with f16 code pairs, no fallback
            assert w.plan_decode_step(1, pkg.F16).device_kernel == f"gemv_staf_q{bits}_g{group}"
            for m in (1, 3, 8):
                x = act_rounded(kat.seeded_activations(3150 + m + ci, m, k), pkg.F16, pkg)
                got = run_gemv(ctx, pkg, w, x, pkg.F16, pkg.F32)
                assert_within_tolerance(got, oracle.gemm_f64(wq, x), f"f16 q{bits}g{group} N={n} K={k} M={m}")
            w.destroy()


def test_in_place_gemv_is_the_planned_kernel(pkg, ctx):
    """The plan names the in-place kernel for a STAF-layout weight with bf16 or f16 activations, the small-batch form
    of the two-dispatch route when the row of blocks is not a multiple of 16 bytes, the per-code kernel when forced."""
    case = _case(3200, 64, 4096, 4, 64)
    w = case.device_weight(ctx, pkg, pkg.LAYOUT_STAF_BLOCKS)
    step = w.plan_decode_step(1)
    assert step.device_kernel == "gemv_staf_q4_g64" and not step.used_fallback, step.device_kernel
    assert step.block[0] == 256 and step.grid[0] >= 1 and step.lds_bytes > 0
    f16_step = w.plan_decode_step(1, pkg.F16)
    assert f16_step.device_kernel == "gemv_staf_q4_g64" and not f16_step.used_fallback      # f16 activations too
    assert w.plan_decode_step(1, pkg.F32).device_kernel == "split_f32_bf16x3+gemv_staf_q4_g64"   # fp32: three bf16 rows
    assert w.plan_decode_step(8).device_kernel == "gemv_staf_q4_g64"         # a matrix this small keeps it up to eight rows
    forced = w.plan_decode_step(1, flags=pkg.FLAG_FORCE_GENERIC)
    assert forced.device_kernel == "gemv_generic" and forced.used_fallback
    w.destroy()
    odd = _case(3201, 16, 64 * 3, 4, 64)                    # 108-byte rows
    w = odd.device_weight(ctx, pkg, pkg.LAYOUT_STAF_BLOCKS)
    # the in-place decode kernel does not read 108-byte rows; the streamed-weight kernel does (4-byte aligned loads),
    # with unrounded weights, from the first row (forced, the per-code kernel)
    assert w.plan_decode_step(1).device_kernel == "qgemm_stream_q4_g64"
    assert w.plan_decode_step(2).device_kernel == "qgemm_stream_q4_g64"
    assert w.plan_decode_step(2, flags=pkg.FLAG_FORCE_GENERIC).device_kernel == "gemv_generic"
    x = act_rounded(kat.seeded_activations(3202, 1, odd.k), pkg.BF16, pkg)
    got = run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.F32)
    assert_within_tolerance(got, oracle.gemm_f64(oracle.dequant_staf_f32(4, 64, odd.n, odd.k, odd.staf_blocks()), x))
    w.destroy()


@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336), (1024, 4096)])
def test_in_place_gemv_llama_shapes(pkg, ctx, n, k):
    """Llama-3-8B projection shapes at q4 g64, all output types, against the oracle and against the
    per-code kernel on the same device buffers."""
    case = _case(3300 + n % 97, n, k, 4, 64)
    w, wq = _device_and_reference(pkg, ctx, case)
    for m in (1, 4):
        x = act_rounded(kat.seeded_activations(3310 + m, m, k), pkg.BF16, pkg)
        say(f"in-place llama N={n} K={k} M={m}")
        got = run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.F32)
        assert_within_tolerance(got, oracle.gemm_f64(wq, x), f"N={n} K={k} M={m}")
        ref = run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.F32, pkg.FLAG_FORCE_GENERIC)
        assert_within_tolerance(got, ref, "against the per-code kernel")
        gbf = run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.BF16)
        assert np.array_equal(oracle.bf16_from_f32(gbf), oracle.bf16_from_f32(got))
        gh = run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.F16)
        assert np.array_equal(gh.astype(np.float16), got.astype(np.float16))
    w.destroy()


def test_in_place_gemv_strided_rows(pkg, ctx):
    """Activation rows wider than K (x_row_stride > K): the padding is never read into the result."""
    n, k, stride = 200, 4096, 4096 + 64
    case = _case(3400, n, k, 4, 64)
    w = case.device_weight(ctx, pkg, pkg.LAYOUT_STAF_BLOCKS)
    wq = oracle.dequant_staf_f32(4, 64, n, k, case.staf_blocks())
    x = np.full((3, stride), 1.0e6, np.float32)
    x[:, :k] = act_rounded(kat.seeded_activations(3401, 3, k), pkg.BF16, pkg)
    got = run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.F32)
    assert_within_tolerance(got, oracle.gemm_f64(wq, x[:, :k]), "strided rows")
    w.destroy()


def _run_batched(pkg, ctx, ws, ns, x, y_dtype):
    from gpu_util import out_from_device
    m = x.shape[0]
    xd = ctx.upload(oracle.bf16_from_f32(x).reshape(x.shape))
    esz = 4 if y_dtype == pkg.F32 else 2
    yds = [ctx.alloc(m * n * esz) for n in ns]
    for yd in yds:
        ctx.fill(yd, 0x7FC00000 if y_dtype == pkg.F32 else 0x7FC07FC0)
    ctx.batched_qgemm(ws, xd, pkg.BF16, yds, y_dtype, m)
    ctx.synchronize()
    out = [out_from_device(yd, y_dtype, (m, n), pkg) for yd, n in zip(yds, ns)]
    xd.free()
    for yd in yds:
        yd.free()
    return out


@pytest.mark.parametrize("ns,k,bits,group", [((4096, 1024, 1024), 4096, 4, 64), ((14336, 14336), 4096, 4, 64),
                                             ((5, 1, 3), 256, 4, 64), ((130, 67), 4096 + 256, 4, 64),
                                             ((257, 63, 129), 1024, 8, 32), ((70, 200), 1024, 3, 64)])
def test_in_place_batched_projections(pkg, ctx, ns, k, bits, group):
    """q+k+v and gate+up left in STAF blocks as one launch each: wavefronts are dealt to the matrices whole, so
    segment boundaries fall inside workgroups; every output against the per-projection oracle."""
    cases = [_case(3500 + i + len(ns) * 10 + bits, n, k, bits, group) for i, n in enumerate(ns)]
    pairs = [_device_and_reference(pkg, ctx, c) for c in cases]
    ws, wqs = [p[0] for p in pairs], [p[1] for p in pairs]
    for m in (1, 3, 8):
        x = act_rounded(kat.seeded_activations(3600 + m, m, k), pkg.BF16, pkg)
        say(f"in-place batched {ns} K={k} q{bits}g{group} M={m}")
        got = _run_batched(pkg, ctx, ws, ns, x, pkg.F32)
        gbf = _run_batched(pkg, ctx, ws, ns, x, pkg.BF16)
        for i in range(len(ns)):
            assert_within_tolerance(got[i], oracle.gemm_f64(wqs[i], x), f"{ns} projection {i} M={m}")
            assert np.array_equal(oracle.bf16_from_f32(gbf[i]), oracle.bf16_from_f32(got[i]))
    for w in ws:
        w.destroy()


@pytest.mark.parametrize("n,k", [(65536, 2048), (1000, 4096), (37, 256)])
def test_in_place_output_head(pkg, ctx, n, k):
    """LM head over STAF blocks with the fused arg-max tail: fp32 logits within tolerance, the token is the
    lowest-index maximum of the device's own logits, twice in a row (the partial keys need no reset), with and
    without a logits buffer."""
    case = _case(3700 + n % 89, n, k, 4, 64)
    w, wq = _device_and_reference(pkg, ctx, case)
    x = act_rounded(kat.seeded_activations(3701, 1, k), pkg.BF16, pkg)
    want = oracle.gemm_f64(wq, x)[0]
    xd = ctx.upload(oracle.bf16_from_f32(x))
    logits = ctx.alloc(n * 4)
    tok = ctx.upload(np.array([-7], np.int32))
    for _ in range(2):
        ctx.fill(logits, 0x7FC00000)
        tok.upload(np.array([-7], np.int32))
        ctx.lmhead_argmax(w, xd, pkg.BF16, logits, tok)
        ctx.synchronize()
        got = logits.download(np.float32)
        assert_within_tolerance(got, want, "in-place head logits")
        token = int(tok.download(np.int32)[0])
        assert token == oracle.argmax_lowest(got)
    tok.upload(np.array([-7], np.int32))
    ctx.lmhead_argmax(w, xd, pkg.BF16, None, tok)
    ctx.synchronize()
    assert int(tok.download(np.int32)[0]) == token
    # ties: identical rows give identical logits; the lowest row wins
    dup = _case(3710, 512, 1024, 4, 64)
    dup.codes[17] = 15; dup.scales[17] = 0.02; dup.zeros[17] = 0.0
    dup.codes[300] = 15; dup.scales[300] = 0.02; dup.zeros[300] = 0.0
    wd = dup.device_weight(ctx, pkg, pkg.LAYOUT_STAF_BLOCKS)
    ones = ctx.upload(oracle.bf16_from_f32(np.ones((1, 1024), np.float32)))
    ctx.lmhead_argmax(wd, ones, pkg.BF16, None, tok)
    ctx.synchronize()
    assert int(tok.download(np.int32)[0]) == 17
    for b in (xd, logits, tok, ones):
        b.free()
    w.destroy(); wd.destroy()


def test_in_place_plan_replay_and_graph(pkg, ctx):
    """A plan over STAF-layout weights (one fused q+k+v-style launch and the fused head) replayed from C and as a
    HIP graph, with fills and uploads between the replays: every replay equals the eager launches bit for bit (the
    direct-to-LDS loads, the partial keys of the head and its finishing launch carry no state between launches)."""
    k = 1024
    ns = (512, 256, 2048)
    cases = [_case(3800 + i, n, k, 4, 64) for i, n in enumerate(ns)]
    ws = [c.device_weight(ctx, pkg, pkg.LAYOUT_STAF_BLOCKS) for c in cases]
    x = ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(3810, 1, k)))
    ys = [ctx.alloc(n * 4) for n in ns]
    tok = ctx.upload(np.array([-3], np.int32))
    ctx.batched_qgemm(ws[:2], x, pkg.BF16, ys[:2], pkg.F32, 1)
    ctx.lmhead_argmax(ws[2], x, pkg.BF16, ys[2], tok)
    ctx.synchronize()
    eager = [y.download(np.float32) for y in ys]
    etok = int(tok.download(np.int32)[0])
    assert etok == oracle.argmax_lowest(eager[2])
    plan = pkg.DispatchPlan(ctx)
    plan.add_batched_linear(ws[:2], x, pkg.BF16, ys[:2], pkg.F32, 1)
    plan.add_output_head(ws[2], x, pkg.BF16, ys[2], tok)
    assert plan.step(0)[0].device_kernel == "gemv_staf_q4_g64"
    stream = ctx.stream_create()
    plan.graph_build(stream)
    for rep in range(4):
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


def test_in_place_gemv_full_size_properties(pkg, ctx):
    """Size-independent properties at the full gate shape (14336 x 4096, q4 g64), where the oracle is too slow to
    be the checker for every element: scaling the activations by a power of two scales every output by the same
    factor bit for bit, and permuting the weight rows permutes the outputs bit for bit (a row's result does not
    depend on which wavefront, span slot or workgroup computes it)."""
    n, k = 14336, 4096
    case = _case(3900, n, k, 4, 64)
    small = _case(3899, 3, 256, 4, 64)
    assert np.array_equal(_q4_blocks(small).reshape(-1), small.staf_blocks())       # the fast builder below
    blocks = _q4_blocks(case)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    w = ctx.weight_prepare_staf(fmt, n, k, blocks.reshape(-1), pkg.LAYOUT_STAF_BLOCKS)
    x = act_rounded(kat.seeded_activations(3901, 1, k), pkg.BF16, pkg)
    y = run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.F32)
    assert np.all(np.isfinite(y))
    y4 = run_gemv(ctx, pkg, w, 4.0 * x, pkg.BF16, pkg.F32)
    assert np.array_equal(y4, 4.0 * y)
    perm = np.random.default_rng(3902).permutation(n)
    wp = ctx.weight_prepare_staf(fmt, n, k, np.ascontiguousarray(blocks[perm]).reshape(-1), pkg.LAYOUT_STAF_BLOCKS)
    yp = run_gemv(ctx, pkg, wp, x, pkg.BF16, pkg.F32)
    assert np.array_equal(yp[0], y[0][perm])
    # and a sample of rows against the oracle
    rows = np.random.default_rng(3903).choice(n, 64, replace=False)
    wq = oracle.dequant_staf_f32(4, 64, 64, k, np.ascontiguousarray(blocks[rows]).reshape(-1))
    assert_within_tolerance(y[0][rows], oracle.gemm_f64(wq, x)[0], "sampled rows")
    w.destroy(); wp.destroy()
