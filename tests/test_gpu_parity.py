"""GPU parity tests: every launch goes through the C ABI and is compared with the CPU oracle
(or with independent exact arithmetic) on identical inputs.

Bars: integer codes, dequantised bf16 bit patterns and argmax indices are bit-exact; floating
point outputs are within relative L2 <= 1e-3 and max-abs <= 2e-2 of an fp64 accumulation of
the same dequantised weights, compared on the fp32 output; the bf16 output must equal
bf16_rne(fp32 output) exactly.
"""
import numpy as np
import pytest

import kat
import oracle
from gpu_util import (Case, act_rounded, assert_within_tolerance, run_gemv, seeded_case)

pytestmark = pytest.mark.gpu
KATS = kat.load_kats()


def _layouts(pkg, case):
    out = [("staf", pkg.LAYOUT_STAF_BLOCKS, None)]
    if case.planes_eligible():
        out += [("planes_f16", pkg.LAYOUT_PLANES, pkg.F16)]
    return out


# ----------------------------------------------------------------------------- codes (a2)
@pytest.mark.parametrize("bits,group", kat.ALL_FORMATS)
def test_unpack_codes_bit_exact(pkg, ctx, bits, group):
    blocks_per_row = int(32 // np.gcd(32, group * bits)) * 5
    k = group * blocks_per_row
    n = 37
    codes = kat.random_codes(1000 + bits * 17 + group, n, k, bits)
    case = Case(bits, group, codes, np.ones((n, blocks_per_row)), np.zeros((n, blocks_per_row)))
    for name, layout, sb in _layouts(pkg, case):
        w = case.device_weight(ctx, pkg, layout, sb)
        out = ctx.alloc(n * k)
        ctx.unpack_codes(w, out)
        ctx.synchronize()
        got = out.download(np.uint8, (n, k))
        assert np.array_equal(got, codes), name
        assert np.array_equal(got, oracle.unpack_staf_codes(bits, group, n, k, case.staf_blocks()))
        out.free(); w.destroy()


# ------------------------------------------------------------------- dequant -> bf16 (a8)
@pytest.mark.parametrize("bits,group", kat.ALL_FORMATS)
def test_dequant_bf16_bit_exact(pkg, ctx, bits, group):
    blocks_per_row = int(32 // np.gcd(32, group * bits)) * 3
    k, n = group * blocks_per_row, 19
    codes = kat.random_codes(2000 + bits * 5 + group, n, k, bits)
    rng = np.random.default_rng(bits + group)
    scales = rng.integers(1, 400, size=(n, blocks_per_row)) / 4096.0      # exact in f16, not pow2
    zeros = rng.integers(-300, 300, size=(n, blocks_per_row)) / 2048.0
    case = Case(bits, group, codes, scales, zeros)
    want = oracle.dequant_staf_bf16(bits, group, n, k, case.staf_blocks())
    for name, layout, sb in _layouts(pkg, case):
        w = case.device_weight(ctx, pkg, layout, sb)
        out = ctx.alloc(n * k * 2)
        ctx.dequant_bf16(w, out)
        ctx.synchronize()
        assert np.array_equal(out.download(np.uint16, (n, k)), want), name
        out.free(); w.destroy()


# ------------------------------------------------------------------- dequant -> fp32 (a11)
@pytest.mark.parametrize("bits,group", kat.ALL_FORMATS)
def test_dequant_f32_bit_exact(pkg, ctx, bits, group):
    """CPUWeightStore.decodeQuantized (Sources/SwiftLM/CPUWeightStore.swift:109-174) on the device: every registered
    format, STAF blocks and planes, bit for bit against the oracle's restatement (scale * q rounded, then + zero)."""
    blocks_per_row = int(32 // np.gcd(32, group * bits)) * 3
    k, n = group * blocks_per_row, 23
    codes = kat.random_codes(2500 + bits * 5 + group, n, k, bits)
    rng = np.random.default_rng(100 + bits + group)
    scales = rng.integers(1, 400, size=(n, blocks_per_row)) / 4096.0      # exact in f16 and bf16, not powers of two
    zeros = rng.integers(-127, 127, size=(n, blocks_per_row)) / 1024.0
    case = Case(bits, group, codes, scales, zeros)
    want = oracle.dequant_staf_f32(bits, group, n, k, case.staf_blocks())
    for name, layout, sb in _layouts(pkg, case):
        w = case.device_weight(ctx, pkg, layout, sb)
        out = ctx.alloc(n * k * 4)
        ctx.fill(out, 0x7FC00000)
        ctx.dequant_f32(w, out)
        ctx.synchronize()
        assert np.array_equal(out.download(np.float32, (n, k)).view(np.uint32), want.view(np.uint32)), name
        out.free(); w.destroy()


def test_dequant_f32_reference_vector_and_seeded_tensor(pkg, ctx):
    """The reference's own CPUWeightStore vector (Tests/SwiftLMTests/Core/TextEmbeddingRuntimeTests.swift:421-476:
    scale 1, zero 0, byte i = (2i mod 16) | ((2i+1 mod 16) << 4) -> 0, 1, ..., 15, 0, ...), and a benchmark-style
    tensor on all three layouts at a shape the eight-codes-per-thread kernel and the per-code kernel both see."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    qs = np.array([((2 * i) % 16) | (((2 * i + 1) % 16) << 4) for i in range(32)], np.uint8)
    block = np.concatenate([np.array([0x00, 0x3C, 0x00, 0x00], np.uint8), qs])
    w = ctx.weight_prepare_staf(fmt, 1, 64, block, pkg.LAYOUT_STAF_BLOCKS)
    out = ctx.alloc(64 * 4)
    ctx.dequant_f32(w, out); ctx.synchronize()
    assert out.download(np.float32, (64,)).tolist() == [float(i % 16) for i in range(64)]
    out.free(); w.destroy()
    n, k = 48, 512
    words, s, z, wq = seeded_case(77, n, k, 4, 64)
    for layout in (pkg.LAYOUT_PLANES, pkg.LAYOUT_TILE16, pkg.LAYOUT_STAF_BLOCKS):
        w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, layout)
        out = ctx.alloc(n * k * 4 + 16)
        for off in (0, 4):                                   # 16-byte aligned output, and one that is not
            ctx.fill(out, 0x7FC00000)
            ctx.dequant_f32(w, out.ptr + off); ctx.synchronize()
            got = np.frombuffer(out.download(np.uint8)[off:off + n * k * 4].tobytes(), np.float32).reshape(n, k)
            assert np.array_equal(got.view(np.uint32), wq.view(np.uint32)), (layout, off)
        out.free(); w.destroy()


def test_bf16_scales_outside_the_f16_range_decode_alike_on_every_layout(pkg, ctx):
    """MLX planes with bf16 scales and biases below the f16 normal range (6.1e-5), on the f16 subnormal grid, below
    it, and above 65504: the converter narrows them to f16 (STAFConverter.swift:326-368), so all three device layouts
    must decode to what the oracle decodes from the converter's blocks, bit for bit, and a GEMV must agree too."""
    bits, group, n, k = 4, 64, 32, 512
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
    words = kat.mlx_planes(kat.random_codes(991, n, k, bits), bits)
    rng = np.random.default_rng(992)
    shape = (n, k // group)
    mag = np.array([3.1e-5, 5.9e-5, 1.3e-6, 7.7e-8, 2.0e-8, 2.9e-8, 6.2e-5, 1.0e-3, 0.02])
    s32 = (rng.choice(mag, shape) * rng.uniform(0.8, 1.2, shape)).astype(np.float32)
    # biases also leave the range at the top (infinite after narrowing); scales stay finite so that no code 0 meets
    # an infinite scale (whose NaN the host and the device may spell differently)
    z32 = (rng.choice(np.concatenate([mag, [70000.0, 65504.0, 65519.0]]), shape) * rng.choice([-1.0, 1.0], shape))
    s, z = oracle.bf16_from_f32(s32).reshape(shape), oracle.bf16_from_f32(z32.astype(np.float32)).reshape(shape)
    with np.errstate(over="ignore"):
        s16 = oracle.bf16_to_f32(s).astype(np.float16)           # numpy's cast is round to nearest even
        z16 = oracle.bf16_to_f32(z).astype(np.float16)
    assert np.any(s16 == 0) and np.any(np.isinf(z16)) and np.any((s16 != 0) & (np.abs(s16) < 6.1e-5))
    blocks = oracle.repack_mlx_to_staf(bits, group, words, s, z, oracle.BF16)
    hdr = blocks.reshape(n * (k // group), -1)[:, :4].copy().view(np.uint16)
    assert np.array_equal(hdr[:, 0], s16.view(np.uint16).ravel())  # the oracle narrows like numpy does
    assert np.array_equal(hdr[:, 1], z16.view(np.uint16).ravel())
    want = oracle.dequant_staf_f32(bits, group, n, k, blocks)
    x = kat.seeded_activations(993, 1, k)
    ys = []
    for layout in (pkg.LAYOUT_STAF_BLOCKS, pkg.LAYOUT_PLANES, pkg.LAYOUT_TILE16):
        w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, layout)
        out = ctx.alloc(n * k * 4)
        ctx.dequant_f32(w, out); ctx.synchronize()
        got = out.download(np.float32, (n, k))
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), layout
        ys.append(run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.F32, 0))
        out.free(); w.destroy()
    finite = np.isfinite(ys[0])
    assert np.array_equal(finite, np.isfinite(ys[1])) and np.array_equal(finite, np.isfinite(ys[2]))
    scale = np.maximum(1e-30, np.abs(ys[0][finite]))
    for y in ys[1:]:
        assert np.max(np.abs(y[finite] - ys[0][finite]) / scale) < 1e-3


# ------------------------------------------------------------- closed-form GEMV KATs (a4)
def _check_kat(pkg, ctx, case, x, tol=2e-6):
    want = kat.exact_gemv(case.codes, case.scales, case.zeros, x, case.group)
    scale = max(1.0, float(np.max(np.abs(want))))
    for name, layout, sb in _layouts(pkg, case):
        w = case.device_weight(ctx, pkg, layout, sb)
        for x_dtype in (pkg.F16, pkg.BF16, pkg.F32):
            if not np.array_equal(act_rounded(x, x_dtype, pkg), x):
                continue                                    # inputs must be exact in the I/O dtype
            for flags in (0, pkg.FLAG_FORCE_GENERIC):
                got = run_gemv(ctx, pkg, w, x, x_dtype, pkg.F32, flags)
                assert np.max(np.abs(got - want)) <= tol * scale * case.k, (name, x_dtype, flags)
        w.destroy()


@pytest.mark.parametrize("c", KATS["single_block"]["cases"], ids=lambda c: f"q{c['bits']}g{c['group']}")
def test_single_block_gemv_kat(pkg, ctx, c):
    codes, s, z, x = kat.single_block_case(c["bits"], c["group"], *c["gemv"])
    _check_kat(pkg, ctx, Case(c["bits"], c["group"], codes, s, z), x)


@pytest.mark.parametrize("bits,group", kat.REFERENCE_FORMATS)
def test_multi_block_and_multi_row_gemv_kat(pkg, ctx, bits, group):
    for codes, s, z, x in (kat.multi_block_case(bits, group), kat.multi_row_case(bits, group)):
        # the reference's f16 inputs are not all exact in bf16; f16/f32 runs cover them
        _check_kat(pkg, ctx, Case(bits, group, codes, s, z), x)


def test_literal_q4_gemv_vector(pkg, ctx):
    v = KATS["literal_q4_gemv"]
    codes = np.array([[int(r["word"][2], 16)] * 64 for r in v["rows"]], np.uint8)
    case = Case(4, 64, codes, [[r["scale"]] for r in v["rows"]], [[r["zero"]] for r in v["rows"]])
    x = np.ones((1, 64), np.float32)
    for name, layout, sb in _layouts(pkg, case):
        w = case.device_weight(ctx, pkg, layout, sb)
        for flags in (0, pkg.FLAG_FORCE_GENERIC):
            for yd in (pkg.F32, pkg.BF16, pkg.F16):
                got = run_gemv(ctx, pkg, w, x, pkg.BF16, yd, flags)
                assert got[0].tolist() == [r["y"] for r in v["rows"]], (name, flags, yd)
        w.destroy()


def test_q4_gemm_with_padded_input_stride(pkg, ctx):
    v = KATS["q4_gemm_padded_stride"]
    k, n, m, stride = v["k"], v["n"], v["m"], v["stride"]
    x = np.full((m, stride), v["poison"], np.float32)
    for mi in range(m):
        for c in range(k):
            x[mi, c] = (mi + 3) * ((c % 7) - 3) * 0.125
    case = Case(4, 64, [[r + 1] * k for r in range(n)], np.full((n, 1), v["scale"]), np.full((n, 1), v["zero"]))
    want = np.array([[0.25 * (r + 1) * x[mi, :k].astype(np.float64).sum() for r in range(n)] for mi in range(m)])
    for name, layout, sb in _layouts(pkg, case):
        w = case.device_weight(ctx, pkg, layout, sb)
        for x_dtype in (pkg.F32, pkg.BF16):
            for flags in (0, pkg.FLAG_FORCE_GENERIC):
                for use_qgemm in (False, True):
                    got = run_gemv(ctx, pkg, w, x, x_dtype, pkg.F32, flags, use_qgemm=use_qgemm)
                    assert np.max(np.abs(got - want)) < 1e-3, (name, x_dtype, flags)   # the reference's bar
        w.destroy()


# ---------------------------------------------------------- seeded benchmark configurations
def _seeded_gemv_check(pkg, ctx, seed, n, k, bits, group, ms, layouts=("planes",), check_codes=False):
    words, s, z, wq = seeded_case(seed, n, k, bits, group)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
    results = {}
    for layout_name in layouts:
        layout = pkg.LAYOUT_PLANES if layout_name == "planes" else pkg.LAYOUT_STAF_BLOCKS
        w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, layout)
        assert w.info.weight_bytes == n * (k // group) * (4 + group * bits // 8)
        if check_codes:
            out = ctx.alloc(n * k)
            ctx.unpack_codes(w, out)
            ctx.synchronize()
            assert np.array_equal(out.download(np.uint8, (n, k)), oracle.unpack_plane_codes(bits, n, k, words))
            out.free()
        for m in ms:
            x = act_rounded(kat.seeded_activations(seed + m, m, k), pkg.BF16, pkg)
            want = oracle.gemm_f64(wq, x)
            y32 = run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.F32)
            results[(layout_name, m)] = assert_within_tolerance(y32, want, f"{layout_name} M={m} {k}->{n}")
            ybf = run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.BF16)
            assert np.array_equal(oracle.bf16_from_f32(ybf), oracle.bf16_from_f32(y32)), "bf16 out != rne(fp32 out)"
        w.destroy()
    return results


def test_config0_q4g64_2048_to_8192(pkg, ctx):
    """benchmark config 0, both layouts (bf16 scale planes and f16 STAF headers dequantise identically)."""
    r = _seeded_gemv_check(pkg, ctx, 100, 8192, 2048, 4, 64, [1], layouts=("planes", "staf"), check_codes=True)
    assert max(v[0] for v in r.values()) < 1e-4


LLAMA_SHAPES = {"q_o": (4096, 4096), "k_v": (1024, 4096), "gate_up": (14336, 4096), "down": (4096, 14336)}


@pytest.mark.parametrize("name", list(LLAMA_SHAPES))
def test_config1_llama3_8b_layer_shapes(pkg, ctx, name):
    n, k = LLAMA_SHAPES[name]
    _seeded_gemv_check(pkg, ctx, 200 + n % 97, n, k, 4, 64, [1, 2, 4, 8])


@pytest.mark.parametrize("n,k,group", [(14336, 4096, 64), (4100, 4096, 128), (517, 14336, 64), (16387, 2048, 64), (3000, 2560, 64)])
def test_activation_rows_share_the_unpacked_codes(pkg, ctx, n, k, group):
    """M = 2 on 4-bit planes (and M = 3, 4 on small matrices with rows of two K-steps) runs on the static-structure
    kernel with every activation row on each unpacked code pair: rows of one, two and seven K-steps, row counts off
    every workgroup boundary, both group sizes; against the oracle and against the same rows taken one at a time."""
    words, s, z, wq = seeded_case(270 + n % 89, n, k, 4, group)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, group)
    w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
    small = 2048 < k <= 4096 and n * (k // group) * (4 + group // 2) < (12 << 20)
    for m in ((2, 3, 4) if small else (2,)):
        step = w.plan_decode_step(m)
        if n >= 3000:
            assert step.device_kernel == f"gemv_rows_q4_g{group}", (m, step.device_kernel)
        x = act_rounded(kat.seeded_activations(271 + m, m, k), pkg.BF16, pkg)
        want = oracle.gemm_f64(wq, x)
        y32 = run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.F32)
        assert_within_tolerance(y32, want, f"M={m} {k}->{n}")
        one = np.concatenate([run_gemv(ctx, pkg, w, x[i:i + 1], pkg.BF16, pkg.F32) for i in range(m)])
        assert np.max(np.abs(one - y32)) <= 1e-5 * max(1.0, float(np.max(np.abs(y32)))), "rows together vs one at a time"
        for yd in (pkg.BF16, pkg.F16):
            y16 = run_gemv(ctx, pkg, w, x, pkg.BF16, yd)
            want16 = (oracle.bf16_to_f32(oracle.bf16_from_f32(y32)).reshape(y32.shape) if yd == pkg.BF16
                      else y32.astype(np.float16).astype(np.float32))
            assert np.array_equal(y16, want16)
    w.destroy()


def test_config1_odd_batch_sizes(pkg, ctx):
    _seeded_gemv_check(pkg, ctx, 260, 1024, 4096, 4, 64, [3, 5, 6, 7])


@pytest.mark.parametrize("bits,group", [(8, 32), (6, 64), (3, 64), (2, 64)])
def test_config2_bit_width_sweep(pkg, ctx, bits, group):
    """gate/up shape 4096->14336, M=1; unpacked codes must match the CPU unpacker bit-exactly."""
    _seeded_gemv_check(pkg, ctx, 300 + bits, 14336, 4096, bits, group, [1], check_codes=True)


@pytest.mark.parametrize("bits,group", [(2, 16), (2, 32), (3, 16), (3, 32), (4, 128), (5, 32), (5, 64), (6, 16),
                                        (6, 32), (8, 64), (8, 128)])
def test_other_registered_formats_seeded(pkg, ctx, bits, group):
    _seeded_gemv_check(pkg, ctx, 400 + bits * 3 + group, 512, 2048, bits, group, [1, 4],
                       layouts=("planes", "staf"), check_codes=True)


def test_ragged_shapes(pkg, ctx):
    """N not a multiple of the row tile, K not a multiple of the wavefront K-step, tiny N."""
    for n, k in [(1, 64), (3, 192), (5, 2048 + 64), (130, 4096 + 2048 + 128), (4099, 320)]:
        _seeded_gemv_check(pkg, ctx, 500 + n, n, k, 4, 64, [1, 3], layouts=("planes", "staf"))
    _seeded_gemv_check(pkg, ctx, 520, 67, 1024 + 512, 8, 32, [1, 2], layouts=("planes", "staf"))
    _seeded_gemv_check(pkg, ctx, 521, 67, 2048 + 256, 3, 64, [1, 2], layouts=("planes", "staf"))


def test_q3_rows_every_code_position_and_row_length(pkg, ctx):
    """3-bit codes on the planes are used where they lie in their words (pairs of fields picked with one mask, the
    activations staged pre-scaled by powers of two).  One-hot activations single out every code position of a lane
    chunk of 32 codes (and of a chunk further along the row, with a negative and a non-unit activation): each output
    is s q x + z x exactly.  Then every row length the kernel is built for (1, 2, 3, 4 and 7 K-steps of 2048 codes)
    against the oracle."""
    rng = np.random.default_rng(530)
    n, k = 70, 4096
    codes = rng.integers(0, 8, (n, k), dtype=np.uint8)
    scales = rng.choice([0.25, 0.5, 1.0], (n, k // 64)); zeros = rng.integers(-4, 5, (n, k // 64)) * 0.5
    case = Case(3, 64, codes, scales, zeros)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(3, 64)
    w = ctx.weight_prepare_mlx(fmt, *case.planes(pkg.BF16, pkg), pkg.BF16, pkg.LAYOUT_PLANES)
    assert w.plan_decode_step(1).device_kernel == "gemv_rows_q3_g64"
    for base, val in ((0, 1.0), (2048 + 37 * 32, -1.0), (4096 - 32, 0.375)):
        for j in range(32):
            x = np.zeros((1, k), np.float32); x[0, base + j] = val
            got = run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.F32)[0]
            g = (base + j) // 64
            want = (scales[:, g] * codes[:, base + j] + zeros[:, g]) * val
            assert np.array_equal(got.astype(np.float64), want), (base, j)
    w.destroy()
    for i, k in enumerate((2048, 4096, 6144, 8192, 14336, 4096 + 64, 2048 - 64)):
        _seeded_gemv_check(pkg, ctx, 531 + i, 300, k, 3, 64, [1], layouts=("planes",))


def test_linearity_and_scaling_at_full_size(pkg, ctx):
    """Size-independent properties at the full gate/up shape: y(2x) == 2*y(x) bit for bit
    (a power-of-two scale commutes with every rounding), and row i of the output only depends on
    row i of the weights (a permuted copy gives the permuted output)."""
    n, k = 14336, 4096
    words, s, z, _ = seeded_case(600, n, k, 4, 64)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
    x = act_rounded(kat.seeded_activations(601, 1, k), pkg.BF16, pkg)
    y1 = run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.F32)
    y2 = run_gemv(ctx, pkg, w, 2.0 * x, pkg.BF16, pkg.F32)
    assert np.array_equal(y2, 2.0 * y1)
    perm = np.random.default_rng(602).permutation(n)
    wp = ctx.weight_prepare_mlx(fmt, words[perm], s[perm], z[perm], pkg.BF16, pkg.LAYOUT_PLANES)
    yp = run_gemv(ctx, pkg, wp, x, pkg.BF16, pkg.F32)
    assert np.array_equal(yp[0], y1[0][perm])
    w.destroy(); wp.destroy()


# -------------------------------------------------------------------------- argmax (a10)
def _argmax_dev(pkg, ctx, v, dtype):
    from gpu_util import act_to_device_array
    d = ctx.upload(act_to_device_array(v, dtype, pkg))
    t = ctx.upload(np.array([-7], np.int32))
    ctx.argmax(d, dtype, v.size, t)
    ctx.synchronize()
    tok = int(t.download(np.int32)[0])
    d.free(); t.free()
    return tok


def test_argmax_ties_nan_and_boundaries(pkg, ctx):
    rng = np.random.default_rng(9)
    specials = [np.full(9, np.nan, np.float32), np.array([np.nan, 1.0, np.nan, 1.0], np.float32),
                np.array([-0.0, 0.0, -0.0], np.float32), np.array([0.0, -0.0], np.float32),
                np.full(5, -np.inf, np.float32), np.array([-np.inf, np.inf, np.inf], np.float32),
                np.array([np.nan, -np.inf, -np.inf], np.float32), np.zeros(70000, np.float32)]
    for v in specials:
        assert _argmax_dev(pkg, ctx, v, pkg.F32) == oracle.argmax_lowest(v)
    # vocabulary-sized vectors take the two-launch form: the same rules must hold across its workgroups
    big = 40000
    for v in (np.full(big, np.nan, np.float32), np.full(big, -np.inf, np.float32),
              np.where(np.arange(big) % 2 == 0, -0.0, 0.0).astype(np.float32),
              np.concatenate([np.full(big - 1, -np.inf, np.float32), [-3.0e38]]).astype(np.float32),
              np.concatenate([np.full(big - 2, np.nan, np.float32), [np.inf, np.inf]]).astype(np.float32)):
        assert _argmax_dev(pkg, ctx, v, pkg.F32) == oracle.argmax_lowest(v)
    for n in (1, 2, 63, 64, 65, 1023, 1024, 1025, 2049, 16383, 16384, 16385, 65536, 70001, 262144):
        for _ in range(3):
            v = rng.integers(-3, 4, size=n).astype(np.float32)         # dense ties
            for dtype in (pkg.F32, pkg.BF16, pkg.F16):
                assert _argmax_dev(pkg, ctx, v, dtype) == int(np.argmax(v)) == oracle.argmax_lowest(v)
        # one maximum duplicated across a lane / wavefront / workgroup-stride boundary
        for a, b in [(0, n - 1), (n // 2, n - 1), (63 % n, 64 % n), (1023 % n, 1024 % n), (255 % n, 256 % n),
                     (65535 % n, 65536 % n)]:
            v = rng.standard_normal(n).astype(np.float32)
            v[a] = v[b] = 100.0
            assert _argmax_dev(pkg, ctx, v, pkg.F32) == min(a, b)


def test_config4_lm_head_fused_argmax(pkg, ctx):
    """2048 -> 65536, 4-bit g64: fp32 logits within tolerance; token == lowest-index argmax of the
    device's own logits and of the CPU reference logits (seed checked for a safe top-2 gap)."""
    n, k = 65536, 2048
    words, s, z, wq = seeded_case(700, n, k, 4, 64)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
    x = act_rounded(kat.seeded_activations(701, 1, k), pkg.BF16, pkg)
    want = oracle.gemm_f64(wq, x)[0]
    xd = ctx.upload(oracle.bf16_from_f32(x))
    logits = ctx.alloc(n * 4)
    tok = ctx.upload(np.array([-7], np.int32))
    for flags in (0, pkg.FLAG_FORCE_GENERIC):
        ctx.fill(logits, 0x7FC00000)
        for _ in range(2):                                   # the scratch cells must self-reset
            tok.upload(np.array([-7], np.int32))
            ctx.lmhead_argmax(w, xd, pkg.BF16, logits, tok, flags)
            ctx.synchronize()
            got = logits.download(np.float32)
            assert_within_tolerance(got, want, "lm head logits")
            token = int(tok.download(np.int32)[0])
            assert token == oracle.argmax_lowest(got)
            top2 = np.sort(want)[-2:]
            assert top2[1] - top2[0] > 1e-3, "seed gives a near-tie; pick another"
            assert token == int(np.argmax(want)) == oracle.argmax_lowest(want.astype(np.float32))
    # logits pointer is optional on the fused path
    tok.upload(np.array([-7], np.int32))
    ctx.lmhead_argmax(w, xd, pkg.BF16, None, tok)
    ctx.synchronize()
    assert int(tok.download(np.int32)[0]) == int(np.argmax(want))
    w.destroy(); xd.free(); logits.free(); tok.free()


def test_lm_head_ties_break_to_lowest_index(pkg, ctx):
    """Duplicate weight rows give bit-identical logits; the fused kernel must return the lowest row."""
    n, k = 4096 + 40, 2048
    words, s, z, wq = seeded_case(710, n, k, 4, 64)
    x = act_rounded(kat.seeded_activations(711, 1, k), pkg.BF16, pkg)
    best = int(np.argmax(oracle.gemm_f64(wq, x)[0]))
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    xd = ctx.upload(oracle.bf16_from_f32(x))
    tok = ctx.upload(np.array([-7], np.int32))
    logits = ctx.alloc(n * 4)
    for dups in ([5, 4099], [4135, 63, 64], [n - 1, 1000], [0, n - 1]):
        w2, s2, z2 = words.copy(), s.copy(), z.copy()
        for d in dups:
            w2[d], s2[d], z2[d] = words[best], s[best], z[best]
        w = ctx.weight_prepare_mlx(fmt, w2, s2, z2, pkg.BF16, pkg.LAYOUT_PLANES)
        for flags in (0, pkg.FLAG_FORCE_GENERIC):
            ctx.lmhead_argmax(w, xd, pkg.BF16, logits, tok, flags)
            ctx.synchronize()
            assert int(tok.download(np.int32)[0]) == min(dups + [best]), (dups, flags)
        w.destroy()
    xd.free(); tok.free(); logits.free()


# ------------------------------------------------------------- zero-copy wrap (boundary b)
def test_wrap_device_buffers_at_offsets(pkg, ctx):
    """One device allocation holding several tensors, addressed as (buffer, offset) like the
    reference's single mapped weight buffer."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    shapes = [(96, 256), (40, 512), (8, 64)]
    payloads, cases, offs, off = [], [], [], 0
    for i, (n, k) in enumerate(shapes):
        words, s, z, wq = seeded_case(800 + i, n, k, 4, 64)
        blocks = pkg.repack_mlx_to_staf(fmt, words, s, z, pkg.BF16)
        off = (off + 255) // 256 * 256                       # the container's 256-byte tensor alignment
        offs.append(off); payloads.append(blocks); cases.append(wq)
        off += blocks.size
    host = np.zeros(off, np.uint8)
    for o, p in zip(offs, payloads):
        host[o:o + p.size] = p
    big = ctx.upload(host)
    for (n, k), o, wq in zip(shapes, offs, cases):
        w = ctx.weight_wrap_staf(fmt, n, k, big, byte_offset=o)
        assert not w.info.owns_memory and w.info.blocks_dev == big.ptr + o
        x = act_rounded(kat.seeded_activations(n, 2, k), pkg.BF16, pkg)
        assert_within_tolerance(run_gemv(ctx, pkg, w, x, pkg.BF16, pkg.F32), oracle.gemm_f64(wq, x), "wrapped")
        w.destroy()
    with pytest.raises(pkg.MI355QError) as e:
        ctx.weight_wrap_staf(fmt, 96, 256, big, payload_bytes=100)
    assert e.value.status_name == "SIZE_MISMATCH"
    big.free()


# ------------------------------------------------------------------ error paths on device
def test_launch_argument_errors(pkg, ctx):
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    words, s, z, _ = seeded_case(900, 8, 128, 4, 64)
    w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
    x = ctx.alloc(4096); y = ctx.alloc(4096)

    def status(fn, *a, **kw):
        with pytest.raises(pkg.MI355QError) as e:
            fn(*a, **kw)
        return e.value.status_name

    assert status(ctx.qgemv, w, x, pkg.BF16, y, pkg.F32, 0) == "INVALID_ARGUMENT"          # M = 0
    assert status(ctx.qgemv, w, x, pkg.BF16, y, pkg.F32, 9) == "INVALID_ARGUMENT"          # M > 8
    assert status(ctx.qgemv, w, x, pkg.BF16, y, pkg.F32, 1, 64) == "SHAPE"                 # stride < K
    assert status(ctx.qgemv, w, x, pkg.BF16, y, pkg.F32, 1, 0, 4) == "SHAPE"               # y stride < N
    assert status(ctx.qgemv, w, None, pkg.BF16, y, pkg.F32, 1) == "INVALID_ARGUMENT"
    assert status(ctx.qgemv, w, x, 7, y, pkg.F32, 1) == "INVALID_ARGUMENT"
    assert status(ctx.qgemm, w, x, pkg.BF16, y, pkg.F32, 16, 0, 0, pkg.FLAG_FORCE_MFMA | pkg.FLAG_FORCE_GENERIC) \
        == "INVALID_ARGUMENT"
    assert status(ctx.batched_qgemm, [w], x, pkg.BF16, [y], pkg.F32, 1) == "KERNEL_NOT_FOUND"   # count 1
    assert status(ctx.argmax, x, pkg.F32, 0, y) == "SHAPE"                                 # empty vector
    assert status(ctx.weight_prepare_mlx, fmt, np.zeros((2, 4), np.uint32), np.zeros((2, 1), np.uint16),
                  np.zeros((2, 1), np.uint16), pkg.BF16) == "SHAPE"                          # K=32 < group
    assert status(ctx.weight_prepare_staf, fmt, 2, 64, np.zeros(71, np.uint8)) == "SIZE_MISMATCH"
    assert status(ctx.lmhead_argmax, w, x, pkg.BF16, None, None) == "INVALID_ARGUMENT"
    w.destroy(); x.free(); y.free()


# ------------------------------------------------------------------------ planner (a5, a9)
def test_decode_and_prefill_plan_records(pkg, ctx):
    """T/QuantizationPlanningTests.swift: which kernel family / fallback reason is recorded."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    words, s, z, _ = seeded_case(950, 8192, 2048, 4, 64)
    w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES)
    st = w.plan_decode_step(1)
    assert st.kernel_name == "gemv_q4_g64" and st.kernel_family == "q4G64GEMV"
    assert st.path == "decodeProjection" and not st.used_fallback and st.fallback_reason is None
    assert st.shape_family == "input20488192Dense" and st.reference_simdgroups == 8
    assert (st.input_dimension, st.output_dimension) == (2048, 8192)
    assert st.weight_bytes == 9_437_184 and st.flops == 2 * 2048 * 8192
    assert st.device_kernel in ("gemv_rows_q4_g64", "gemv_planes_q4_g64") and st.block[0] in (256, 512) and st.grid[0] >= 1
    forced = w.plan_decode_step(1, flags=pkg.FLAG_FORCE_GENERIC)
    assert forced.used_fallback and forced.fallback_reason == "disabledByEnvironment"
    assert forced.device_kernel == "gemv_generic" and forced.grid[:2] == (2048, 1)
    last = w.plan_prefill_steps(16, is_last_token=True)
    assert len(last) == 1 and last[0].kernel_name == "gemv_q4_g64"
    assert last[0].fallback_reason == "lastTokenProjectionUsesDecodeKernel" and last[0].sequence_length == 1
    pre = w.plan_prefill_steps(512)
    assert pre[0].path == "prefillProjection" and pre[0].sequence_length == 512
    assert pre[0].flops == 2 * 512 * 2048 * 8192
    ws = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_STAF_BLOCKS)
    st2 = ws.plan_decode_step(1)
    assert st2.layout == pkg.LAYOUT_STAF_BLOCKS and st2.kernel_name == "gemv_q4_g64"
    w.destroy(); ws.destroy()


# ------------------------------------------------------- dispatch plan replay (boundary b)
def test_plan_replay_matches_direct_launches(pkg, ctx):
    """A plan built once (projections of two layers + the output head) replayed from C and as a
    HIP graph must reproduce the eager launches bit for bit, on every replay."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    shapes = [(512, 1024), (256, 1024), (1024, 512), (2048, 1024)]          # last one: the head
    ws, xs, ys, eager = [], [], [], []
    for i, (n, k) in enumerate(shapes):
        words, s, z, _ = seeded_case(1100 + i, n, k, 4, 64)
        ws.append(ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, pkg.LAYOUT_PLANES))
        xs.append(ctx.upload(oracle.bf16_from_f32(kat.seeded_activations(1200 + i, 1, k))))
        ys.append(ctx.alloc(n * 4))
    token = ctx.upload(np.array([-9], np.int32))
    for i in range(3):
        ctx.qgemv(ws[i], xs[i], pkg.BF16, ys[i], pkg.F32, 1)
    ctx.lmhead_argmax(ws[3], xs[3], pkg.BF16, ys[3], token)
    ctx.synchronize()
    eager = [y.download(np.float32) for y in ys]
    eager_token = int(token.download(np.int32)[0])
    assert eager_token == oracle.argmax_lowest(eager[3])

    plan = pkg.DispatchPlan(ctx)
    for i in range(3):
        plan.add_linear(ws[i], xs[i], pkg.BF16, ys[i], pkg.F32, 1, layer_index=i // 2, tensor_name=f"t{i}.weight")
    plan.add_output_head(ws[3], xs[3], pkg.BF16, ys[3], token, tensor_name="lm_head.weight")
    assert len(plan) == 4
    st, layer, name = plan.step(1)
    assert (st.kernel_name, layer, name) == ("gemv_q4_g64", 0, "t1.weight")
    assert st.path == "decodeProjection" and st.output_dimension == 256
    head, _, hname = plan.step(3)
    assert head.fallback_reason == "lastTokenProjectionUsesDecodeKernel" and hname == "lm_head.weight"

    stream = ctx.stream_create()

    def check(label):
        ctx.synchronize(stream)
        for y, want in zip(ys, eager):
            assert np.array_equal(y.download(np.float32), want), label
        assert int(token.download(np.int32)[0]) == eager_token, label

    def scrub():
        for y in ys:
            ctx.fill(y, 0x7FC00000, stream)
        token.upload(np.array([-9], np.int32))

    for rep in range(3):
        scrub()
        plan.encode(stream)
        check(f"stream replay {rep}")
    scrub()
    plan.encode(stream, 1, 2)                                     # a sub-range only touches its outputs
    ctx.synchronize(stream)
    assert np.all(np.isnan(ys[0].download(np.float32))) and np.array_equal(ys[1].download(np.float32), eager[1])
    plan.graph_build(stream)
    for rep in range(4):                                          # graph replays interleaved with eager work
        scrub()
        plan.graph_launch(stream)
        check(f"graph replay {rep}")
        ctx.qgemv(ws[0], xs[0], pkg.BF16, ys[0], pkg.F32, 1, stream=stream)
        ctx.synchronize(stream)
    with pytest.raises(pkg.MI355QError):                          # a built graph freezes the plan
        plan.add_linear(ws[0], xs[0], pkg.BF16, ys[0], pkg.F32, 1)
    plan.destroy()
    for o in ws:
        o.destroy()
    for b in xs + ys + [token]:
        b.free()


def test_buffer_copy_kernel(pkg, ctx):
    src = np.random.default_rng(3).integers(0, 2**32, size=1 << 18, dtype=np.uint32)
    a = ctx.upload(src); b = ctx.alloc(src.nbytes)
    ctx.copy(b, a, src.nbytes)
    ctx.synchronize()
    assert np.array_equal(b.download(np.uint32), src)
    with pytest.raises(pkg.MI355QError):
        ctx.copy(b.ptr + 4, a, 64)
    a.free(); b.free()
