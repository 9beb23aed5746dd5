"""GPU parity tests of the quantized embedding gather through the C ABI
(embedding_lookup[_seq]_q{b}_g{g}, MetalSourceGenerator+Embedding.swift:79-153, 229-322).

Bar: the fp32 output is bit-exact against the CPU oracle (dequantisation is two separate roundings on
both sides); bf16 / f16 outputs equal the rounding of the fp32 output; the reference's own vectors hold.
"""
import numpy as np
import pytest

import kat
import oracle
from gpu_util import Case, out_from_device

pytestmark = pytest.mark.gpu
KATS = kat.load_kats()


def _lookup(ctx, pkg, w, ids, dim, out_dtype, scale=None, stride=0):
    ids = np.asarray(ids, np.int32)
    td = ctx.upload(ids)
    s = stride or dim
    od = ctx.alloc(ids.size * s * (4 if out_dtype == pkg.F32 else 2))
    ctx.fill(od, 0x7FC00000 if out_dtype == pkg.F32 else 0x7FC07FC0)
    ctx.embedding_lookup(w, td, ids.size, od, out_dtype, stride, scale)
    ctx.synchronize()
    y = out_from_device(od, out_dtype, (ids.size, s), pkg)
    td.free(); od.free()
    return y


def test_reference_embedding_vectors(pkg, ctx):
    v = KATS["embedding_q4_row_of_twos"]
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    case = Case(4, 64, [[t] * v["dim"] for t in v["row_values"]], np.ones((2, 1)), np.zeros((2, 1)))
    w = ctx.weight_prepare_staf(fmt, 2, v["dim"], case.staf_blocks(), pkg.LAYOUT_STAF_BLOCKS)
    assert np.all(_lookup(ctx, pkg, w, [v["token"]], v["dim"], pkg.F32) == v["expected"])
    assert np.all(_lookup(ctx, pkg, w, [v["token"]], v["dim"], pkg.F32, v["scale"]) == v["expected_scaled"])
    w.destroy()
    v = KATS["embedding_q3_sequence"]
    dim, rows = v["dim"], v["rows"]
    codes = np.array([[(i + 3 * g + 5 * t) % 8 for g in range(dim // 64) for i in range(64)] for t in range(rows)], np.uint8)
    s = np.array([[0.03125 * (g + 1) + 0.0078125 * t for g in range(dim // 64)] for t in range(rows)])
    z = np.array([[-0.125 + 0.0625 * t - 0.015625 * g for g in range(dim // 64)] for t in range(rows)])
    blocks = kat.staf_blocks(codes, s, z, 3, 64)
    fmt3 = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(3, 64)
    w = ctx.weight_prepare_staf(fmt3, rows, dim, blocks, pkg.LAYOUT_STAF_BLOCKS)
    got = _lookup(ctx, pkg, w, v["tokens"], dim, pkg.F32)
    for pos, t in enumerate(v["tokens"]):
        want = s[t].repeat(64) * codes[t] + z[t].repeat(64)
        assert np.max(np.abs(got[pos] - want)) < v["bar"]
    assert np.array_equal(got, oracle.embedding_lookup_staf_f32(3, 64, rows, dim, blocks, v["tokens"]))
    w.destroy()


@pytest.mark.parametrize("bits,group", kat.ALL_FORMATS)
def test_embedding_lookup_bit_exact_every_format_and_layout(pkg, ctx, bits, group):
    rng = np.random.default_rng(bits * 31 + group)
    vocab = 257
    dim = 384                                   # 3 x 128: whole groups and whole 32-bit words at every width
    codes = rng.integers(0, 1 << bits, (vocab, dim), dtype=np.uint8)
    case = Case(bits, group, codes, rng.choice([0.015625, 0.03125, 0.0625], (vocab, dim // group)),
                rng.integers(-16, 16, (vocab, dim // group)) * 0.03125)
    blocks = case.staf_blocks()
    ids = np.concatenate([[0, vocab - 1], rng.integers(0, vocab, 29)])
    want = oracle.embedding_lookup_staf_f32(bits, group, vocab, dim, blocks, ids)
    want_scaled = oracle.embedding_lookup_staf_f32(bits, group, vocab, dim, blocks, ids, 45.25)
    layouts = [pkg.LAYOUT_STAF_BLOCKS, pkg.LAYOUT_PLANES]
    if (bits, group) == (4, 64) and dim % 128 == 0:
        layouts.append(pkg.LAYOUT_TILE16)
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
    for layout in layouts:
        w = ctx.weight_prepare_staf(fmt, vocab, dim, blocks, layout)
        assert np.array_equal(_lookup(ctx, pkg, w, ids, dim, pkg.F32), want), layout
        assert np.array_equal(_lookup(ctx, pkg, w, ids, dim, pkg.F32, 45.25), want_scaled), layout
        ybf = _lookup(ctx, pkg, w, ids, dim, pkg.BF16, 45.25)
        assert np.array_equal(oracle.bf16_from_f32(ybf), oracle.bf16_from_f32(want_scaled)), layout
        yh = _lookup(ctx, pkg, w, ids[:3], dim, pkg.F16)
        assert np.array_equal(yh, want[:3].astype(np.float16).astype(np.float32)), layout
        w.destroy()


def test_embedding_lookup_strides_bounds_and_errors(pkg, ctx):
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    rng = np.random.default_rng(8)
    vocab, dim = 50, 4096
    case = Case(4, 64, rng.integers(0, 16, (vocab, dim), dtype=np.uint8), np.full((vocab, dim // 64), 0.125),
                np.full((vocab, dim // 64), -1.0))
    blocks = case.staf_blocks()
    w = ctx.weight_prepare_staf(fmt, vocab, dim, blocks, pkg.LAYOUT_PLANES)
    ids = [3, 49, 0, 7]
    got = _lookup(ctx, pkg, w, ids, dim, pkg.F32, stride=dim + 24)
    assert np.array_equal(got[:, :dim], oracle.embedding_lookup_staf_f32(4, 64, vocab, dim, blocks, ids))
    assert np.all(np.isnan(got[:, dim:]))                       # padding of the output rows untouched
    got = _lookup(ctx, pkg, w, [5, -1, 50, 6], dim, pkg.F32)    # ids outside the table: rows of zeros
    assert np.all(got[1] == 0) and np.all(got[2] == 0)
    assert np.array_equal(got[[0, 3]], oracle.embedding_lookup_staf_f32(4, 64, vocab, dim, blocks, [5, 6]))
    td = ctx.upload(np.array([1], np.int32)); od = ctx.alloc(dim * 4)
    with pytest.raises(pkg.MI355QError):
        ctx.embedding_lookup(w, td, 0, od, pkg.F32)
    with pytest.raises(pkg.MI355QError):
        ctx.embedding_lookup(w, None, 1, od, pkg.F32)
    with pytest.raises(pkg.MI355QError):
        ctx.embedding_lookup(w, td, 1, od, pkg.F32, dim - 8)
    td.free(); od.free(); w.destroy()
