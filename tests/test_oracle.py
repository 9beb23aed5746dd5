"""CPU tests that pin the oracle against the reference's golden vectors and against
independent formulations (Python big integers, numpy float16/float64, exact rationals).

None of these needs a GPU.  A mistake in the oracle (wrong nibble order, wrong slot formula,
dropped bias term, transposed operand) fails at least one of them.
"""
import numpy as np
import pytest

import kat
import oracle

KATS = kat.load_kats()


# ------------------------------------------------------------------ formats (a1)
def test_registry_matches_reference_table():
    for bits, group in kat.ALL_FORMATS:
        f = oracle.format_for_mlx(bits, group)
        assert f is not None
        assert f.bytes_per_block == 4 + group * bits // 8
        assert f.scheme == kat.SCHEME_IDS[(bits, group)]
        assert f.in_reference == (0 if (bits, group) in kat.NEW_FORMATS else 1)
        g = oracle.format_for_scheme(f.scheme)
        assert (g.bits, g.group) == (bits, group)
    # unknown pairs are rejected, never defaulted
    for bits, group in [(4, 32), (7, 64), (1, 64), (8, 16), (4, 256), (3, 128)]:
        assert oracle.format_for_mlx(bits, group) is None
    assert oracle.format_for_scheme(0x99) is None
    # 0x42 aliases q4g128
    alias = oracle.format_for_scheme(0x42)
    assert (alias.bits, alias.group) == (4, 128)


def test_block_sizes_of_baseline_formats():
    want = {(4, 64): 36, (8, 32): 36, (3, 64): 28, (6, 64): 52, (2, 64): 20}
    for (bits, group), size in want.items():
        assert oracle.format_for_mlx(bits, group).bytes_per_block == size


# ------------------------------------------------------------- bf16 / f16 (a12)
def test_bf16_rne_known_patterns():
    cases = {1.0: 0x3F80, -0.5: 0xBF00, 0.0: 0x0000, 0.0625: 0x3D80,
             float(np.float32(1.00390625)): 0x3F80,     # 1 + 2^-8: tie -> even (down)
             float(np.float32(1.01171875)): 0x3F82,     # 1 + 3*2^-8: tie -> even (up)
             float(np.float32(1.0078125)): 0x3F81}      # 1 + 2^-7 exactly representable
    for v, bits in cases.items():
        assert oracle.bf16_from_f32_scalar(v) == bits
        assert int(oracle.bf16_from_f32(np.array([v], np.float32))[0]) == bits


def test_bf16_vector_twin_matches_c():
    rng = np.random.default_rng(1)
    v = rng.standard_normal(4096).astype(np.float32) * np.float32(3.0)
    vec = oracle.bf16_from_f32(v)
    for i in range(0, 4096, 37):
        assert int(vec[i]) == oracle.bf16_from_f32_scalar(float(v[i]))
    back = oracle.bf16_to_f32(vec)
    assert np.all(np.abs(back - v) <= np.abs(v) * 2.0 ** -8)


def test_f16_exhaustive_roundtrip_against_numpy():
    allh = np.arange(65536, dtype=np.uint16)
    asf = allh.view(np.float16).astype(np.float32)
    for h in range(0, 65536):
        f = oracle.f16_to_f32_scalar(h)
        if np.isnan(asf[h]):
            assert np.isnan(f)
            continue
        assert f == asf[h], h
    # float32 -> f16 against numpy on a dense sample incl. ties, subnormals, overflow
    rng = np.random.default_rng(2)
    samples = np.concatenate([
        rng.standard_normal(20000).astype(np.float32),
        (rng.standard_normal(5000) * 1e-6).astype(np.float32),
        (rng.standard_normal(5000) * 7e4).astype(np.float32),
        asf[~np.isnan(asf)][::7],
        np.array([2049.0, 2051.0, 65519.9, 65520.0, 5.96e-8, 2.98e-8, 2.99e-8], np.float32)])
    with np.errstate(over="ignore"):
        want = samples.astype(np.float16).view(np.uint16)
    for v, w in zip(samples, want):
        assert oracle.f16_from_f32_scalar(float(v)) == int(w), float(v)


# ------------------------------------------------------------------ unpack (a2)
@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 8])
def test_unpack_slot_formulas_equal_bitstream_closed_form(bits):
    """Brute force: every position of a 64-code run x every code value; the reference's
    per-width slot formulas must equal q_k = (stream >> k*bits) & mask."""
    n = 64
    for value in range(1 << bits):
        for k in range(n):
            codes = np.zeros(n, np.uint8)
            codes[k] = value
            stream = kat.pack_lsb_first(codes, bits)          # independent packer
            assert np.array_equal(oracle.pack_stream(codes, bits), stream)
            assert oracle.unpack_code(stream, k, bits) == value
            assert oracle.unpack_code_stream(stream, k, bits) == value
            if k:  # neighbours stay zero (no bleed across slots)
                assert oracle.unpack_code(stream, k - 1, bits) == 0
    rng = np.random.default_rng(bits)
    codes = rng.integers(0, 1 << bits, size=256, dtype=np.uint8)
    stream = kat.pack_lsb_first(codes, bits)
    got = [oracle.unpack_code(stream, k, bits) for k in range(256)]
    assert got == codes.tolist()
    assert np.array_equal(kat.unpack_lsb_first(stream, 256, bits), codes)


def test_q6_byte_formulas_from_reference_test():
    codes = np.arange(64, dtype=np.uint8)
    qs = np.zeros(48, np.uint8)
    for g in range(16):
        w0, w1, w2, w3 = (int(c) for c in codes[4 * g:4 * g + 4])
        qs[3 * g + 0] = (w0 & 0x3F) | ((w1 & 0x03) << 6)
        qs[3 * g + 1] = ((w1 >> 2) & 0x0F) | ((w2 & 0x0F) << 4)
        qs[3 * g + 2] = ((w2 >> 4) & 0x03) | ((w3 & 0x3F) << 2)
    assert np.array_equal(oracle.pack_stream(codes, 6), qs)
    assert [oracle.unpack_code(qs, k, 6) for k in range(64)] == codes.tolist()


def test_literal_nibble_word_vector():
    v = KATS["literal_nibble_repack"]
    words = np.array([[int(w, 16) for w in v["mlx_words"]]], dtype=np.uint32)
    s = np.array([[int(v["scale_f16_bits"], 16)]], np.uint16)
    z = np.array([[int(v["zero_f16_bits"], 16)]], np.uint16)
    blocks = oracle.repack_mlx_to_staf(4, 64, words, s, z, oracle.F16)
    assert blocks.tobytes().hex() == v["staf_block_hex"]
    codes = oracle.unpack_staf_codes(4, 64, 1, 64, blocks)
    assert codes[0, :8].tolist() == [0, 1, 2, 3, 4, 5, 6, 7] and not codes[0, 8:].any()
    assert np.array_equal(oracle.unpack_plane_codes(4, 1, 64, words), codes)


# ------------------------------------------------------------------ repack (a3)
def test_literal_q4_layout_vector():
    v = KATS["literal_q4_layout"]
    words = np.full((v["rows"], 8), int(v["word"], 16), dtype=np.uint32)
    s = np.full((v["rows"], 1), int(v["scale_f16_bits"], 16), np.uint16)
    z = np.full((v["rows"], 1), int(v["zero_f16_bits"], 16), np.uint16)
    blocks = oracle.repack_mlx_to_staf(4, 64, words, s, z, oracle.F16)
    assert blocks.size == v["payload_bytes"]
    for r in range(v["rows"]):
        blk = blocks[36 * r:36 * r + 36]
        assert blk[:4].tobytes() == bytes([0x00, 0x40, 0x00, 0x38])
        assert np.all(blk[4:] == 0x01)


def test_bf16_scales_are_converted_not_copied():
    v = KATS["bf16_scale_conversion"]
    codes = np.array([[k % 16 for k in range(64)]], np.uint8)
    words = kat.mlx_planes(codes, 4)
    s = np.array([[kat.bf16_bits_exact(v["scale"])]], np.uint16)
    z = np.array([[kat.bf16_bits_exact(v["zero"])]], np.uint16)
    blocks = oracle.repack_mlx_to_staf(4, 64, words, s, z, oracle.BF16)
    assert int(blocks[:2].view("<u2")[0]) == int(v["scale_f16_bits"], 16)
    assert int(blocks[2:4].view("<u2")[0]) == int(v["zero_f16_bits"], 16)
    assert np.array_equal(blocks[4:], kat.pack_lsb_first(codes[0], 4))
    # f32 scales take the same path
    blocks32 = oracle.repack_mlx_to_staf(4, 64, words, np.array([[v["scale"]]], np.float32),
                                         np.array([[v["zero"]]], np.float32), oracle.F32)
    assert np.array_equal(blocks32, blocks)


@pytest.mark.parametrize("case", KATS["roundtrip_multirow"]["cases"],
                         ids=lambda c: f"q{c['bits']}g{c['group']}")
def test_multirow_repack_is_byte_exact(case):
    codes, scales, zeros = kat.roundtrip_case(case["bits"], case["group"], case["rows"],
                                              case["blocks"], case["scale_base"], case["zero_base"])
    want = kat.staf_blocks(codes, scales, zeros, case["bits"], case["group"])   # independent
    words = kat.mlx_planes(codes, case["bits"])
    s16 = scales.astype(np.float16).view(np.uint16)
    z16 = zeros.astype(np.float16).view(np.uint16)
    got = oracle.repack_mlx_to_staf(case["bits"], case["group"], words, s16, z16, oracle.F16)
    assert np.array_equal(got, want)
    k = case["group"] * case["blocks"]
    w2, s2, z2 = oracle.staf_to_planes(case["bits"], case["group"], case["rows"], k, got)
    assert np.array_equal(w2, words) and np.array_equal(s2, s16) and np.array_equal(z2, z16)


@pytest.mark.parametrize("bits,group", kat.ALL_FORMATS)
def test_word_view_equals_byte_view(bits, group):
    """MLX little-endian word plane and STAF byte stream are the same bit stream."""
    blocks_per_row = 32 // np.gcd(32, group * bits) * 2   # whole words per row
    k = group * int(blocks_per_row)
    codes = kat.random_codes(100 + bits * 7 + group, 3, k, bits)
    words = kat.mlx_planes(codes, bits)
    s = np.full((3, k // group), 0x3C00, np.uint16)
    z = np.zeros((3, k // group), np.uint16)
    blocks = oracle.repack_mlx_to_staf(bits, group, words, s, z, oracle.F16)
    assert np.array_equal(oracle.unpack_staf_codes(bits, group, 3, k, blocks), codes)
    assert np.array_equal(oracle.unpack_plane_codes(bits, 3, k, words), codes)
    bpb = 4 + group * bits // 8
    for r in range(3):
        for b in range(k // group):
            qs = blocks[(r * (k // group) + b) * bpb + 4:(r * (k // group) + b + 1) * bpb]
            assert np.array_equal(qs, kat.pack_lsb_first(codes[r, b * group:(b + 1) * group], bits))


# ----------------------------------------------------------------- dequant (a11)
@pytest.mark.parametrize("case", KATS["single_block"]["cases"],
                         ids=lambda c: f"q{c['bits']}g{c['group']}")
def test_single_block_dequant_is_exact(case):
    bits, group = case["bits"], case["group"]
    scale, zero = case["dequant"]
    codes, s, z, _ = kat.single_block_case(bits, group, scale, zero)
    blocks = kat.staf_blocks(codes, s, z, bits, group)
    got = oracle.dequant_staf_f32(bits, group, 1, group, blocks)
    want = np.array([[scale * int(q) + zero for q in codes[0]]], np.float64)   # exact: pow2 scale
    assert np.array_equal(got.astype(np.float64), want)
    bf = oracle.dequant_staf_bf16(bits, group, 1, group, blocks)
    assert np.array_equal(bf, oracle.bf16_from_f32(got))


def test_two_row_q3_dequant():
    v = KATS["dequant_two_rows_q3g64"]
    codes = np.array([[k % 8 for k in range(64)], [7 - (k % 8) for k in range(64)]], np.uint8)
    s = np.full((2, 1), v["scale"]); z = np.full((2, 1), v["zero"])
    blocks = kat.staf_blocks(codes, s, z, 3, 64)
    got = oracle.dequant_staf_f32(3, 64, 2, 64, blocks)
    assert np.array_equal(got, (codes.astype(np.float32) * np.float32(v["scale"]) + np.float32(v["zero"])))


def test_cpu_weight_store_vector():
    qs = np.array([((2 * i) % 16) | (((2 * i + 1) % 16) << 4) for i in range(32)], np.uint8)
    block = np.concatenate([np.array([0x00, 0x3C, 0x00, 0x00], np.uint8), qs])
    got = oracle.dequant_staf_f32(4, 64, 1, 64, block)
    assert got[0].tolist() == [float(i % 16) for i in range(64)]


def test_planes_and_staf_dequant_agree_with_bf16_scales():
    """benchmark-style bf16 scales are exact in f16 for the configured value range, so both
    layouts dequantise to identical fp32 weights."""
    w = kat.seeded_weights(7, 16, 256)
    for bits, group in [(4, 64), (8, 32), (6, 64), (3, 64), (2, 64)]:
        codes, s, z = oracle.quantize_affine(w, bits, group, oracle.BF16)
        a = oracle.dequant_planes_f32(bits, group, 16, 256, codes, s, z, oracle.BF16)
        blocks = oracle.repack_mlx_to_staf(bits, group, codes, s, z, oracle.BF16)
        b = oracle.dequant_staf_f32(bits, group, 16, 256, blocks)
        assert np.array_equal(a, b)
        qmax = (1 << bits) - 1
        step = oracle.bf16_to_f32(s).max()
        # half a step, plus the bf16 rounding of scale (felt at the top code) and of bias
        assert np.max(np.abs(a - w)) <= 0.5 * step + qmax * step * 2.0 ** -8 + 0.08 * 2.0 ** -8
        assert oracle.unpack_plane_codes(bits, 16, 256, codes).max() <= qmax


# -------------------------------------------------------------------- gemv (a4/a6)
def test_literal_q4_gemv_vector():
    v = KATS["literal_q4_gemv"]
    words = np.array([[int(r["word"], 16)] * 8 for r in v["rows"]], np.uint32)
    s = np.array([[kat.f16_bits(r["scale"])] for r in v["rows"]], np.uint16)
    z = np.array([[kat.f16_bits(r["zero"])] for r in v["rows"]], np.uint16)
    blocks = oracle.repack_mlx_to_staf(4, 64, words, s, z, oracle.F16)
    x = np.ones((1, 64), np.float32)
    y = oracle.qgemm_staf_ref_f32(4, 64, blocks, x, 2, 64)
    assert y[0].tolist() == [r["y"] for r in v["rows"]]
    w = oracle.dequant_staf_f32(4, 64, 2, 64, blocks)
    assert oracle.gemm_f64(w, x)[0].tolist() == [r["y"] for r in v["rows"]]


@pytest.mark.parametrize("case", KATS["single_block"]["cases"],
                         ids=lambda c: f"q{c['bits']}g{c['group']}")
def test_single_block_gemv(case):
    bits, group = case["bits"], case["group"]
    scale, zero = case["gemv"]
    codes, s, z, x = kat.single_block_case(bits, group, scale, zero)
    want = kat.exact_gemv(codes, s, z, x, group)
    blocks = kat.staf_blocks(codes, s, z, bits, group)
    w = oracle.dequant_staf_f32(bits, group, 1, group, blocks)
    assert np.allclose(oracle.gemm_f64(w, x), want, rtol=0, atol=1e-12)
    assert np.allclose(oracle.qgemm_staf_ref_f32(bits, group, blocks, x, 1, group), want,
                       rtol=1e-6, atol=1e-5)


@pytest.mark.parametrize("bits,group", kat.REFERENCE_FORMATS)
def test_multi_block_and_multi_row_gemv(bits, group):
    for codes, s, z, x in (kat.multi_block_case(bits, group), kat.multi_row_case(bits, group)):
        n, k = codes.shape
        want = kat.exact_gemv(codes, s, z, x, group)
        blocks = kat.staf_blocks(codes, s, z, bits, group)
        w = oracle.dequant_staf_f32(bits, group, n, k, blocks)
        assert np.allclose(oracle.gemm_f64(w, x), want, rtol=0, atol=1e-9)
        for threads in (1, 3):
            got = oracle.qgemm_staf_ref_f32(bits, group, blocks, x, n, k, threads=threads)
            assert np.allclose(got, want, rtol=1e-5, atol=1e-4)
        if (k * bits) % 32 == 0:
            words, s16, z16 = oracle.staf_to_planes(bits, group, n, k, blocks)
            got = oracle.qgemm_planes_ref_f32(bits, group, words, s16, z16, oracle.F16, x, n, k, 2)
            assert np.array_equal(got, oracle.qgemm_staf_ref_f32(bits, group, blocks, x, n, k))


def test_integer_dot_product_special_case():
    """scale=1, zero=0 reduces the path to an integer dot product (exact in fp32 here)."""
    for bits, group in kat.ALL_FORMATS:
        k = group * 4 * (2 if (group * 4 * bits) % 32 else 1)
        codes = kat.random_codes(bits * 31 + group, 5, k, bits)
        xi = np.random.default_rng(3).integers(-4, 5, size=(2, k))
        s = np.ones((5, k // group)); z = np.zeros((5, k // group))
        blocks = kat.staf_blocks(codes, s, z, bits, group)
        want = xi @ codes.astype(np.int64).T
        got = oracle.qgemm_staf_ref_f32(bits, group, blocks, xi.astype(np.float32), 5, k)
        assert np.array_equal(got.astype(np.int64), want)


def test_q4_gemm_with_padded_input_stride():
    v = KATS["q4_gemm_padded_stride"]
    k, n, m, stride = v["k"], v["n"], v["m"], v["stride"]
    x = np.full((m, stride), v["poison"], np.float32)
    for mi in range(m):
        for c in range(k):
            x[mi, c] = (mi + 3) * ((c % 7) - 3) * 0.125
    codes = np.array([[r + 1] * k for r in range(n)], np.uint8)
    s = np.full((n, 1), v["scale"]); z = np.full((n, 1), v["zero"])
    blocks = kat.staf_blocks(codes, s, z, 4, 64)
    want = np.array([[0.25 * (r + 1) * x[mi, :k].astype(np.float64).sum() for r in range(n)]
                     for mi in range(m)])
    got = oracle.qgemm_staf_ref_f32(4, 64, blocks, x, n, k)
    assert np.max(np.abs(got - want)) < 1e-3
    w = oracle.dequant_staf_f32(4, 64, n, k, blocks)
    assert np.max(np.abs(oracle.gemm_f64(w, x, x_stride=stride) - want)) < 1e-9


def test_q3_dequant_bf16_then_gemm():
    v = KATS["q3_dequant_then_gemm"]
    k, n, m, group = v["k"], v["n"], v["m"], v["group"]
    nb = k // group
    codes = np.array([[(e + 3 * b + 5 * r) % 8 for b in range(nb) for e in range(group)]
                      for r in range(n)], np.uint8)
    s = np.array([[0.03125 * (b + 1) + 0.0078125 * r for b in range(nb)] for r in range(n)])
    z = np.array([[-0.125 + 0.0625 * r - 0.015625 * b for b in range(nb)] for r in range(n)])
    x = np.array([((i % 17) - 8) * 0.0625 for i in range(m * k)], np.float32).reshape(m, k)
    blocks = kat.staf_blocks(codes, s, z, 3, group)
    want = kat.exact_gemv(codes, s, z, x, group)
    wb = oracle.bf16_to_f32(oracle.dequant_staf_bf16(3, group, n, k, blocks))
    assert np.max(np.abs(oracle.gemm_f64(wb, x) - want)) < 0.02     # the reference's own bar


# ------------------------------------------------------------------ argmax (a10)
def test_argmax_lowest_index_brute_force():
    assert oracle.argmax_lowest(np.zeros(0, np.float32)) == 0
    assert oracle.argmax_lowest(np.full(9, np.nan, np.float32)) == 0
    assert oracle.argmax_lowest(np.array([np.nan, 1.0, np.nan, 1.0], np.float32)) == 1
    assert oracle.argmax_lowest(np.array([-0.0, 0.0, -0.0], np.float32)) == 0
    assert oracle.argmax_lowest(np.array([0.0, -0.0], np.float32)) == 0
    assert oracle.argmax_lowest(np.full(5, -np.inf, np.float32)) == 0
    assert oracle.argmax_lowest(np.array([-np.inf, np.inf, np.inf], np.float32)) == 1
    rng = np.random.default_rng(5)
    for n in (1, 2, 63, 64, 65, 127, 128, 129, 1000):
        for _ in range(20):
            v = rng.integers(-3, 4, size=n).astype(np.float32)    # many ties
            assert oracle.argmax_lowest(v) == int(np.argmax(v))   # numpy: first occurrence


# --------------------------------------------------------------- quantizer (D7)
def test_quantizer_formula_on_a_hand_group():
    w = np.linspace(-0.05, 0.04, 64, dtype=np.float32)[None, :]
    codes, s, z = oracle.quantize_affine(w, 4, 64, oracle.F32)
    scale = np.float32((w.max() - w.min()) / np.float32(15))
    assert s[0, 0] == scale and z[0, 0] == w.min()
    q = oracle.unpack_plane_codes(4, 1, 64, codes)[0]
    want = np.clip(np.floor((w[0] - w.min()) / scale + np.float32(0.5)), 0, 15).astype(np.uint8)
    assert np.array_equal(q, want)
    assert q[0] == 0 and q[-1] == 15
    # constant group: scale floors at 1e-10, codes all zero
    codes, s, z = oracle.quantize_affine(np.full((1, 64), 0.25, np.float32), 4, 64, oracle.F32)
    assert s[0, 0] == np.float32(1e-10) and not codes.any()


# ------------------------------------------------------------------ quantized embedding gather (N1)
def _q3_embedding_rows(v):
    dim, group, rows = v["dim"], v["group"], v["rows"]
    codes = np.array([[(i + 3 * g + 5 * t) % 8 for g in range(dim // group) for i in range(group)]
                      for t in range(rows)], np.uint8)
    s = np.array([[0.03125 * (g + 1) + 0.0078125 * t for g in range(dim // group)] for t in range(rows)])
    z = np.array([[-0.125 + 0.0625 * t - 0.015625 * g for g in range(dim // group)] for t in range(rows)])
    return codes, s, z


def test_embedding_lookup_reference_vectors():
    v = KATS["embedding_q4_row_of_twos"]
    codes = np.array([[t] * v["dim"] for t in v["row_values"]], np.uint8)
    blocks = kat.staf_blocks(codes, np.ones((2, 1)), np.zeros((2, 1)), 4, 64)
    out = oracle.embedding_lookup_staf_f32(4, 64, 2, v["dim"], blocks, [v["token"]])
    assert out.shape == (1, 64) and np.all(np.abs(out - v["expected"]) < 0.001)
    out = oracle.embedding_lookup_staf_f32(4, 64, 2, v["dim"], blocks, [v["token"]], v["scale"])
    assert np.all(np.abs(out - v["expected_scaled"]) < 0.001)

    v = KATS["embedding_q3_sequence"]
    codes, s, z = _q3_embedding_rows(v)
    blocks = kat.staf_blocks(codes, s, z, 3, 64)
    out = oracle.embedding_lookup_staf_f32(3, 64, v["rows"], v["dim"], blocks, v["tokens"])
    for pos, t in enumerate(v["tokens"]):
        want = (s[t].repeat(64).astype(np.float32) * codes[t].astype(np.float32) + z[t].repeat(64).astype(np.float32))
        assert np.max(np.abs(out[pos] - want)) < v["bar"]                  # the reference's own bar


def test_embedding_lookup_is_a_row_gather_of_the_dequantised_table():
    """Independent of the gather loop: every output row equals the corresponding row of the CPU dequant
    (itself pinned by the CPUWeightStore vector), times the scale; an id outside the table is an error."""
    rng = np.random.default_rng(21)
    for bits, group in [(4, 64), (8, 32), (3, 64), (6, 16), (2, 32), (5, 32)]:
        vocab, dim = 37, group * 6
        codes = rng.integers(0, 1 << bits, (vocab, dim), dtype=np.uint8)
        s = rng.uniform(0.01, 0.1, (vocab, dim // group)); z = rng.uniform(-0.5, 0.5, (vocab, dim // group))
        blocks = kat.staf_blocks(codes, s, z, bits, group)
        table = oracle.dequant_staf_f32(bits, group, vocab, dim, blocks)
        ids = rng.integers(0, vocab, 11)
        assert np.array_equal(oracle.embedding_lookup_staf_f32(bits, group, vocab, dim, blocks, ids), table[ids])
        scaled = oracle.embedding_lookup_staf_f32(bits, group, vocab, dim, blocks, ids, 1.75)
        assert np.array_equal(scaled, table[ids] * np.float32(1.75))
    with pytest.raises(ValueError):
        oracle.embedding_lookup_staf_f32(4, 64, 2, 64, kat.staf_blocks(np.zeros((2, 64), np.uint8), np.ones((2, 1)),
                                                                        np.zeros((2, 1)), 4, 64), [2])


# ------------------------------------------------------------------ gated activation (swiglu / gelu_gated)
def test_gated_activation_closed_forms_and_fp64():
    """The reference holds no value test of its gated-activation kernels, so the restatement is pinned by what the
    formulas fix: act(0) = 0, u = 0 -> 0, large g -> g u exactly (sigmoid and tanh saturate to 1 in fp32), very negative
    g -> 0 (exp overflows to inf), silu(1) and gelu_tanh(1) from their definitions, and an fp64 evaluation of both
    formulas on seeded values; with a 16-bit buffer type, gate, up and the product are each rounded to it."""
    g = np.array([0.0, 30.0, -100.0, 1.0, 5.0, 88.0, -0.0], np.float32)
    u = np.array([3.0, 2.0, 7.0, 1.0, 0.0, 0.5, 2.0], np.float32)
    for kind in (oracle.SILU, oracle.GELU_TANH):
        out = oracle.gated_activation_f32(g, u, kind)
        assert out[0] == 0.0 and out[1] == 60.0 and out[2] == 0.0 and out[4] == 0.0 and out[5] == 44.0 and out[6] == 0.0
    assert abs(oracle.gated_activation_f32(g, u, oracle.SILU)[3] - 1.0 / (1.0 + np.exp(-1.0))) < 1e-7
    assert abs(oracle.gated_activation_f32(g, u, oracle.GELU_TANH)[3] - 0.5 * (1.0 + np.tanh(0.7978845608 * 1.044715))) < 1e-7
    rng = np.random.default_rng(12)
    gs = (rng.standard_normal(4000) * 4).astype(np.float32)
    us = rng.standard_normal(4000).astype(np.float32)
    g64, u64 = gs.astype(np.float64), us.astype(np.float64)
    silu = g64 / (1.0 + np.exp(-g64)) * u64
    gelu = 0.5 * g64 * (1.0 + np.tanh(0.7978845608 * (g64 + 0.044715 * g64 ** 3))) * u64
    assert np.allclose(oracle.gated_activation_f32(gs, us, oracle.SILU), silu, rtol=3e-6, atol=1e-7)
    # 1 + tanh cancels for negative g: an absolute error of a few fp32 steps of |g u|
    assert np.allclose(oracle.gated_activation_f32(gs, us, oracle.GELU_TANH), gelu, rtol=1e-5, atol=5e-6)
    # a sign error, a dropped cubic term or a transposed operand moves these by far more than the bars above
    assert not np.allclose(oracle.gated_activation_f32(gs, us, oracle.SILU), gelu, rtol=1e-3, atol=1e-4)
    # buffer type bf16: inputs and output on the bf16 grid
    gb = oracle.bf16_to_f32(oracle.bf16_from_f32(gs)); ub = oracle.bf16_to_f32(oracle.bf16_from_f32(us))
    want = oracle.bf16_to_f32(oracle.bf16_from_f32(oracle.gated_activation_f32(gb, ub, oracle.SILU)))
    assert np.array_equal(oracle.gated_activation_f32(gs, us, oracle.SILU, oracle.BF16), want)
