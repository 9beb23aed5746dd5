"""CPU-side checks of the C ABI: the library loads, exports every declared symbol, and the
host-only entry points (format registry, MLX->STAF repack, shape families, error paths) behave
like the reference interface they replace.  No compute entry point is called here."""
import ctypes as C
import subprocess

import numpy as np
import pytest

import kat
import oracle
from conftest import load_package

pkg = load_package()
KATS = kat.load_kats()


def test_library_loads_and_exports_every_declared_symbol():
    lib = pkg.library()
    assert lib.mi355q_abi_version() == 1
    names = pkg.exported_symbols()
    assert len(names) >= 40
    nm = subprocess.run(["nm", "-D", "--defined-only", pkg.LIB_PATH], capture_output=True, text=True, check=True)
    exported = {line.split()[-1] for line in nm.stdout.splitlines() if " T " in line}
    for name in names:
        assert name in exported, name
        getattr(lib, name)


# ---- T/SupportedQuantizationsContractTests.swift: registry <-> documented table ------------
def test_registry_contract():
    fmts = pkg.QuantizationFormatRegistry.all_formats()
    assert {(f.bits, f.group_size) for f in fmts} == set(kat.ALL_FORMATS)
    for f in fmts:
        assert f.scheme_identifier == kat.SCHEME_IDS[(f.bits, f.group_size)]
        assert f.bytes_per_block == 4 + f.group_size * f.bits // 8
        assert f.weights_per_block == f.group_size and f.is_quantized
        assert f.is_aligned == (f.bits in (2, 4, 8))
        assert f.gemv_kernel_name == f"gemv_q{f.bits}_g{f.group_size}"
        assert f.gemm_kernel_name_for(pkg.F32) == f"gemm_q{f.bits}_g{f.group_size}_f32s"
        assert f.gemm_kernel_name_for(pkg.F16) == f"gemm_q{f.bits}_g{f.group_size}"
        assert f.dequant_to_bfloat_kernel_name == f"dequant_q{f.bits}_g{f.group_size}_bf16"
        assert f.block_struct_name == f"BlockQ{f.bits}Affine{f.group_size}"
        assert f.embedding_lookup_token == f"q{f.bits}_g{f.group_size}"
        assert f.in_reference_registry == ((f.bits, f.group_size) not in kat.NEW_FORMATS)
        direct = (f.bits, f.group_size) in [(4, 64), (4, 128), (8, 32), (8, 64)]
        assert f.has_direct_gemm == direct
        assert f.direct_gemm_threadgroup_memory_length == (max(2 * f.group_size, 256) * 4 if direct else 0)
        assert f.batched_gemm_counts == ((2, 3) if f.bits == 4 else ())
        o = oracle.format_for_mlx(f.bits, f.group_size)
        assert (o.scheme, o.bytes_per_block) == (f.scheme_identifier, f.bytes_per_block)
        assert pkg.QuantizationFormatRegistry.format(f.scheme_identifier) == f
    alias = pkg.QuantizationFormatRegistry.format(0x42)
    assert (alias.bits, alias.group_size) == (4, 128)


@pytest.mark.parametrize("bits,group", [(4, 32), (7, 64), (1, 64), (8, 16), (4, 256), (3, 128), (0, 0)])
def test_unknown_pairs_are_rejected_without_default(bits, group):
    with pytest.raises(pkg.MI355QError) as e:
        pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
    assert e.value.status_name == "UNSUPPORTED_FORMAT"


@pytest.mark.parametrize("scheme", [0x00, 0x01, 0x02, 0x70, 0x71, 0xFF, 0x99])
def test_dense_and_rotor_schemes_are_outside_this_path(scheme):
    with pytest.raises(pkg.MI355QError) as e:
        pkg.QuantizationFormatRegistry.format(scheme)
    assert e.value.status_name == "UNSUPPORTED_FORMAT"


def test_bf16_host_rule():
    for v in [1.0, -0.5, 0.0625, 1.00390625, 1.01171875, 3.14159, -1e-8, 65504.0]:
        assert pkg.bf16_from_f32(v) == oracle.bf16_from_f32_scalar(v)


# ---- repack: T/STAFDeepTests.swift, T/STAFRoundtripTests.swift, T/STAFQuantizedRoundtripTests.swift
def test_repack_literal_nibble_vector():
    v = KATS["literal_nibble_repack"]
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    words = np.array([[int(w, 16) for w in v["mlx_words"]]], np.uint32)
    s = np.array([[int(v["scale_f16_bits"], 16)]], np.uint16)
    z = np.array([[int(v["zero_f16_bits"], 16)]], np.uint16)
    blocks = pkg.repack_mlx_to_staf(fmt, words, s, z, pkg.F16)
    assert blocks.tobytes().hex() == v["staf_block_hex"]


def test_repack_literal_layout_vector():
    v = KATS["literal_q4_layout"]
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    words = np.full((v["rows"], 8), int(v["word"], 16), np.uint32)
    s = np.full((v["rows"], 1), int(v["scale_f16_bits"], 16), np.uint16)
    z = np.full((v["rows"], 1), int(v["zero_f16_bits"], 16), np.uint16)
    blocks = pkg.repack_mlx_to_staf(fmt, words, s, z, pkg.F16)
    assert blocks.size == v["payload_bytes"]
    assert blocks.reshape(4, 36)[:, :4].tobytes() == bytes([0x00, 0x40, 0x00, 0x38]) * 4
    assert np.all(blocks.reshape(4, 36)[:, 4:] == 1)


def test_repack_converts_bf16_and_f32_scales_to_f16():
    v = KATS["bf16_scale_conversion"]
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    codes = np.array([[k % 16 for k in range(64)]], np.uint8)
    words = kat.mlx_planes(codes, 4)
    s = np.array([[kat.bf16_bits_exact(v["scale"])]], np.uint16)
    z = np.array([[kat.bf16_bits_exact(v["zero"])]], np.uint16)
    blocks = pkg.repack_mlx_to_staf(fmt, words, s, z, pkg.BF16)
    assert int(blocks[:2].view("<u2")[0]) == int(v["scale_f16_bits"], 16)
    assert int(blocks[2:4].view("<u2")[0]) == int(v["zero_f16_bits"], 16)
    assert np.array_equal(blocks[4:], kat.pack_lsb_first(codes[0], 4))
    b32 = pkg.repack_mlx_to_staf(fmt, words, np.array([[v["scale"]]], np.float32),
                                 np.array([[v["zero"]]], np.float32), pkg.F32)
    assert np.array_equal(b32, blocks)


def test_host_f16_conversion_matches_numpy_through_repack():
    """The library's own float->half rounding (used for scale normalisation) against numpy."""
    rng = np.random.default_rng(11)
    vals = np.concatenate([rng.standard_normal(4000).astype(np.float32) * np.float32(0.05),
                           (rng.standard_normal(500) * 1e-6).astype(np.float32),
                           (rng.standard_normal(500) * 3e4).astype(np.float32),
                           np.array([0.0, -0.0, 65504.0, 65519.0, 65520.0, 7e4, 5.96e-8, 2.98e-8, 2.99e-8,
                                     6.1e-5, 6.0e-5, np.inf, -np.inf], np.float32)])
    n = vals.size
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(8, 32)
    words = np.zeros((n, 8), np.uint32)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    blocks = pkg.repack_mlx_to_staf(fmt, words, vals.reshape(n, 1), vals.reshape(n, 1), pkg.F32).reshape(n, 36)
    got = blocks[:, :2].copy().view("<u2").ravel()
    assert np.array_equal(got, want)
    assert np.array_equal(blocks[:, 2:4].copy().view("<u2").ravel(), want)


@pytest.mark.parametrize("bits,group", kat.ALL_FORMATS)
def test_repack_matches_oracle_and_independent_packer(bits, group):
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
    blocks_per_row = int(32 // np.gcd(32, group * bits)) * 3
    k = group * blocks_per_row
    codes = kat.random_codes(bits * 13 + group, 5, k, bits)
    rng = np.random.default_rng(group)
    scales = (rng.integers(1, 64, size=(5, blocks_per_row)) / 256.0)
    zeros = (rng.integers(-64, 64, size=(5, blocks_per_row)) / 128.0)
    words = kat.mlx_planes(codes, bits)
    s16 = scales.astype(np.float16).view(np.uint16)
    z16 = zeros.astype(np.float16).view(np.uint16)
    got = pkg.repack_mlx_to_staf(fmt, words, s16, z16, pkg.F16)
    assert np.array_equal(got, kat.staf_blocks(codes, scales, zeros, bits, group))
    assert np.array_equal(got, oracle.repack_mlx_to_staf(bits, group, words, s16, z16, oracle.F16))


def test_repack_error_paths():
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    lib = pkg.library()
    words = np.zeros((1, 4), np.uint32)          # K = 32: not a multiple of the group size
    s = np.zeros((1, 1), np.uint16)
    out = np.zeros(64, np.uint8)
    rc = lib.mi355q_repack_mlx_to_staf(fmt.scheme_identifier, 1, 4, words.ctypes.data, s.ctypes.data,
                                       s.ctypes.data, pkg.F16, out.ctypes.data, out.size)
    assert pkg.STATUS_NAMES[rc] == "SHAPE"
    words = np.zeros((1, 8), np.uint32)
    rc = lib.mi355q_repack_mlx_to_staf(fmt.scheme_identifier, 1, 8, words.ctypes.data, s.ctypes.data,
                                       s.ctypes.data, pkg.F16, out.ctypes.data, 35)
    assert pkg.STATUS_NAMES[rc] == "SIZE_MISMATCH"
    rc = lib.mi355q_repack_mlx_to_staf(0x99, 1, 8, words.ctypes.data, s.ctypes.data, s.ctypes.data, pkg.F16,
                                       out.ctypes.data, out.size)
    assert pkg.STATUS_NAMES[rc] == "UNSUPPORTED_FORMAT"
    rc = lib.mi355q_repack_mlx_to_staf(fmt.scheme_identifier, 1, 8, None, s.ctypes.data, s.ctypes.data, pkg.F16,
                                       out.ctypes.data, out.size)
    assert pkg.STATUS_NAMES[rc] == "INVALID_ARGUMENT"
    assert b"null" in lib.mi355q_last_error()


# ---- MetalCompileContext.swift:5-90: decode shape families ---------------------------------
def test_shape_families():
    want = {
        (8192, 2048): ("input20488192Dense", 8, 2048, "gemv_2048_8192"),     # benchmark config 0
        (65536, 2048): ("vocabDense", 16, 2048, "gemv_vocab"),                # benchmark config 4
        (2048, 2048): ("input2048SquareDense", 8, 2048, "gemv_2048_sq"),
        (6144, 2048): ("input20486144Dense", 4, 2048, "gemv_2048_6144"),
        (4096, 2048): ("input2048ExpandedDense", 8, 2048, "gemv_2048"),
        (4096, 8192): ("input8192Tiled", 8, 1024, "gemv_8192_tiled"),
        (32768, 4096): ("largeDense", 8, 512, "gemv_large"),
        (4096, 4096): ("generic", 4, 256, "gemv"),
        (14336, 4096): ("generic", 4, 256, "gemv"),
        (4096, 14336): ("generic", 4, 256, "gemv"),
        (1024, 4096): ("generic", 4, 256, "gemv"),
    }
    for (n, k), expect in want.items():
        assert pkg.shape_family(n, k) == expect, (n, k)


# ---- failure handling that a host can force without a GPU ----------------------------------
def test_null_handles_and_missing_device_fail_cleanly():
    lib = pkg.library()
    assert pkg.STATUS_NAMES[lib.mi355q_qgemv(None, None, None, None, 1, None, 1, 1, 0, 0, 0)] == "NULL_HANDLE"
    assert pkg.STATUS_NAMES[lib.mi355q_weight_destroy(None)] == "NULL_HANDLE"
    assert pkg.STATUS_NAMES[lib.mi355q_weight_query(None, None)] == "NULL_HANDLE"
    assert pkg.STATUS_NAMES[lib.mi355q_context_destroy(None)] == "NULL_HANDLE"
    assert pkg.STATUS_NAMES[lib.mi355q_plan_decode_step(None, 1, 1, 0, None)] == "NULL_HANDLE"
    assert pkg.STATUS_NAMES[lib.mi355q_context_create(0, None)] == "INVALID_ARGUMENT"
    try:
        import torch
        has_gpu = torch.cuda.device_count() > 0
    except Exception:
        has_gpu = False
    if not has_gpu:
        with pytest.raises(pkg.MI355QError) as e:
            pkg.Context(0)
        assert e.value.status_name == "DEVICE"
        assert "no CPU path" in str(e.value)
