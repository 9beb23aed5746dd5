"""CPU tests of the KV cache oracle and of the host-side sizing functions of the library.

Pinned by the reference's vectors: head-slot sizes (Tests/MetalCompilerTests/Core/KVCacheSizingContractTests.swift:
34-96), the q8 quantise / dequantise round trip of 0, 8, ..., 248 with error < 1.5 and the unsigned read of payload
bytes 200..231 (QuantizedQ8CorrectnessTests.swift:7-158), the supported-scheme set (STAFFormat.swift:239-262); and
by exact rational arithmetic for the codes of seeded vectors."""
from fractions import Fraction

import numpy as np
import pytest

import oracle
from __graft_entry__ import load_package

pkg = load_package()

SIZES = [  # (scheme, head dimension, bytes per head slot) -- KVCacheSizingContractTests.swift
    (0x00, 128, 256), (0x01, 192, 512), (0x02, 128, 512), (0x10, 128, 192), (0x11, 128, 192), (0x40, 128, 128),
    (0x42, 128, 128), (0x21, 128, 128), (0x61, 128, 64)]


def test_head_slot_sizes_of_the_reference():
    for scheme, head_dim, want in SIZES:
        assert oracle.kv_bytes_per_head_slot(scheme, head_dim) == want
        assert pkg.kv_bytes_per_head_slot(scheme, head_dim) == want
    for rotor, base, hd in [(0x70, 0x10, 128), (0x71, 0x40, 256)]:       # rotor schemes size as their base scheme
        assert pkg.kv_bytes_per_head_slot(rotor, hd) == pkg.kv_bytes_per_head_slot(base, hd) == oracle.kv_bytes_per_head_slot(rotor, hd)
    # ceil(headDim / weightsPerBlock) x bytesPerBlock rounded to the slot alignment, for every registered format
    for hd in (64, 80, 96, 128, 256):
        for fmt in pkg.QuantizationFormatRegistry.all_formats():
            if not fmt.in_reference_registry:
                continue
            raw = -(-hd // fmt.group_size) * fmt.bytes_per_block
            assert pkg.kv_bytes_per_head_slot(fmt.scheme_identifier, hd) == -(-raw // 64) * 64
    assert pkg.kv_bytes_per_head_slot(0x99, 128) == 0 and oracle.kv_bytes_per_head_slot(0x99, 128) == 0
    spec = pkg.KVCacheSpecification(0x10, pkg.KV_SEQUENCE_MAJOR, 4, 128, 16)      # :163-183
    assert spec.bytes_per_token_slot == 4 * 192 and spec.bytes_per_layer == 16 * 4 * 192
    assert spec.offset(2, 5) == 2 * 16 * 192 + 5 * 192
    assert pkg.KVCacheSpecification(0x10, pkg.KV_HEAD_MAJOR, 4, 128, 16).offset(2, 5) == 5 * 4 * 192 + 2 * 192


def test_supported_scheme_set():
    supported = {0x00, 0x01, 0x02, 0x10, 0x11, 0x12, 0x40, 0x41, 0x42}
    for scheme in [0x00, 0x01, 0x02, 0x10, 0x11, 0x12, 0x20, 0x21, 0x30, 0x31, 0x40, 0x41, 0x42, 0x50, 0x51, 0x52,
                   0x60, 0x61, 0x70, 0x71, 0xFF]:
        assert pkg.kv_scheme_is_supported(scheme) == (scheme in supported)
        want_bits = 8 if scheme in (0x10, 0x11, 0x12) else 4 if scheme in (0x40, 0x41, 0x42) else 0
        assert oracle.lib().orc_kv_quant_bits(scheme) == want_bits


def test_q8_round_trip_vector_of_the_reference():
    x = np.arange(32, dtype=np.float32) * 8.0                   # 0, 8, ..., 248: payload bytes above 127
    slot = oracle.kv_write_slot(0x10, x)
    assert slot[4:36].max() == 255 and slot[4:36].min() == 0
    back = oracle.kv_read_slot(0x10, slot, 32)
    assert np.max(np.abs(back.astype(np.float16).astype(np.float32) - x)) < 1.5       # the reference's bar
    # exact: scale = 248/255 in fp32, codes = round(8 i / scale); header = f16(scale), f16(0)
    scale = np.float32(248.0) / np.float32(255.0)
    assert slot[:2].view(np.float16)[0] == np.float16(scale) and slot[2:4].view(np.uint16)[0] == 0
    want = [int(Fraction(8 * i) / Fraction(float(scale)) + Fraction(1, 2)) for i in range(32)]
    assert slot[4:36].tolist() == want


def test_q8_read_is_unsigned():
    block = np.zeros(36, np.uint8)
    block[:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    block[4:] = np.arange(200, 232)
    assert np.array_equal(oracle.kv_read_slot(0x10, block, 32), np.arange(200, 232, dtype=np.float32))


@pytest.mark.parametrize("scheme,bits,group", [(0x10, 8, 32), (0x11, 8, 64), (0x12, 8, 128), (0x40, 4, 64), (0x41, 4, 128), (0x42, 4, 128)])
def test_codes_by_exact_arithmetic(scheme, bits, group):
    """Independent of the C loop: every code equals floor((v - min) / scale + 1/2) in exact rationals (ties cannot
    occur for these inputs), the header holds f16(scale) and f16(min), and reading returns f16(scale) * q + f16(min)
    with two fp32 roundings; head dimensions that end inside a group leave the rest of the block untouched."""
    rng = np.random.default_rng(scheme)
    levels = (1 << bits) - 1
    for head_dim in (group, 2 * group, group + group // 2 + 3, 7):
        x = rng.standard_normal(head_dim).astype(np.float32) * 3
        slot = np.full(oracle.kv_bytes_per_head_slot(scheme, head_dim), 0xEE, np.uint8)
        oracle.kv_write_slot(scheme, x, slot)
        bpb = 4 + group * bits // 8
        want_read = np.zeros(head_dim, np.float32)
        for g in range(-(-head_dim // group)):
            v = x[g * group:(g + 1) * group]
            lo, hi = v.min(), v.max()
            scale = max(np.float32(np.float32(hi - lo) / np.float32(levels)), np.float32(1e-10))
            block = slot[g * bpb:(g + 1) * bpb]
            assert block[:2].view(np.float16)[0] == np.float16(scale) and block[2:4].view(np.float16)[0] == np.float16(lo)
            vals = list(v) + ([np.float32(0.0)] if bits == 4 and len(v) % 2 else [])
            codes = []
            for t in vals:
                ratio = Fraction(float(np.float32(t - lo))) / Fraction(float(scale))
                assert (ratio * 2).denominator != 1 or ratio.denominator == 1      # no tie at .5
                q = min(max(int(np.floor(float(ratio + Fraction(1, 2)))), 0), levels)
                codes.append(q)
            if bits == 8:
                assert block[4:4 + len(v)].tolist() == codes
                assert np.all(block[4 + len(v):] == 0xEE)
            else:
                packed = [codes[2 * i] | (codes[2 * i + 1] << 4) for i in range(len(codes) // 2)]
                assert block[4:4 + len(packed)].tolist() == packed
                assert np.all(block[4 + len(packed):] == 0xEE)
            hs, hz = np.float32(block[:2].view(np.float16)[0]), np.float32(block[2:4].view(np.float16)[0])
            want_read[g * group:g * group + len(v)] = [np.float32(np.float32(hs * np.float32(q)) + hz) for q in codes[:len(v)]]
        assert np.array_equal(oracle.kv_read_slot(scheme, slot, head_dim), want_read)
        # quantisation error is at most half a step of the stored scale (plus the f16 rounding of scale and min)
        step = float(np.max(np.abs(oracle.kv_read_slot(scheme, slot, head_dim) - x)))
        assert step <= 0.51 * float(x.max() - x.min()) / levels + 0.02 * float(np.max(np.abs(x)))


def test_dense_schemes_and_constant_groups():
    x = np.array([1.0, -2.5, 3.14159, 65504.0, 1e-8, 0.0], np.float32)
    assert np.array_equal(oracle.kv_write_slot(0x00, x)[:12].view(np.float16), x.astype(np.float16))
    assert np.array_equal(oracle.kv_write_slot(0x01, x)[:12].view(np.uint16), oracle.bf16_from_f32(x))
    assert np.array_equal(oracle.kv_write_slot(0x02, x)[:24].view(np.float32), x)
    # a constant group: scale clamps to 1e-10 (f16: 0), every code 0, the value comes back as f16(min)
    slot = oracle.kv_write_slot(0x40, np.full(64, 0.75, np.float32))
    assert slot[:2].view(np.uint16)[0] == 0 and not slot[4:36].any()
    assert np.all(oracle.kv_read_slot(0x40, slot, 64) == 0.75)
    with pytest.raises(ValueError):
        oracle.kv_write_slot(0x52, np.zeros(64, np.float32), np.zeros(64, np.uint8))
