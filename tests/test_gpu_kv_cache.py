"""GPU parity tests of the quantized KV cache write / read through the C ABI: cache bytes and read-back values are
bit-exact against the CPU oracle (write_kv_quantized / read_kv_element,
Sources/MetalCompiler/Generator/MetalSourceGenerator+Attention.swift:1923-1956, 2057-2180)."""
import numpy as np
import pytest

import oracle
from gpu_util import act_to_device_array, act_rounded, out_from_device

pytestmark = pytest.mark.gpu
SCHEMES = [0x00, 0x01, 0x02, 0x10, 0x11, 0x12, 0x40, 0x41, 0x42]


def _roundtrip(pkg, ctx, scheme, layout_mode, kv_heads, head_dim, max_pos, first, count, src_dtype, seed, pad=0):
    rng = np.random.default_rng(seed)
    spec = pkg.KVCacheSpecification(scheme, layout_mode, kv_heads, head_dim, max_pos)
    row = kv_heads * head_dim
    x = np.full((count, row + pad), 777.0, np.float32)
    x[:, :row] = act_rounded((rng.standard_normal((count, row)) * rng.choice([0.1, 1.0, 30.0], (count, 1))).astype(np.float32),
                             src_dtype, pkg)
    cache0 = np.full(spec.bytes_per_layer, 0xEE, np.uint8)
    cd = ctx.upload(cache0)
    xd = ctx.upload(act_to_device_array(x, src_dtype, pkg))
    ctx.kv_cache_write(spec, cd, xd, src_dtype, first, count, (row + pad) if pad else 0)
    ctx.synchronize()
    got = cd.download(np.uint8, (cache0.size,))
    want = oracle.kv_cache_write(scheme, layout_mode, kv_heads, head_dim, max_pos, x[:, :row], first, cache0.copy())
    assert np.array_equal(got, want), f"cache bytes differ: scheme 0x{scheme:02x} layout {layout_mode} hd {head_dim}"
    for out_dtype in (pkg.F32, pkg.BF16, pkg.F16):
        od = ctx.alloc(count * (row + pad) * (4 if out_dtype == pkg.F32 else 2))
        ctx.fill(od, 0x7FC00000 if out_dtype == pkg.F32 else 0x7FC07FC0)
        ctx.kv_cache_read(spec, cd, od, out_dtype, first, count, (row + pad) if pad else 0)
        ctx.synchronize()
        y = out_from_device(od, out_dtype, (count, row + pad), pkg)
        ref = oracle.kv_cache_read(scheme, layout_mode, kv_heads, head_dim, max_pos, want, first, count)
        if out_dtype == pkg.F32:
            assert np.array_equal(y[:, :row], ref)
        elif out_dtype == pkg.BF16:
            assert np.array_equal(oracle.bf16_from_f32(y[:, :row]), oracle.bf16_from_f32(ref))
        else:
            assert np.array_equal(y[:, :row], ref.astype(np.float16).astype(np.float32))
        if pad:
            assert np.all(np.isnan(y[:, row:]))
        od.free()
    cd.free(); xd.free()
    return x[:, :row], oracle.kv_cache_read(scheme, layout_mode, kv_heads, head_dim, max_pos, want, first, count)


@pytest.mark.parametrize("scheme", SCHEMES)
def test_kv_cache_bytes_bit_exact(pkg, ctx, scheme):
    for i, (layout, heads, hd, max_pos, first, count, dt) in enumerate([
            (pkg.KV_SEQUENCE_MAJOR, 8, 128, 64, 0, 17, pkg.BF16),
            (pkg.KV_HEAD_MAJOR, 8, 128, 64, 40, 24, pkg.F16),
            (pkg.KV_SEQUENCE_MAJOR, 2, 256, 8, 7, 1, pkg.F32),       # decode: one position appended
            (pkg.KV_HEAD_MAJOR, 3, 80, 16, 3, 5, pkg.BF16),          # head dimension ends inside a group
            (pkg.KV_SEQUENCE_MAJOR, 1, 7, 4, 0, 4, pkg.F32),         # shorter than any group, odd
            (pkg.KV_HEAD_MAJOR, 4, 128, 32, 5, 9, pkg.F32),          # 128-element heads from fp32 rows
            (pkg.KV_SEQUENCE_MAJOR, 4, 128, 32, 0, 6, pkg.BF16),     # the same with an odd row stride
            (pkg.KV_SEQUENCE_MAJOR, 3, 128, 16, 2, 5, pkg.BF16),     # an odd number of 128-element vectors
            (pkg.KV_HEAD_MAJOR, 3, 128, 16, 0, 7, pkg.F16),          # row stride a multiple of two, not of four
            (pkg.KV_HEAD_MAJOR, 1, 128, 8, 0, 1, pkg.F32)]):         # a single vector
        pad = {1: 8, 6: 7, 8: 2}.get(i, 0)
        x, back = _roundtrip(pkg, ctx, scheme, layout, heads, hd, max_pos, first, count, dt, 100 * scheme + i, pad=pad)
        if scheme in (0x10, 0x11, 0x12):
            assert np.max(np.abs(back - x)) <= 0.51 * 8 * 30 / 255 + 0.02 * np.max(np.abs(x))


def test_reference_q8_vectors_on_the_gpu(pkg, ctx):
    """QuantizedQ8CorrectnessTests.swift:7-158: 0, 8, ..., 248 survives the q8 g32 round trip within 1.5, and payload
    bytes 200..231 with scale 1 read back as 200..231."""
    spec = pkg.KVCacheSpecification(0x10, pkg.KV_SEQUENCE_MAJOR, 1, 32, 1)
    x = np.arange(32, dtype=np.float32)[None, :] * 8.0
    cd = ctx.alloc(spec.bytes_per_layer); ctx.fill(cd, 0)
    xd = ctx.upload(x.astype(np.float16).view(np.uint16))
    od = ctx.alloc(32 * 2)
    ctx.kv_cache_write(spec, cd, xd, pkg.F16, 0, 1)
    ctx.kv_cache_read(spec, cd, od, pkg.F16, 0, 1)
    ctx.synchronize()
    assert np.max(np.abs(od.download(np.uint16, (32,)).view(np.float16).astype(np.float32) - x[0])) < 1.5
    assert np.array_equal(cd.download(np.uint8, (spec.bytes_per_layer,))[:36], oracle.kv_write_slot(0x10, x[0])[:36])
    block = np.zeros(spec.bytes_per_layer, np.uint8)
    block[:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    block[4:36] = np.arange(200, 232)
    cd.upload(block)
    of = ctx.alloc(32 * 4)
    ctx.kv_cache_read(spec, cd, of, pkg.F32, 0, 1)
    ctx.synchronize()
    assert np.array_equal(of.download(np.float32, (32,)), np.arange(200, 232, dtype=np.float32))
    for b in (cd, xd, od, of):
        b.free()


def test_kv_cache_argument_errors(pkg, ctx):
    spec = pkg.KVCacheSpecification(0x40, pkg.KV_SEQUENCE_MAJOR, 2, 64, 8)
    cd = ctx.alloc(spec.bytes_per_layer); xd = ctx.alloc(8 * 128 * 4)
    for bad, name in [(pkg.KVCacheSpecification(0x52, 0, 2, 64, 8), "UNSUPPORTED_FORMAT"),       # q3: sizable, no kernels
                      (pkg.KVCacheSpecification(0x71, 0, 2, 64, 8), "UNSUPPORTED_FORMAT"),       # rotor: needs the pre-rotation
                      (pkg.KVCacheSpecification(0x40, 2, 2, 64, 8), "INVALID_ARGUMENT")]:
        with pytest.raises(pkg.MI355QError) as err:
            ctx.kv_cache_write(bad, cd, xd, pkg.F32, 0, 1)
        assert err.value.status_name == name
    with pytest.raises(pkg.MI355QError) as err:
        ctx.kv_cache_write(spec, cd, xd, pkg.F32, 6, 3)                  # positions 6..8 leave the cache
    assert err.value.status_name == "SHAPE"
    with pytest.raises(pkg.MI355QError):
        ctx.kv_cache_write(spec, cd, xd, pkg.F32, 0, 1, 100)             # row stride shorter than heads x head dim
    with pytest.raises(pkg.MI355QError):
        ctx.kv_cache_read(spec, cd, None, pkg.F32, 0, 1)
    cd.free(); xd.free()


@pytest.mark.parametrize("scheme,out_dtype", [(0x40, 1), (0x10, 2), (0x01, 1)])
def test_kv_cache_read_of_more_positions_than_one_grid_dimension(pkg, ctx, scheme, out_dtype):
    """One read of 70 000 positions (more than the 65 535 workgroups a grid holds along y) returns what three
    shorter reads return, and its last positions match the oracle."""
    heads, hd, count = 1, 64, 70000
    spec = pkg.KVCacheSpecification(scheme, pkg.KV_SEQUENCE_MAJOR, heads, hd, count)
    rng = np.random.default_rng(scheme)
    x = rng.standard_normal((count, hd)).astype(np.float32)
    xd = ctx.upload(x)
    cd = ctx.alloc(spec.bytes_per_layer); ctx.fill(cd, 0)
    ctx.kv_cache_write(spec, cd, xd, pkg.F32, 0, count)
    esz = 4 if out_dtype == pkg.F32 else 2
    whole = ctx.alloc(count * hd * esz); ctx.fill(whole, 0x7FC07FC0)
    parts = ctx.alloc(count * hd * esz); ctx.fill(parts, 0x7FC07FC0)
    ctx.kv_cache_read(spec, cd, whole, out_dtype, 0, count)
    for first, n in [(0, 30000), (30000, 30000), (60000, 10000)]:
        ctx.kv_cache_read(spec, cd, pkg.DeviceBuffer(ctx, parts.ptr + first * hd * esz, n * hd * esz), out_dtype, first, n)
    ctx.synchronize()
    a = whole.download(np.uint8)
    assert np.array_equal(a, parts.download(np.uint8))
    tail_first, tail = 65530, 40
    cache = cd.download(np.uint8, (spec.bytes_per_layer,))
    ref = oracle.kv_cache_read(scheme, pkg.KV_SEQUENCE_MAJOR, heads, hd, count, cache, tail_first, tail)
    got = out_from_device(whole, out_dtype, (count, hd), pkg)[tail_first:tail_first + tail]
    if out_dtype == pkg.F32:
        assert np.array_equal(got, ref)
    else:
        assert np.array_equal(oracle.bf16_from_f32(got), oracle.bf16_from_f32(ref))
    for b in (xd, cd, whole, parts):
        b.free()
