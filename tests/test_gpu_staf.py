"""GPU tests: a model.staf written to disk, opened, uploaded as one device buffer and served to the kernels
(STAFLoader.load -> STAFWeightStore.resolvedBufferAccess -> dispatch; the reference's end-to-end checks are
Tests/MetalCompilerTests/Core/STAFDeepTests.swift:15-129 and STAFEndToEndGEMVTests.swift)."""
import numpy as np
import pytest

import kat
import oracle
from gpu_util import Case, act_rounded, act_to_device_array, assert_within_tolerance, out_from_device

pytestmark = pytest.mark.gpu


def _gemv(ctx, pkg, w, x, n):
    xd = ctx.upload(act_to_device_array(x, pkg.BF16, pkg))
    yd = ctx.alloc(n * 4)
    ctx.qgemv(w, xd, pkg.BF16, yd, pkg.F32, 1)
    ctx.synchronize()
    y = out_from_device(yd, pkg.F32, (n,), pkg)
    xd.free(); yd.free()
    return y


def test_projections_served_from_a_container(pkg, ctx, tmp_path):
    rng = np.random.default_rng(12)
    cases = {}
    tensors = [dict(name="model.norm.weight", scheme_identifier=0x01, shape=[64], payload=bytes(128))]
    for name, bits, group, n, k in [("layers.0.q_proj.weight", 4, 64, 96, 512), ("layers.0.up_proj.weight", 8, 32, 40, 256),
                                    ("layers.0.down_proj.weight", 3, 64, 33, 256), ("embed.weight", 4, 64, 48, 256)]:
        c = Case(bits, group, rng.integers(0, 1 << bits, (n, k), dtype=np.uint8),
                 rng.choice([0.015625, 0.03125], (n, k // group)), rng.integers(-8, 8, (n, k // group)) * 0.0625)
        cases[name] = c
        scheme = kat.SCHEME_IDS[(bits, group)]
        tensors.append(dict(name=name, scheme_identifier=scheme, shape=[n, k * bits // 32], payload=c.staf_blocks().tobytes()))
    path = str(tmp_path / "model.staf")
    pkg.staf_write(path, tensors, {"staf.converter_version": (pkg.STAF_UINT32, 3)})
    f = pkg.STAFFile(path)
    region = f.upload(ctx)
    assert region.nbytes == f.payload_region().size
    assert np.array_equal(region.download(np.uint8, (region.nbytes,)), f.payload_region())
    for name, c in cases.items():
        x = act_rounded(rng.standard_normal(c.k).astype(np.float32), pkg.BF16, pkg)
        want = oracle.gemm_f64(oracle.dequant_staf_f32(c.bits, c.group, c.n, c.k, c.staf_blocks()), x[None, :])[0]
        layouts = [pkg.LAYOUT_STAF_BLOCKS, pkg.LAYOUT_PLANES] + ([pkg.LAYOUT_TILE16] if (c.bits, c.group, c.k % 128) == (4, 64, 0) else [])
        for layout in layouts:
            w = f.weight(ctx, name, layout, region)
            info = w.info
            assert (info.n_rows, info.k, info.layout) == (c.n, c.k, layout)
            assert_within_tolerance(_gemv(ctx, pkg, w, x, c.n), want, f"{name} layout {layout}")
            w.destroy()
    # the embedding table of the same container, gathered bit-exactly
    c = cases["embed.weight"]
    w = f.weight(ctx, "embed.weight", pkg.LAYOUT_STAF_BLOCKS, region)
    ids = np.array([5, 0, 47], np.int32)
    td = ctx.upload(ids); od = ctx.alloc(3 * c.k * 4)
    ctx.embedding_lookup(w, td, 3, od, pkg.F32)
    ctx.synchronize()
    assert np.array_equal(od.download(np.float32, (3, c.k)),
                          oracle.embedding_lookup_staf_f32(4, 64, c.n, c.k, c.staf_blocks(), ids))
    td.free(); od.free(); w.destroy()
    with pytest.raises(pkg.MI355QError) as err:
        f.weight(ctx, "model.norm.weight", pkg.LAYOUT_STAF_BLOCKS, region)      # dense tensor: not a packed format
    assert err.value.status_name == "UNSUPPORTED_FORMAT"
    with pytest.raises(pkg.MI355QError) as err:
        f.weight(ctx, "nope", pkg.LAYOUT_STAF_BLOCKS, region)
    assert err.value.status_name == "NOT_FOUND"
    region.free(); f.close()


def test_reference_q4_vector_through_a_container(pkg, ctx, tmp_path):
    """STAFDeepTests.swift:15-129: row 0 = codes of 3 with scale 1 and bias 0, row 1 = codes of 2 with scale 2 and
    bias 1, against x = 1: 192 and 320.  Here the rows travel through repack -> container -> device -> GEMV."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    words = np.zeros((2, 8), np.uint32)
    words[0, :] = 0x33333333      # 64 codes of 3, scale 1, bias 0  -> 192
    words[1, :] = 0x22222222      # 64 codes of 2, scale 2, bias 1  -> 320
    s = np.array([[0x3C00], [0x4000]], np.uint16); z = np.array([[0x0000], [0x3C00]], np.uint16)
    blocks = pkg.repack_mlx_to_staf(fmt, words, s, z, pkg.F16)
    path = str(tmp_path / "kat.staf")
    pkg.staf_write(path, [dict(name="test.weight", scheme_identifier=0x40, shape=[2, 8], payload=blocks.tobytes())], None)
    f = pkg.STAFFile(path)
    region = f.upload(ctx)
    for layout in (pkg.LAYOUT_STAF_BLOCKS, pkg.LAYOUT_PLANES):
        w = f.weight(ctx, "test.weight", layout, region)
        y = _gemv(ctx, pkg, w, np.ones(64, np.float32), 2)
        assert y[0] == 192.0 and y[1] == 320.0
        w.destroy()
    region.free(); f.close()
