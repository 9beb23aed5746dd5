"""The entry point that allocates nothing (mi355q_lmhead_argmax_static) against mi355q_lmhead_argmax: same kernels, the
partial keys in a device array of the library image instead of the context's allocation.  Two calls in a row, the
second on a smaller head, so that keys left by the first call sit behind the ones the second call uses."""
import numpy as np
import pytest

import oracle
from gpu_util import act_rounded, seeded_case
import kat

pytestmark = pytest.mark.gpu


def _head(pkg, ctx, fn, w, xd, n):
    logits = ctx.alloc(n * 4)
    tok = ctx.upload(np.array([-7], np.int32))
    fn(w, xd, pkg.BF16, logits, tok)
    ctx.synchronize()
    out = logits.download(np.float32), int(tok.download(np.int32)[0])
    logits.free(); tok.free()
    return out


@pytest.mark.parametrize("layout", ["LAYOUT_PLANES", "LAYOUT_TILE16", "LAYOUT_STAF_BLOCKS"])
def test_static_head_equals_head_on_two_calls_in_a_row(pkg, ctx, layout):
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    assert pkg.library().mi355q_lmhead_argmax_static_capacity() == 32768
    cases = []
    for seed, n, k in ((810, 32768, 2048), (820, 1536, 4096)):       # the second head is the smaller one
        words, s, z, wq = seeded_case(seed, n, k, 4, 64)
        w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, getattr(pkg, layout))
        x = act_rounded(kat.seeded_activations(seed + 1, 1, k), pkg.BF16, pkg)
        xd = ctx.upload(oracle.bf16_from_f32(x))
        cases.append((w, xd, n, oracle.gemm_f64(wq, x)[0]))
    # the two static calls back to back, nothing else in between
    got = [_head(pkg, ctx, ctx.lmhead_argmax_static, w, xd, n) for w, xd, n, _ in cases]
    ref = [_head(pkg, ctx, ctx.lmhead_argmax, w, xd, n) for w, xd, n, _ in cases]
    for (g_logits, g_tok), (r_logits, r_tok), (_, _, n, want) in zip(got, ref, cases):
        assert g_tok == r_tok == oracle.argmax_lowest(g_logits)
        assert np.array_equal(g_logits.view(np.uint32), r_logits.view(np.uint32))      # same kernels: bit for bit
        assert np.linalg.norm(g_logits - want) / np.linalg.norm(want) <= 1e-3
    # and once more in the other order: the larger head after the smaller one
    again = [_head(pkg, ctx, ctx.lmhead_argmax_static, w, xd, n) for w, xd, n, _ in reversed(cases)]
    for (g_logits, g_tok), (r_logits, r_tok) in zip(again, reversed(ref)):
        assert g_tok == r_tok and np.array_equal(g_logits.view(np.uint32), r_logits.view(np.uint32))
    for w, xd, _, _ in cases:
        w.destroy(); xd.free()


def test_static_head_refuses_more_workgroups_than_keys(pkg, ctx):
    """A head launch of more workgroups than the array has keys is an error, not a partial result."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    n, k = 32768 * 16 + 16, 64                          # K = 64: one K-step, 16 rows per workgroup -> 32769 workgroups
    rng = np.random.default_rng(3)
    words = rng.integers(0, 2**32, size=(n, k // 8), dtype=np.uint32)
    s = np.full((n, 1), 0x3C00, np.uint16); z = np.zeros((n, 1), np.uint16)
    w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.F16, pkg.LAYOUT_PLANES)
    xd = ctx.upload(oracle.bf16_from_f32(np.ones((1, k), np.float32)))
    tok = ctx.upload(np.array([-7], np.int32))
    with pytest.raises(pkg.MI355QError) as e:
        ctx.lmhead_argmax_static(w, xd, pkg.BF16, None, tok)
    assert "workgroups exceed 32768" in str(e.value)
    ctx.lmhead_argmax(w, xd, pkg.BF16, None, tok)       # the allocating entry point takes it
    ctx.synchronize()
    assert int(tok.download(np.int32)[0]) >= 0
    w.destroy(); xd.free(); tok.free()


@pytest.mark.parametrize("layout", ["LAYOUT_PLANES", "LAYOUT_TILE16", "LAYOUT_STAF_BLOCKS"])
def test_static_head_allocates_nothing_with_f16_and_fp32_activations(pkg, layout):
    """fp32 activations (and f16 ones on TILE16 records) reach mi355q_lmhead_argmax through routes that keep scratch in
    the context; the entry point that allocates nothing must not take them.  On a fresh context, whose scratch buffers
    do not exist yet: the context's scratch stays at zero bytes over both calls, the logits hold the bar against the
    oracle, and the token is the lowest-index maximum of the logits the call returned."""
    c = pkg.Context(0)
    try:
        fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
        for seed, n, k in ((830, 3000, 2048), (840, 520, 4096)):          # the second head is the smaller one
            words, s, z = oracle.quantize_affine(kat.seeded_weights(seed, n, k), 4, 64, oracle.F16)
            wq = oracle.dequant_planes_f32(4, 64, n, k, words, s, z, oracle.F16)
            w = c.weight_prepare_mlx(fmt, words, s, z, pkg.F16, getattr(pkg, layout))
            for xt, npdt in ((pkg.F32, np.float32), (pkg.F16, np.float16)):
                xa = kat.seeded_activations(seed + 1, 1, k).astype(npdt)
                xd = c.upload(xa.view(np.uint16) if xt == pkg.F16 else xa)
                logits, tok = c.alloc(n * 4), c.upload(np.array([-7], np.int32))
                before = c.scratch_bytes()
                c.lmhead_argmax_static(w, xd, xt, logits, tok)
                c.synchronize()
                assert c.scratch_bytes() == before == (0, 0, 0), "the entry point that allocates nothing grew the context's scratch"
                got, token = logits.download(np.float32), int(tok.download(np.int32)[0])
                want = oracle.gemm_f64(wq, xa.astype(np.float32))[0]
                assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-3
                assert token == oracle.argmax_lowest(got)
                for b in (xd, logits, tok):
                    b.free()
            w.destroy()
    finally:
        c.close()
