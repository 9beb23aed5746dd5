"""Seeded sweep of odd shapes through every decode path (C ABI): row counts from one row to a few hundred, row
lengths that are one group, a few groups, one K-step plus a tail, activation batches of 1..8 rows, every format the
reference registry holds plus q6 g64 / q2 g64, on STAF blocks (in place), planes and TILE16 records.  Each result is
held to the path's bars (relative L2 <= 1e-3, max-abs <= 2e-2 against an fp64 accumulation of the same dequantised
weights).  The launch heuristics pick different kernels, wavefront counts, ring depths and rows per wavefront across
these shapes; none of them may read or write outside its buffers (the outputs sit between NaN canaries)."""
import sys

import numpy as np
import pytest

import kat
import oracle
from gpu_util import act_rounded, assert_within_tolerance, out_from_device, seeded_case

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, file=sys.stderr, flush=True)


def _run_with_canaries(pkg, ctx, w, x, n):
    """y [M, N] fp32, written into the middle of a larger NaN-filled buffer: the margins must stay untouched."""
    m, k = x.shape
    margin = 64
    xd = ctx.upload(oracle.bf16_from_f32(x).reshape(x.shape))
    total = margin + m * n + margin
    yd = ctx.alloc(total * 4)
    ctx.fill(yd, 0x7FC00000)
    ctx.qgemm(w, xd, pkg.BF16, yd.ptr + margin * 4, pkg.F32, m)
    ctx.synchronize()
    raw = yd.download(np.float32, (total,))
    xd.free(); yd.free()
    assert np.all(np.isnan(raw[:margin])) and np.all(np.isnan(raw[margin + m * n:])), "wrote outside the output"
    return raw[margin:margin + m * n].reshape(m, n)


@pytest.mark.parametrize("chunk", range(24))
def test_seeded_shape_sweep(pkg, ctx, chunk):
    rng = np.random.default_rng(9000 + chunk)
    formats = list(kat.ALL_FORMATS)
    for case in range(14):
        bits, group = formats[int(rng.integers(len(formats)))]
        unit = group * (32 // int(np.gcd(32, group * bits)))            # K such that a row is whole 32-bit words
        kind = int(rng.integers(4))
        if kind == 0:
            k = unit * int(rng.integers(1, 4))
        elif kind == 1:
            k = unit * int(rng.integers(4, 24))
        elif kind == 2:
            k = 2048 + unit * int(rng.integers(0, 5))
        else:
            k = 256 * int(rng.integers(1, 30))
            k = (k + unit - 1) // unit * unit
        n = int(rng.choice([1, 2, 3, 15, 16, 17, 63, 64, 65, int(rng.integers(66, 400))]))
        m = int(rng.integers(1, 9))                                     # 1..8: the decode kernels (larger batches are the GEMM's)
        words, s, z, wq = seeded_case(9100 + 100 * chunk + case, n, k, bits, group)
        fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(bits, group)
        x = act_rounded(kat.seeded_activations(9200 + case, m, k), pkg.BF16, pkg)
        want = oracle.gemm_f64(wq, x)
        layouts = [pkg.LAYOUT_STAF_BLOCKS, pkg.LAYOUT_PLANES]
        if (bits, group) == (4, 64) and k % 128 == 0:
            layouts.append(pkg.LAYOUT_TILE16)
        for layout in layouts:
            say(f"sweep chunk {chunk} case {case}: q{bits}g{group} N={n} K={k} M={m} layout {layout}")
            w = ctx.weight_prepare_mlx(fmt, words, s, z, pkg.BF16, layout)
            got = _run_with_canaries(pkg, ctx, w, x, n)
            assert_within_tolerance(got, want, f"q{bits}g{group} N={n} K={k} M={m} layout {layout}")
            w.destroy()
