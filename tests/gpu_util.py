"""Helpers for the GPU parity tests: build packed weights in either layout, run launches through
the C ABI, and compare against the CPU oracle with the tolerances the path is specified with."""
from __future__ import annotations

import numpy as np

import kat
import oracle

# fp results: relative L2 <= 1e-3 and max-abs <= 2e-2 against an fp64 accumulation of the same
# dequantised weights (the path's stated tolerance)
REL_L2_TOL = 1e-3
MAX_ABS_TOL = 2e-2


def rel_l2(got, want) -> float:
    got = np.asarray(got, np.float64); want = np.asarray(want, np.float64)
    den = np.linalg.norm(want)
    return float(np.linalg.norm(got - want) / den) if den else float(np.linalg.norm(got - want))


def assert_within_tolerance(got, want, what=""):
    got = np.asarray(got, np.float64); want = np.asarray(want, np.float64)
    assert np.all(np.isfinite(got)), what
    r, a = rel_l2(got, want), float(np.max(np.abs(got - want)))
    assert r <= REL_L2_TOL and a <= MAX_ABS_TOL, f"{what}: rel-L2 {r:.3e}, max-abs {a:.3e}"
    return r, a


def act_to_device_array(x_f32: np.ndarray, dtype: int, pkg) -> np.ndarray:
    """fp32 activations -> host array in the I/O dtype (bf16/f16 as uint16 bit patterns)."""
    if dtype == pkg.BF16:
        return oracle.bf16_from_f32(x_f32).reshape(x_f32.shape)
    if dtype == pkg.F16:
        return x_f32.astype(np.float16).view(np.uint16)
    return x_f32.astype(np.float32)


def act_rounded(x_f32: np.ndarray, dtype: int, pkg) -> np.ndarray:
    """The fp32 value the device sees after rounding to the I/O dtype."""
    if dtype == pkg.BF16:
        return oracle.bf16_to_f32(oracle.bf16_from_f32(x_f32)).reshape(x_f32.shape)
    if dtype == pkg.F16:
        return x_f32.astype(np.float16).astype(np.float32)
    return x_f32.astype(np.float32)


def out_from_device(buf, dtype: int, shape, pkg) -> np.ndarray:
    if dtype == pkg.F32:
        return buf.download(np.float32, shape)
    raw = buf.download(np.uint16, shape)
    if dtype == pkg.BF16:
        return oracle.bf16_to_f32(raw).reshape(shape)
    return raw.view(np.float16).astype(np.float32)


class Case:
    """A packed weight in host form: codes [N,K] plus per-group scale/zero as exact floats."""

    def __init__(self, bits, group, codes, scales, zeros):
        self.bits, self.group = bits, group
        self.codes = np.ascontiguousarray(codes, np.uint8)
        self.scales = np.asarray(scales, np.float64)
        self.zeros = np.asarray(zeros, np.float64)
        self.n, self.k = self.codes.shape

    def staf_blocks(self):
        return kat.staf_blocks(self.codes, self.scales, self.zeros, self.bits, self.group)

    def planes(self, sb_dtype, pkg):
        words = kat.mlx_planes(self.codes, self.bits)
        if sb_dtype == pkg.BF16:
            s = oracle.bf16_from_f32(self.scales.astype(np.float32)).reshape(self.scales.shape)
            z = oracle.bf16_from_f32(self.zeros.astype(np.float32)).reshape(self.zeros.shape)
            assert np.array_equal(oracle.bf16_to_f32(s).reshape(self.scales.shape), self.scales.astype(np.float32))
        else:
            s = self.scales.astype(np.float16).view(np.uint16)
            z = self.zeros.astype(np.float16).view(np.uint16)
        return words, s, z

    def device_weight(self, ctx, pkg, layout, sb_dtype=None):
        fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(self.bits, self.group)
        if layout == pkg.LAYOUT_STAF_BLOCKS:
            return ctx.weight_prepare_staf(fmt, self.n, self.k, self.staf_blocks(), pkg.LAYOUT_STAF_BLOCKS)
        sb = pkg.F16 if sb_dtype is None else sb_dtype
        words, s, z = self.planes(sb, pkg)
        return ctx.weight_prepare_mlx(fmt, words, s, z, sb, pkg.LAYOUT_PLANES)

    def planes_eligible(self):
        return (self.k * self.bits) % 32 == 0


def run_gemv(ctx, pkg, w, x_f32, x_dtype, y_dtype, flags=0, x_stride=None, use_qgemm=False):
    """x_f32 [M, stride] -> y [M, N] as float32 (after the device's output rounding)."""
    m, stride = x_f32.shape
    info = w.info
    n = int(info.n_rows)
    xd = ctx.upload(act_to_device_array(x_f32, x_dtype, pkg))
    yd = ctx.alloc(m * n * (4 if y_dtype == pkg.F32 else 2))
    ctx.fill(yd, 0x7FC07FC0 if y_dtype != pkg.F32 else 0x7FC00000)      # NaN canary
    fn = ctx.qgemm if use_qgemm else ctx.qgemv
    fn(w, xd, x_dtype, yd, y_dtype, m, stride if x_stride is None else x_stride, 0, flags)
    ctx.synchronize()
    y = out_from_device(yd, y_dtype, (m, n), pkg)
    xd.free(); yd.free()
    return y


def seeded_case(seed, n, k, bits, group):
    """benchmark-style tensors: W ~ N(0, 0.02^2) quantised per group to bf16 scale/bias planes.
    Returns (codes_words, scales_bf16, biases_bf16, dequantised fp32 weights)."""
    w = kat.seeded_weights(seed, n, k)
    words, s, z = oracle.quantize_affine(w, bits, group, oracle.BF16)
    wq = oracle.dequant_planes_f32(bits, group, n, k, words, s, z, oracle.BF16)
    return words, s, z, wq
