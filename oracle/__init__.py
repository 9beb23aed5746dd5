"""ctypes/numpy front end of the CPU oracle -- TEST INFRASTRUCTURE ONLY.

Only the test suite, the smoke check and the benchmark's CPU-baseline leg import this
module; the shipped library never does.  The arithmetic lives in ``qlin_oracle.c`` (each
function there cites the reference file:line it restates); this file only marshals numpy
arrays.  ``build()`` compiles the C file with gcc into ``oracle/_build``.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libqlin_oracle.so")
_lib = None

F16, BF16, F32 = 0, 1, 2
_SB_NP = {F16: np.uint16, BF16: np.uint16, F32: np.float32}


class Format(C.Structure):
    _fields_ = [("scheme", C.c_int32), ("bits", C.c_int32), ("group", C.c_int32),
                ("bytes_per_block", C.c_int32), ("in_reference", C.c_int32)]


def build(force: bool = False) -> str:
    """Compile the C oracle (gcc).  Returns the path of the shared object."""
    src = os.path.join(_HERE, "qlin_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        vp, sz, i32 = C.c_void_p, C.c_size_t, C.c_int
        L.orc_format_for_mlx.argtypes = [i32, i32, C.POINTER(Format)]
        L.orc_format_for_scheme.argtypes = [i32, C.POINTER(Format)]
        L.orc_bf16_from_f32.argtypes = [C.c_float]; L.orc_bf16_from_f32.restype = C.c_uint16
        L.orc_bf16_to_f32.argtypes = [C.c_uint16]; L.orc_bf16_to_f32.restype = C.c_float
        L.orc_f16_from_f32.argtypes = [C.c_float]; L.orc_f16_from_f32.restype = C.c_uint16
        L.orc_f16_to_f32.argtypes = [C.c_uint16]; L.orc_f16_to_f32.restype = C.c_float
        L.orc_unpack_code.argtypes = [vp, i32, i32]; L.orc_unpack_code.restype = C.c_uint32
        L.orc_unpack_code_stream.argtypes = [vp, sz, i32]; L.orc_unpack_code_stream.restype = C.c_uint32
        L.orc_pack_stream.argtypes = [vp, sz, i32, vp]; L.orc_pack_stream.restype = None
        L.orc_repack_mlx_to_staf.argtypes = [i32, i32, sz, sz, vp, vp, vp, i32, vp]
        L.orc_staf_to_planes.argtypes = [i32, i32, sz, sz, vp, vp, vp, vp]
        L.orc_unpack_staf_codes.argtypes = [i32, i32, sz, sz, vp, vp]
        L.orc_unpack_plane_codes.argtypes = [i32, sz, sz, vp, vp]
        L.orc_dequant_staf_f32.argtypes = [i32, i32, sz, sz, vp, vp]
        L.orc_dequant_planes_f32.argtypes = [i32, i32, sz, sz, vp, vp, vp, i32, vp]
        L.orc_dequant_staf_bf16.argtypes = [i32, i32, sz, sz, vp, vp]
        L.orc_embedding_lookup_staf_f32.argtypes = [i32, i32, sz, sz, vp, vp, sz, i32, C.c_float, vp]
        L.orc_kv_quant_bits.argtypes = [i32]; L.orc_kv_quant_group.argtypes = [i32]
        L.orc_kv_bytes_per_head_slot.argtypes = [i32, sz]; L.orc_kv_bytes_per_head_slot.restype = sz
        L.orc_kv_write_slot.argtypes = [i32, vp, sz, vp]; L.orc_kv_read_slot.argtypes = [i32, vp, sz, vp]
        L.orc_kv_slot_offset.argtypes = [i32, sz, sz, sz, sz, sz]; L.orc_kv_slot_offset.restype = sz
        L.orc_gemm_f64.argtypes = [vp, vp, sz, sz, sz, sz, vp]; L.orc_gemm_f64.restype = None
        L.orc_qgemm_staf_ref_f32.argtypes = [i32, i32, vp, vp, sz, sz, sz, sz, vp, i32]
        L.orc_qgemm_planes_ref_f32.argtypes = [i32, i32, vp, vp, vp, i32, vp, sz, sz, sz, sz, vp, i32]
        L.orc_argmax_lowest.argtypes = [vp, sz]; L.orc_argmax_lowest.restype = C.c_int32
        L.orc_gated_activation_f32.argtypes = [vp, vp, sz, i32, i32, vp]; L.orc_gated_activation_f32.restype = None
        L.orc_quantize_affine.argtypes = [vp, sz, sz, i32, i32, i32, vp, vp, vp]
        _lib = L
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def _check(rc: int, what: str):
    if rc != 0:
        raise ValueError(f"oracle.{what} failed with code {rc}")


# ------------------------------------------------------------------ formats
def format_for_mlx(bits: int, group: int):
    f = Format()
    return f if lib().orc_format_for_mlx(bits, group, C.byref(f)) == 0 else None


def format_for_scheme(scheme: int):
    f = Format()
    return f if lib().orc_format_for_scheme(scheme, C.byref(f)) == 0 else None


def bytes_per_block(bits: int, group: int) -> int:
    return 4 + group * bits // 8


# ------------------------------------------------------------ float formats
def bf16_from_f32(a) -> np.ndarray:
    """Round-to-nearest-even float32 -> bf16 bit patterns (vectorised twin of orc_bf16_from_f32)."""
    bits = _c(a, np.float32).view(np.uint32)
    lsb = (bits >> np.uint32(16)) & np.uint32(1)
    with np.errstate(over="ignore"):
        r = bits + np.uint32(0x7FFF) + lsb
    return (r >> np.uint32(16)).astype(np.uint16)


def bf16_to_f32(h) -> np.ndarray:
    return (_c(h, np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def f16_from_f32_scalar(v: float) -> int:
    return int(lib().orc_f16_from_f32(float(np.float32(v))))


def f16_to_f32_scalar(h: int) -> float:
    return float(lib().orc_f16_to_f32(int(h)))


def bf16_from_f32_scalar(v: float) -> int:
    return int(lib().orc_bf16_from_f32(float(np.float32(v))))


# ----------------------------------------------------------- pack / unpack
def pack_stream(codes, bits: int) -> np.ndarray:
    codes = _c(codes, np.uint8).ravel()
    out = np.zeros((codes.size * bits + 7) // 8, dtype=np.uint8)
    lib().orc_pack_stream(_p(codes), codes.size, bits, _p(out))
    return out


def unpack_code(qs, k: int, bits: int) -> int:
    qs = _c(qs, np.uint8)
    return int(lib().orc_unpack_code(_p(qs), k, bits))


def unpack_code_stream(qs, k: int, bits: int) -> int:
    qs = _c(qs, np.uint8)
    return int(lib().orc_unpack_code_stream(_p(qs), k, bits))


def repack_mlx_to_staf(bits, group, codes, scales, biases, sb_dtype) -> np.ndarray:
    """codes uint32 [N, K*bits/32]; scales/biases [N, K/group] in sb_dtype -> STAF block bytes."""
    codes = _c(codes, np.uint32)
    n, packed = codes.shape
    scales = _c(scales, _SB_NP[sb_dtype]); biases = _c(biases, _SB_NP[sb_dtype])
    k = packed * 32 // bits
    out = np.zeros(n * (k // group) * bytes_per_block(bits, group), dtype=np.uint8)
    _check(lib().orc_repack_mlx_to_staf(bits, group, n, packed, _p(codes), _p(scales), _p(biases),
                                        sb_dtype, _p(out)), "repack_mlx_to_staf")
    return out


def staf_to_planes(bits, group, n, k, blocks):
    blocks = _c(blocks, np.uint8)
    codes = np.zeros((n, k * bits // 32), dtype=np.uint32)
    s = np.zeros((n, k // group), dtype=np.uint16)
    z = np.zeros((n, k // group), dtype=np.uint16)
    _check(lib().orc_staf_to_planes(bits, group, n, k, _p(blocks), _p(codes), _p(s), _p(z)),
           "staf_to_planes")
    return codes, s, z


def unpack_staf_codes(bits, group, n, k, blocks) -> np.ndarray:
    blocks = _c(blocks, np.uint8)
    out = np.zeros((n, k), dtype=np.uint8)
    _check(lib().orc_unpack_staf_codes(bits, group, n, k, _p(blocks), _p(out)), "unpack_staf_codes")
    return out


def unpack_plane_codes(bits, n, k, codes) -> np.ndarray:
    codes = _c(codes, np.uint32)
    out = np.zeros((n, k), dtype=np.uint8)
    _check(lib().orc_unpack_plane_codes(bits, n, k, _p(codes), _p(out)), "unpack_plane_codes")
    return out


# ------------------------------------------------------------------ dequant
def dequant_staf_f32(bits, group, n, k, blocks) -> np.ndarray:
    blocks = _c(blocks, np.uint8)
    out = np.zeros((n, k), dtype=np.float32)
    _check(lib().orc_dequant_staf_f32(bits, group, n, k, _p(blocks), _p(out)), "dequant_staf_f32")
    return out


def dequant_planes_f32(bits, group, n, k, codes, scales, biases, sb_dtype) -> np.ndarray:
    codes = _c(codes, np.uint32)
    scales = _c(scales, _SB_NP[sb_dtype]); biases = _c(biases, _SB_NP[sb_dtype])
    out = np.zeros((n, k), dtype=np.float32)
    _check(lib().orc_dequant_planes_f32(bits, group, n, k, _p(codes), _p(scales), _p(biases),
                                        sb_dtype, _p(out)), "dequant_planes_f32")
    return out


def dequant_staf_bf16(bits, group, n, k, blocks) -> np.ndarray:
    blocks = _c(blocks, np.uint8)
    out = np.zeros((n, k), dtype=np.uint16)
    _check(lib().orc_dequant_staf_bf16(bits, group, n, k, _p(blocks), _p(out)), "dequant_staf_bf16")
    return out


# --------------------------------------------------------------------- gemm
def embedding_lookup_staf_f32(bits, group, vocab, dim, table, token_ids, embedding_scale=None) -> np.ndarray:
    table = _c(table, np.uint8)
    ids = _c(token_ids, np.int32)
    out = np.zeros((ids.size, dim), dtype=np.float32)
    _check(lib().orc_embedding_lookup_staf_f32(bits, group, vocab, dim, _p(table), _p(ids), ids.size,
                                               0 if embedding_scale is None else 1,
                                               0.0 if embedding_scale is None else float(embedding_scale), _p(out)),
           "embedding_lookup_staf_f32")
    return out


# --------------------------------------------------------------------- KV cache
def kv_bytes_per_head_slot(scheme: int, head_dim: int) -> int:
    return int(lib().orc_kv_bytes_per_head_slot(scheme, head_dim))


def kv_write_slot(scheme: int, src, slot=None) -> np.ndarray:
    """Quantise one head vector into a slot (a fresh zeroed slot unless one is given)."""
    src = _c(src, np.float32)
    if slot is None:
        slot = np.zeros(kv_bytes_per_head_slot(scheme, src.size), np.uint8)
    _check(lib().orc_kv_write_slot(scheme, _p(src), src.size, _p(slot)), "kv_write_slot")
    return slot


def kv_read_slot(scheme: int, slot, head_dim: int) -> np.ndarray:
    slot = _c(slot, np.uint8)
    out = np.zeros(head_dim, np.float32)
    _check(lib().orc_kv_read_slot(scheme, _p(slot), head_dim, _p(out)), "kv_read_slot")
    return out


def kv_cache_write(scheme, layout_mode, kv_heads, head_dim, max_positions, src, first_position, cache=None):
    """src [positions, kv_heads * head_dim] fp32 -> cache bytes; the reference's fill loop
    (MC/Generator/MetalSourceGenerator+Attention.swift:1233-1250, slot addressing :762-769)."""
    src = _c(src, np.float32).reshape(-1, kv_heads * head_dim)
    slot = kv_bytes_per_head_slot(scheme, head_dim)
    if cache is None:
        cache = np.zeros(kv_heads * max_positions * slot, np.uint8)
    for p in range(src.shape[0]):
        for h in range(kv_heads):
            off = int(lib().orc_kv_slot_offset(layout_mode, h, first_position + p, kv_heads, max_positions, slot))
            kv_write_slot(scheme, src[p, h * head_dim:(h + 1) * head_dim], cache[off:off + slot])
    return cache


def kv_cache_read(scheme, layout_mode, kv_heads, head_dim, max_positions, cache, first_position, count):
    cache = _c(cache, np.uint8)
    slot = kv_bytes_per_head_slot(scheme, head_dim)
    out = np.zeros((count, kv_heads * head_dim), np.float32)
    for p in range(count):
        for h in range(kv_heads):
            off = int(lib().orc_kv_slot_offset(layout_mode, h, first_position + p, kv_heads, max_positions, slot))
            out[p, h * head_dim:(h + 1) * head_dim] = kv_read_slot(scheme, cache[off:off + slot], head_dim)
    return out


def gemm_f64(w, x, x_stride=None) -> np.ndarray:
    """fp64 accumulation of fp32 weights w [N,K] against x [M, x_stride>=K] -> y [M,N] float64."""
    w = _c(w, np.float32); x = _c(x, np.float32)
    n, k = w.shape
    m = x.shape[0]
    stride = x.shape[1] if x_stride is None else x_stride
    y = np.zeros((m, n), dtype=np.float64)
    lib().orc_gemm_f64(_p(w), _p(x), m, n, k, stride, _p(y))
    return y


def qgemm_staf_ref_f32(bits, group, blocks, x, n, k, threads=1) -> np.ndarray:
    blocks = _c(blocks, np.uint8); x = _c(x, np.float32)
    m, stride = x.shape
    y = np.zeros((m, n), dtype=np.float32)
    _check(lib().orc_qgemm_staf_ref_f32(bits, group, _p(blocks), _p(x), m, n, k, stride, _p(y),
                                        threads), "qgemm_staf_ref_f32")
    return y


def qgemm_planes_ref_f32(bits, group, codes, scales, biases, sb_dtype, x, n, k, threads=1):
    codes = _c(codes, np.uint32); x = _c(x, np.float32)
    scales = _c(scales, _SB_NP[sb_dtype]); biases = _c(biases, _SB_NP[sb_dtype])
    m, stride = x.shape
    y = np.zeros((m, n), dtype=np.float32)
    _check(lib().orc_qgemm_planes_ref_f32(bits, group, _p(codes), _p(scales), _p(biases), sb_dtype,
                                          _p(x), m, n, k, stride, _p(y), threads),
           "qgemm_planes_ref_f32")
    return y


SILU, GELU_TANH = 0, 1


def gated_activation_f32(gate, up, kind=SILU, dtype=F32):
    """activation(T(gate)) * T(up), rounded to T: the gated MLP's elementwise step, fp32 arithmetic."""
    gate = _c(gate, np.float32); up = _c(up, np.float32)
    out = np.zeros(gate.shape, np.float32)
    lib().orc_gated_activation_f32(_p(gate), _p(up), gate.size, kind, dtype, _p(out))
    return out


def argmax_lowest(v) -> int:
    v = _c(v, np.float32).ravel()
    return int(lib().orc_argmax_lowest(_p(v), v.size))


# ---------------------------------------------------------------- quantizer
def quantize_affine(w, bits, group, sb_dtype=BF16):
    """fp32 [N,K] -> (codes uint32 [N, K*bits/32], scales, biases [N, K/group] in sb_dtype)."""
    w = _c(w, np.float32)
    n, k = w.shape
    codes = np.zeros((n, k * bits // 32), dtype=np.uint32)
    s = np.zeros((n, k // group), dtype=_SB_NP[sb_dtype])
    z = np.zeros((n, k // group), dtype=_SB_NP[sb_dtype])
    _check(lib().orc_quantize_affine(_p(w), n, k, bits, group, sb_dtype, _p(codes), _p(s), _p(z)),
           "quantize_affine")
    return codes, s, z
