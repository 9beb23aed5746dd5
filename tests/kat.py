"""Known-answer generators shared by the CPU and GPU test suites.

Everything here is an *independent* formulation (Python big integers, numpy float16/float64):
it never calls the oracle or the HIP library, so it can pin both.  The parameters come from
``tests/golden/reference_kats.json`` (transcribed from the reference's own tests).
"""
from __future__ import annotations

import json
import os
from fractions import Fraction

import numpy as np

_GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_kats.json")

# every (bits, group) the reference registers, plus the two formats the benchmark adds (q6 g64, q2 g64)
REFERENCE_FORMATS = [(2, 16), (2, 32), (3, 16), (3, 32), (3, 64), (4, 64), (4, 128), (5, 32),
                     (5, 64), (6, 16), (6, 32), (8, 32), (8, 64), (8, 128)]
NEW_FORMATS = [(2, 64), (6, 64)]
ALL_FORMATS = REFERENCE_FORMATS + NEW_FORMATS

SCHEME_IDS = {(2, 16): 0x60, (2, 32): 0x61, (2, 64): 0x62, (3, 16): 0x50, (3, 32): 0x51,
              (3, 64): 0x52, (4, 64): 0x40, (4, 128): 0x41, (5, 32): 0x30, (5, 64): 0x31,
              (6, 16): 0x20, (6, 32): 0x21, (6, 64): 0x22, (8, 32): 0x10, (8, 64): 0x11,
              (8, 128): 0x12}


def load_kats() -> dict:
    with open(_GOLDEN) as f:
        return json.load(f)


def bytes_per_block(bits: int, group: int) -> int:
    return 4 + group * bits // 8


def pack_lsb_first(codes, bits: int) -> np.ndarray:
    """LSB-first bit stream via one big integer: stream = sum(code_k << (k*bits))."""
    acc = 0
    mask = (1 << bits) - 1
    for k, c in enumerate(codes):
        acc |= (int(c) & mask) << (k * bits)
    nbytes = (len(codes) * bits + 7) // 8
    return np.frombuffer(acc.to_bytes(nbytes, "little"), dtype=np.uint8).copy()


def unpack_lsb_first(stream: np.ndarray, n: int, bits: int) -> np.ndarray:
    acc = int.from_bytes(bytes(bytearray(stream.tolist())), "little")
    mask = (1 << bits) - 1
    return np.array([(acc >> (k * bits)) & mask for k in range(n)], dtype=np.uint8)


def f16_bits(v: float) -> int:
    return int(np.array([v], dtype=np.float16).view(np.uint16)[0])


def bf16_bits_exact(v: float) -> int:
    """bf16 bit pattern of a value that is exactly representable in bf16."""
    b = int(np.array([v], dtype=np.float32).view(np.uint32)[0])
    assert b & 0xFFFF == 0, f"{v} is not exactly representable in bf16"
    return b >> 16


def staf_blocks(codes: np.ndarray, scales: np.ndarray, zeros: np.ndarray, bits: int,
                group: int) -> np.ndarray:
    """codes [N,K] ints, scales/zeros [N,K/group] floats (exact in f16) -> STAF block bytes."""
    n, k = codes.shape
    bpr = k // group
    out = bytearray()
    for r in range(n):
        for b in range(bpr):
            out += int(f16_bits(scales[r, b])).to_bytes(2, "little")
            out += int(f16_bits(zeros[r, b])).to_bytes(2, "little")
            out += bytes(pack_lsb_first(codes[r, b * group:(b + 1) * group], bits).tolist())
    return np.frombuffer(bytes(out), dtype=np.uint8).copy()


def mlx_planes(codes: np.ndarray, bits: int) -> np.ndarray:
    """codes [N,K] -> uint32 [N, K*bits/32] (row bit streams viewed as little-endian words)."""
    n, k = codes.shape
    assert (k * bits) % 32 == 0
    rows = [pack_lsb_first(codes[r], bits) for r in range(n)]
    return np.stack(rows).view("<u4").reshape(n, k * bits // 32).copy()


def exact_gemv(codes, scales, zeros, x, group: int) -> np.ndarray:
    """sum_k (s*q+z)*x_k in exact rational arithmetic; codes [N,K], x [M,K] -> [M,N] float64."""
    n, k = codes.shape
    m = x.shape[0]
    y = np.zeros((m, n), dtype=np.float64)
    xf = [[Fraction(float(v)) for v in x[mi]] for mi in range(m)]
    for r in range(n):
        w = [Fraction(float(scales[r, c // group])) * int(codes[r, c]) +
             Fraction(float(zeros[r, c // group])) for c in range(k)]
        for mi in range(m):
            y[mi, r] = float(sum(wc * xc for wc, xc in zip(w, xf[mi])))
    return y


# ---- closed-form KAT generators (parameters: tests/golden/reference_kats.json) -------------

def single_block_case(bits: int, group: int, scale: float, zero: float):
    codes = np.array([[k % (1 << bits) for k in range(group)]], dtype=np.uint8)
    x = np.array([[(k % 10) * 0.125 - 0.5 for k in range(group)]], dtype=np.float16)
    return codes, np.array([[scale]]), np.array([[zero]]), x.astype(np.float32)


def multi_block_case(bits: int, group: int, blocks: int = 4):
    codes = np.array([[(k + 7 * b) % (1 << bits) for b in range(blocks) for k in range(group)]],
                     dtype=np.uint8)
    scales = np.array([[0.0625 * (b + 1) for b in range(blocks)]])
    zeros = np.array([[-0.25 + 0.125 * b for b in range(blocks)]])
    x = np.array([[(k % 11) * 0.0625 - 0.3 for k in range(group * blocks)]], dtype=np.float32)
    x = x.astype(np.float16).astype(np.float32)
    return codes, scales, zeros, x


def multi_row_case(bits: int, group: int, rows: int = 4, blocks: int = 4):
    codes = np.array([[(k + 7 * b + 3 * r) % (1 << bits) for b in range(blocks)
                       for k in range(group)] for r in range(rows)], dtype=np.uint8)
    scales = np.array([[0.0625 * (b + 1) + 0.015625 * r for b in range(blocks)]
                       for r in range(rows)])
    zeros = np.array([[-0.25 + 0.125 * b + 0.03125 * r for b in range(blocks)]
                      for r in range(rows)])
    x = np.array([[(k % 13) * 0.046875 - 0.25 for k in range(group * blocks)]], dtype=np.float32)
    x = x.astype(np.float16).astype(np.float32)
    return codes, scales, zeros, x


def roundtrip_case(bits, group, rows, blocks, scale_base, zero_base):
    mask = (1 << bits) - 1
    codes = np.array([[((r * 37 + b * 11 + i) & mask) for b in range(blocks)
                       for i in range(group)] for r in range(rows)], dtype=np.uint8)
    scales = np.array([[scale_base * (b + 1) for b in range(blocks)] for r in range(rows)])
    zeros = np.array([[zero_base + r * 0.125 for b in range(blocks)] for r in range(rows)])
    return codes, scales, zeros


# ---- seeded benchmark-style inputs -----------------------------------------------------------

def seeded_weights(seed: int, n: int, k: int) -> np.ndarray:
    """W ~ N(0, 0.02^2) fp32, PCG64-seeded."""
    rng = np.random.Generator(np.random.PCG64(seed))
    return (rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02)).astype(np.float32)


def seeded_activations(seed: int, m: int, k: int) -> np.ndarray:
    """x ~ N(0,1) fp32 (caller rounds to the I/O dtype)."""
    rng = np.random.Generator(np.random.PCG64(seed ^ 0x5EED))
    return rng.standard_normal((m, k), dtype=np.float32)


def random_codes(seed: int, n: int, k: int, bits: int) -> np.ndarray:
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.integers(0, 1 << bits, size=(n, k), dtype=np.uint8)
