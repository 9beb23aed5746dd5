"""Host-side mirror (Python/ctypes) of the quantized-linear interface over libmi355_qlinear.so.

The names follow the reference's planner/encoder contract (QuantizationFormat,
QuantizationFormatRegistry, STAFWeightLayout, dispatch steps, quantization-plan entries); the
arithmetic all happens in the HIP library.  There is no CPU fallback: loading fails loudly when
the shared library is missing, and creating a ``Context`` fails when there is no MI355X.
"""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmi355_qlinear.so")

# BufferPrecision
F16, BF16, F32 = 0, 1, 2
# STAFWeightLayout
LAYOUT_STAF_BLOCKS, LAYOUT_PLANES, LAYOUT_TILE16 = 0, 1, 2
# launch flags
FLAG_NONE, FLAG_FORCE_GENERIC, FLAG_FORCE_SMALL_M, FLAG_FORCE_MFMA, FLAG_PROBE_CLOCK, FLAG_FORCE_TWO_STEP = 0, 1, 2, 4, 8, 16
FLAG_FORCE_STREAM = 32
GATED_SILU, GATED_GELU_TANH = 0, 1      # ElementwiseKind .swiglu / .geluGated
FLAG_PROBE_TILED = 64      # measurement aid: the tiled fused kernel where the wide-tile one would be taken
FLAG_PROBE_WIDE = 128      # ... the wide-tile kernel wherever it reads the weight, whatever the size

STATUS_NAMES = {0: "OK", -1: "INVALID_ARGUMENT", -2: "UNSUPPORTED_FORMAT", -3: "SHAPE", -4: "NULL_HANDLE",
                -5: "DEVICE", -6: "OUT_OF_MEMORY", -7: "KERNEL_NOT_FOUND", -8: "SIZE_MISMATCH",
                -9: "INVALID_FILE", -10: "IO", -11: "NOT_FOUND"}
FALLBACK_NAMES = {0: None, 1: "inputStrideMismatch", 2: "lastTokenProjectionUsesDecodeKernel",
                  3: "disabledByEnvironment", 4: "unavailableAcceleration"}
PATH_NAMES = {0: "prefillProjection", 1: "decodeProjection"}
FAMILY_NAMES = {0: "generic", 1: "largeDense", 2: "input2048SquareDense", 3: "input20486144Dense",
                4: "input20488192Dense", 5: "input2048ExpandedDense", 6: "input8192Tiled", 7: "vocabDense"}


def probe_route(fmt, layout, n, k, x_dtype, m, flags=0, decode_entry=False, library_available=True, sb_dtype=None,
                x_row_stride=0):
    """The route table on a synthetic weight (no device needed): (what the launcher would run, what the plan names)."""
    a = C.create_string_buffer(128)
    b = C.create_string_buffer(128)
    _check(library().mi355q_probe_route(fmt.scheme_identifier, layout, BF16 if sb_dtype is None else sb_dtype, n, k, x_dtype, m,
                                        x_row_stride, flags, int(decode_entry), int(library_available), a, b, 128))
    return a.value.decode(), b.value.decode()


def probe_shared_route(fmt, layout, ns, k, x_dtype, m, flags=0, sb_dtype=None, x_row_stride=0):
    """The same for two or three projections of ns rows that share their activations: (what mi355q_batched_qgemm would
    run, the device kernel the plan record of the shared step names)."""
    a = C.create_string_buffer(128)
    b = C.create_string_buffer(128)
    rows = (C.c_uint64 * len(ns))(*ns)
    _check(library().mi355q_probe_shared_route(fmt.scheme_identifier, layout, BF16 if sb_dtype is None else sb_dtype, len(ns), rows,
                                               k, x_dtype, m, x_row_stride, flags, a, b, 128))
    return a.value.decode(), b.value.decode()


class MI355QError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"[{STATUS_NAMES.get(status, status)}] {message}")
        self.status = status
        self.status_name = STATUS_NAMES.get(status, str(status))


class _Format(C.Structure):
    _fields_ = [("scheme_identifier", C.c_uint8), ("bits", C.c_uint8), ("is_quantized", C.c_uint8),
                ("is_aligned", C.c_uint8), ("group_size", C.c_uint32), ("weights_per_block", C.c_uint32),
                ("bytes_per_block", C.c_uint32), ("has_direct_gemm", C.c_uint8),
                ("batched_gemm_counts", C.c_uint8), ("in_reference_registry", C.c_uint8),
                ("reserved0", C.c_uint8), ("direct_gemm_threadgroup_memory_length", C.c_uint32),
                ("block_struct_name", C.c_char * 32), ("gemv_kernel_name", C.c_char * 32),
                ("gemm_kernel_name_f32s", C.c_char * 32), ("gemm_kernel_name", C.c_char * 32),
                ("dequant_to_bfloat_kernel_name", C.c_char * 32), ("embedding_lookup_token", C.c_char * 16)]


class _StafEntry(C.Structure):
    _fields_ = [("name", C.c_void_p), ("name_length", C.c_uint32), ("scheme_identifier", C.c_uint8),
                ("semantic_role", C.c_uint8), ("original_dtype", C.c_uint8), ("dimension_count", C.c_uint8),
                ("shape", C.c_uint32 * 8), ("payload_offset", C.c_uint64), ("payload_size", C.c_uint64),
                ("buffer_offset", C.c_uint64), ("alignment", C.c_uint32), ("block_size", C.c_uint32),
                ("group_size", C.c_uint32), ("checksum", C.c_uint32), ("shard_index", C.c_uint32)]


class _StafMetadata(C.Structure):
    _fields_ = [("key", C.c_char_p), ("type", C.c_uint8), ("payload0", C.c_uint64), ("text", C.c_void_p),
                ("text_length", C.c_uint32)]


class _StafTensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("scheme_identifier", C.c_uint8), ("semantic_role", C.c_uint8),
                ("original_dtype", C.c_uint8), ("dimension_count", C.c_uint32), ("shape", C.c_uint32 * 8),
                ("payload", C.c_void_p), ("payload_size", C.c_uint64), ("shard_index", C.c_uint32)]


class _KvLayout(C.Structure):
    _fields_ = [("scheme", C.c_uint8), ("layout_mode", C.c_uint8), ("reserved0", C.c_uint16),
                ("kv_head_count", C.c_uint32), ("head_dimension", C.c_uint32),
                ("maximum_sequence_length", C.c_uint32), ("head_slot_bytes", C.c_uint32)]


class _DeviceInfo(C.Structure):
    _fields_ = [("name", C.c_char * 64), ("arch", C.c_char * 32), ("compute_units", C.c_int32),
                ("wavefront_size", C.c_int32), ("lds_bytes_per_workgroup", C.c_int32), ("reserved0", C.c_int32),
                ("hbm_bytes", C.c_uint64), ("hbm_peak_gbps", C.c_double), ("mfma_bf16_peak_tflops", C.c_double)]


class _WeightInfo(C.Structure):
    _fields_ = [("scheme_identifier", C.c_uint8), ("bits", C.c_uint8), ("layout", C.c_uint8),
                ("sb_dtype", C.c_uint8), ("group_size", C.c_uint32), ("n_rows", C.c_uint64), ("k", C.c_uint64),
                ("weight_bytes", C.c_uint64), ("blocks_dev", C.c_void_p), ("codes_dev", C.c_void_p),
                ("scales_dev", C.c_void_p), ("biases_dev", C.c_void_p), ("owns_memory", C.c_uint8),
                ("reserved", C.c_uint8 * 7)]


class _Step(C.Structure):
    _fields_ = [("kernel_name", C.c_char * 48), ("device_kernel", C.c_char * 48), ("kernel_family", C.c_char * 32),
                ("grid", C.c_uint32 * 3), ("block", C.c_uint32 * 3), ("lds_bytes", C.c_uint32),
                ("rows_per_workgroup", C.c_uint32), ("reference_simdgroups", C.c_uint32),
                ("reference_tile_elements", C.c_uint32), ("shape_family", C.c_int32), ("path", C.c_int32),
                ("scheme_identifier", C.c_uint8), ("layout", C.c_uint8), ("used_fallback", C.c_uint8),
                ("fallback_reason", C.c_uint8), ("input_dimension", C.c_uint32), ("output_dimension", C.c_uint32),
                ("sequence_length", C.c_uint32), ("input_row_stride", C.c_uint32), ("weight_bytes", C.c_uint64),
                ("flops", C.c_uint64)]


_lib = None


def library() -> C.CDLL:
    """Load the HIP shared library; raise (never fall back) when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is missing: build it with `python swift-mlx-lm_amd/build.py` "
                          "(there is no CPU implementation to fall back to)")
    L = C.CDLL(LIB_PATH)
    vp, u32, u64, u8, i32, sz = C.c_void_p, C.c_uint32, C.c_uint64, C.c_uint8, C.c_int32, C.c_size_t
    P = C.POINTER
    sig = {
        "mi355q_last_error": (C.c_char_p, []),
        "mi355q_abi_version": (i32, []),
        "mi355q_format_for_mlx_quantization": (i32, [C.c_int, C.c_int, P(_Format)]),
        "mi355q_format_for_scheme": (i32, [u8, P(_Format)]),
        "mi355q_format_count": (i32, []),
        "mi355q_format_at": (i32, [i32, P(_Format)]),
        "mi355q_bf16_from_f32": (C.c_uint16, [C.c_float]),
        "mi355q_repack_mlx_to_staf": (i32, [u8, sz, sz, vp, vp, vp, C.c_int, vp, sz]),
        "mi355q_context_create": (i32, [C.c_int, P(vp)]),
        "mi355q_context_destroy": (i32, [vp]),
        "mi355q_device_query": (i32, [vp, P(_DeviceInfo)]),
        "mi355q_context_set_library_use": (i32, [vp, C.c_int]),
        "mi355q_buffer_alloc": (i32, [vp, sz, P(vp)]),
        "mi355q_buffer_free": (i32, [vp, vp]),
        "mi355q_buffer_upload": (i32, [vp, vp, vp, sz]),
        "mi355q_buffer_download": (i32, [vp, vp, vp, sz]),
        "mi355q_buffer_fill": (i32, [vp, vp, vp, u32, sz]),
        "mi355q_stream_create": (i32, [vp, P(vp)]),
        "mi355q_stream_destroy": (i32, [vp, vp]),
        "mi355q_stream_synchronize": (i32, [vp, vp]),
        "mi355q_event_create": (i32, [vp, P(vp)]),
        "mi355q_event_destroy": (i32, [vp, vp]),
        "mi355q_event_record": (i32, [vp, vp, vp]),
        "mi355q_event_synchronize": (i32, [vp, vp]),
        "mi355q_event_elapsed_ms": (i32, [vp, vp, vp, P(C.c_float)]),
        "mi355q_weight_prepare_mlx": (i32, [vp, u8, u64, u64, vp, vp, vp, C.c_int, C.c_int, P(vp)]),
        "mi355q_weight_prepare_staf": (i32, [vp, u8, u64, u64, vp, sz, C.c_int, P(vp)]),
        "mi355q_weight_wrap_staf": (i32, [vp, u8, u64, u64, vp, sz, P(vp)]),
        "mi355q_weight_wrap_planes": (i32, [vp, u8, u64, u64, vp, vp, vp, C.c_int, P(vp)]),
        "mi355q_weight_query": (i32, [vp, P(_WeightInfo)]),
        "mi355q_weight_destroy": (i32, [vp]),
        "mi355q_qgemv": (i32, [vp, vp, vp, vp, C.c_int, vp, C.c_int, u32, u32, u32, u32]),
        "mi355q_qgemm": (i32, [vp, vp, vp, vp, C.c_int, vp, C.c_int, u32, u32, u32, u32]),
        "mi355q_gated_activation_apply": (i32, [vp, vp, vp, vp, vp, C.c_int, u32, u32, u32, C.c_int]),
        "mi355q_gated_qgemm": (i32, [vp, vp, vp, vp, vp, C.c_int, vp, C.c_int, u32, u32, u32, C.c_int, u32]),
        "mi355q_batched_qgemm": (i32, [vp, vp, u32, P(vp), vp, C.c_int, P(vp), C.c_int, u32, u32, u32]),
        "mi355q_dequant_bf16": (i32, [vp, vp, vp, vp]),
        "mi355q_dequant_f32": (i32, [vp, vp, vp, vp]),
        "mi355q_gemm_bf16": (i32, [vp, vp, vp, C.c_int, vp, vp, C.c_int, u32, u32, u32, u32, u32]),
        "mi355q_unpack_codes": (i32, [vp, vp, vp, vp]),
        "mi355q_argmax": (i32, [vp, vp, vp, C.c_int, u32, vp]),
        "mi355q_embedding_lookup": (i32, [vp, vp, vp, vp, u32, vp, C.c_int, u32, C.c_int, C.c_float]),
        "mi355q_lmhead_argmax": (i32, [vp, vp, vp, vp, C.c_int, vp, vp, u32]),
        "mi355q_lmhead_argmax_static": (i32, [vp, vp, vp, vp, C.c_int, vp, vp, u32]),
        "mi355q_lmhead_argmax_static_capacity": (u32, []),
        "mi355q_shape_family_resolve": (i32, [u32, u32, P(i32), P(u32), P(u32), C.c_char_p, sz]),
        "mi355q_plan_create": (i32, [vp, P(vp)]),
        "mi355q_plan_destroy": (i32, [vp]),
        "mi355q_plan_add_linear": (i32, [vp, vp, vp, C.c_int, vp, C.c_int, u32, u32, u32, u32, i32, C.c_char_p]),
        "mi355q_plan_add_batched_linear": (i32, [vp, u32, vp, vp, C.c_int, vp, C.c_int, u32, u32, u32, i32,
                                                  C.c_char_p]),
        "mi355q_plan_add_gated_mlp": (i32, [vp, vp, vp, vp, C.c_int, vp, C.c_int, u32, u32, u32, C.c_int, u32, i32, C.c_char_p]),
        "mi355q_plan_add_output_head": (i32, [vp, vp, vp, C.c_int, vp, vp, u32, C.c_char_p]),
        "mi355q_plan_step_count": (i32, [vp]),
        "mi355q_plan_step_at": (i32, [vp, i32, P(_Step), P(i32), C.c_char_p, sz]),
        "mi355q_plan_encode": (i32, [vp, vp, u32, u32]),
        "mi355q_plan_graph_build": (i32, [vp, vp]),
        "mi355q_plan_graph_launch": (i32, [vp, vp]),
        "mi355q_buffer_copy": (i32, [vp, vp, vp, vp, sz]),
        "mi355q_buffer_read_probe": (i32, [vp, vp, vp, sz]),
        "mi355q_clock_probe_read": (i32, [vp, P(u64), P(u64)]),
        "mi355q_context_scratch_bytes": (i32, [vp, P(u64)]),
        "mi355q_probe_wide_shape": (None, [u32, u32]),
        "mi355q_probe_route": (i32, [u8, u32, u32, u64, u64, C.c_int, u32, u32, u32, C.c_int, C.c_int, C.c_char_p, C.c_char_p, sz]),
        "mi355q_probe_shared_route": (i32, [u8, u32, u32, u32, P(u64), u64, C.c_int, u32, u32, u32, C.c_char_p, C.c_char_p, sz]),
        "mi355q_kv_scheme_is_supported": (i32, [u8]),
        "mi355q_kv_bytes_per_head_slot": (u32, [u8, u32]),
        "mi355q_kv_cache_write": (i32, [vp, vp, P(_KvLayout), vp, vp, C.c_int, u32, u32, u32]),
        "mi355q_kv_cache_read": (i32, [vp, vp, P(_KvLayout), vp, vp, C.c_int, u32, u32, u32]),
        "mi355q_staf_open": (i32, [C.c_char_p, P(vp)]),
        "mi355q_staf_close": (None, [vp]),
        "mi355q_staf_format_version": (u32, [vp]),
        "mi355q_staf_tensor_count": (u32, [vp]),
        "mi355q_staf_tensor_at": (i32, [vp, u32, P(_StafEntry)]),
        "mi355q_staf_find": (i32, [vp, C.c_char_p, P(_StafEntry)]),
        "mi355q_staf_payload_region": (vp, [vp, P(u64)]),
        "mi355q_staf_metadata_count": (u32, [vp]),
        "mi355q_staf_metadata_at": (i32, [vp, u32, P(_StafMetadata)]),
        "mi355q_staf_is_valid": (i32, [C.c_char_p, P(C.c_char_p), u32, P(_StafMetadata), u32, P(i32)]),
        "mi355q_staf_write": (i32, [C.c_char_p, P(_StafTensor), u32, P(_StafMetadata), u32]),
        "mi355q_staf_upload": (i32, [vp, vp, P(vp), P(u64)]),
        "mi355q_staf_weight": (i32, [vp, vp, vp, C.c_char_p, C.c_int, P(vp)]),
        "mi355q_plan_decode_step": (i32, [vp, u32, C.c_int, u32, P(_Step)]),
        "mi355q_plan_prefill_steps": (i32, [vp, u32, u32, C.c_int, C.c_int, u32, P(_Step), P(u32)]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)          # AttributeError here means the ABI and this binding diverged
        fn.restype, fn.argtypes = res, args
    _lib = L
    return L


EXPORTED_SYMBOLS = None  # filled lazily by exported_symbols()


def exported_symbols():
    """Names this binding expects the library to export (== every declaration of the C headers)."""
    import re
    text = ""
    for name in ("mi355_qlinear.h", "mi355_qlinear_probe.h"):
        with open(os.path.join(_HERE, "..", "include", name)) as f:
            text += f.read()
    return sorted(set(re.findall(r"MI355Q_API\s+[A-Za-z0-9_ ]+?\**\s*\b(mi355q_[a-z0-9_]+)\s*\(", text)))


def _check(status: int):
    if status != 0:
        msg = library().mi355q_last_error()
        raise MI355QError(status, msg.decode() if msg else "")


# --------------------------------------------------------------------------------- formats
@dataclass(frozen=True)
class QuantizationFormat:
    scheme_identifier: int
    bits: int
    group_size: int
    weights_per_block: int
    bytes_per_block: int
    is_quantized: bool
    is_aligned: bool
    has_direct_gemm: bool
    batched_gemm_counts: tuple
    in_reference_registry: bool
    direct_gemm_threadgroup_memory_length: int
    block_struct_name: str
    gemv_kernel_name: str
    gemm_kernel_name_f32s: str
    gemm_kernel_name: str
    dequant_to_bfloat_kernel_name: str
    embedding_lookup_token: str

    @staticmethod
    def _from(c: _Format) -> "QuantizationFormat":
        return QuantizationFormat(
            c.scheme_identifier, c.bits, c.group_size, c.weights_per_block, c.bytes_per_block,
            bool(c.is_quantized), bool(c.is_aligned), bool(c.has_direct_gemm),
            tuple(i for i in range(8) if c.batched_gemm_counts >> i & 1), bool(c.in_reference_registry),
            c.direct_gemm_threadgroup_memory_length, c.block_struct_name.decode(), c.gemv_kernel_name.decode(),
            c.gemm_kernel_name_f32s.decode(), c.gemm_kernel_name.decode(),
            c.dequant_to_bfloat_kernel_name.decode(), c.embedding_lookup_token.decode())

    def gemm_kernel_name_for(self, buffer_precision: int) -> str:
        return self.gemm_kernel_name_f32s if buffer_precision == F32 else self.gemm_kernel_name

    def weight_bytes(self, n: int, k: int) -> int:
        return n * (k // self.group_size) * self.bytes_per_block


class QuantizationFormatRegistry:
    @staticmethod
    def format_for_mlx_quantization(bits: int, group_size: int) -> QuantizationFormat:
        c = _Format()
        _check(library().mi355q_format_for_mlx_quantization(bits, group_size, C.byref(c)))
        return QuantizationFormat._from(c)

    @staticmethod
    def format(scheme_identifier: int) -> QuantizationFormat:
        c = _Format()
        _check(library().mi355q_format_for_scheme(scheme_identifier, C.byref(c)))
        return QuantizationFormat._from(c)

    @staticmethod
    def all_formats():
        L = library()
        out = []
        for i in range(L.mi355q_format_count()):
            c = _Format()
            _check(L.mi355q_format_at(i, C.byref(c)))
            out.append(QuantizationFormat._from(c))
        return out


def bf16_from_f32(value: float) -> int:
    return int(library().mi355q_bf16_from_f32(float(np.float32(value))))


def _np_sb(a, sb_dtype):
    return np.ascontiguousarray(a, dtype=np.float32 if sb_dtype == F32 else np.uint16)


def repack_mlx_to_staf(fmt: QuantizationFormat, codes, scales, biases, sb_dtype: int) -> np.ndarray:
    """STAFPayloadConverter.repackMLXQuantized on host memory (no GPU needed)."""
    codes = np.ascontiguousarray(codes, dtype=np.uint32)
    n, packed = codes.shape
    scales, biases = _np_sb(scales, sb_dtype), _np_sb(biases, sb_dtype)
    k = packed * 32 // fmt.bits
    out = np.zeros(max(1, n * (k // fmt.group_size) * fmt.bytes_per_block), dtype=np.uint8)
    _check(library().mi355q_repack_mlx_to_staf(fmt.scheme_identifier, n, packed, codes.ctypes.data,
                                               scales.ctypes.data, biases.ctypes.data, sb_dtype,
                                               out.ctypes.data, out.size))
    return out


# ------------------------------------------------------------------------- device objects
class DeviceBuffer:
    def __init__(self, ctx: "Context", ptr: int, nbytes: int):
        self.ctx, self.ptr, self.nbytes = ctx, ptr, nbytes

    def download(self, dtype, shape=None) -> np.ndarray:
        dtype = np.dtype(dtype)
        out = np.empty(self.nbytes // dtype.itemsize, dtype=dtype)
        _check(library().mi355q_buffer_download(self.ctx.handle, out.ctypes.data, self.ptr, out.nbytes))
        return out.reshape(shape) if shape is not None else out

    def upload(self, array: np.ndarray):
        a = np.ascontiguousarray(array)
        assert a.nbytes <= self.nbytes
        _check(library().mi355q_buffer_upload(self.ctx.handle, self.ptr, a.ctypes.data, a.nbytes))

    def free(self):
        if self.ptr:
            _check(library().mi355q_buffer_free(self.ctx.handle, self.ptr))
            self.ptr = 0

    def offset(self, nbytes: int) -> int:
        return self.ptr + nbytes


@dataclass(frozen=True)
class DispatchStep:
    """One planned launch together with its quantization-plan entry."""
    kernel_name: str
    device_kernel: str
    kernel_family: str
    grid: tuple
    block: tuple
    lds_bytes: int
    rows_per_workgroup: int
    reference_simdgroups: int
    reference_tile_elements: int
    shape_family: str
    path: str
    scheme_identifier: int
    layout: int
    used_fallback: bool
    fallback_reason: str | None
    input_dimension: int
    output_dimension: int
    sequence_length: int
    input_row_stride: int
    weight_bytes: int
    flops: int

    @staticmethod
    def _from(s: _Step) -> "DispatchStep":
        return DispatchStep(s.kernel_name.decode(), s.device_kernel.decode(), s.kernel_family.decode(),
                            tuple(s.grid), tuple(s.block), s.lds_bytes, s.rows_per_workgroup,
                            s.reference_simdgroups, s.reference_tile_elements, FAMILY_NAMES[s.shape_family],
                            PATH_NAMES[s.path], s.scheme_identifier, s.layout, bool(s.used_fallback),
                            FALLBACK_NAMES[s.fallback_reason], s.input_dimension, s.output_dimension,
                            s.sequence_length, s.input_row_stride, s.weight_bytes, s.flops)


class PackedWeight:
    """A prepared (or wrapped) packed weight: the STAFWeightBufferAccess of one tensor."""

    def __init__(self, ctx: "Context", handle: int, keepalive=()):
        self.ctx, self.handle, self._keep = ctx, handle, keepalive

    @property
    def info(self) -> _WeightInfo:
        i = _WeightInfo()
        _check(library().mi355q_weight_query(self.handle, C.byref(i)))
        return i

    @property
    def format(self) -> QuantizationFormat:
        return QuantizationFormatRegistry.format(self.info.scheme_identifier)

    def plan_decode_step(self, m: int = 1, x_dtype: int = BF16, flags: int = 0) -> DispatchStep:
        s = _Step()
        _check(library().mi355q_plan_decode_step(self.handle, m, x_dtype, flags, C.byref(s)))
        return DispatchStep._from(s)

    def plan_prefill_steps(self, maximum_sequence_length: int, input_row_stride: int = 0, x_dtype: int = BF16,
                           is_last_token: bool = False, flags: int = 0):
        steps = (_Step * 2)()
        n = C.c_uint32(0)
        _check(library().mi355q_plan_prefill_steps(self.handle, maximum_sequence_length, input_row_stride, x_dtype,
                                                   int(is_last_token), flags, steps, C.byref(n)))
        return [DispatchStep._from(steps[i]) for i in range(n.value)]

    def destroy(self):
        if self.handle:
            _check(library().mi355q_weight_destroy(self.handle))
            self.handle = 0


class DispatchPlan:
    """Ordered projection steps built once and replayed per token (MetalDispatchPlan + encodeSteps)."""

    def __init__(self, ctx: "Context"):
        h = C.c_void_p()
        _check(library().mi355q_plan_create(ctx.handle, C.byref(h)))
        self.ctx, self.handle, self._keep = ctx, h.value, []

    def add_linear(self, w: "PackedWeight", x, x_dtype, y, y_dtype, m=1, x_row_stride=0, y_row_stride=0, flags=0,
                   layer_index=-1, tensor_name: str | None = None):
        _check(library().mi355q_plan_add_linear(self.handle, w.handle, Context._ptr(x), x_dtype, Context._ptr(y),
                                                y_dtype, m, x_row_stride, y_row_stride, flags, layer_index,
                                                tensor_name.encode() if tensor_name else None))
        self._keep.append((w, x, y))

    def add_batched_linear(self, weights, x, x_dtype, ys, y_dtype, m=1, x_row_stride=0, flags=0, layer_index=-1,
                           tensor_name: str | None = None):
        """2 or 3 projections sharing x (q+k+v, gate+up) as one step; one launch when M <= 8."""
        n = len(weights)
        wh = (C.c_void_p * n)(*[w.handle for w in weights])
        yh = (C.c_void_p * n)(*[Context._ptr(y) for y in ys])
        _check(library().mi355q_plan_add_batched_linear(self.handle, n, wh, Context._ptr(x), x_dtype, yh, y_dtype, m,
                                                        x_row_stride, flags, layer_index,
                                                        tensor_name.encode() if tensor_name else None))
        self._keep.append((list(weights), x, list(ys)))

    def add_gated_mlp(self, w_gate, w_up, x, x_dtype, y, y_dtype, m=1, activation=GATED_SILU, x_row_stride=0,
                      y_row_stride=0, flags=0, layer_index=-1, tensor_name: str | None = None):
        """gate_proj + up_proj + swiglu / gelu_gated as one step: y = act(x Wgate^T) * (x Wup^T)."""
        _check(library().mi355q_plan_add_gated_mlp(self.handle, w_gate.handle, w_up.handle, Context._ptr(x), x_dtype,
                                                   Context._ptr(y), y_dtype, m, x_row_stride, y_row_stride, activation,
                                                   flags, layer_index, tensor_name.encode() if tensor_name else None))
        self._keep.append(([w_gate, w_up], x, y))

    def add_output_head(self, w: "PackedWeight", x, x_dtype, logits_f32, token_out, flags=0,
                        tensor_name: str | None = None):
        _check(library().mi355q_plan_add_output_head(self.handle, w.handle, Context._ptr(x), x_dtype,
                                                     Context._ptr(logits_f32), Context._ptr(token_out), flags,
                                                     tensor_name.encode() if tensor_name else None))
        self._keep.append((w, x, logits_f32, token_out))

    def __len__(self):
        return library().mi355q_plan_step_count(self.handle)

    def step(self, index: int):
        s, layer = _Step(), C.c_int32()
        name = C.create_string_buffer(128)
        _check(library().mi355q_plan_step_at(self.handle, index, C.byref(s), C.byref(layer), name, 128))
        return DispatchStep._from(s), layer.value, name.value.decode()

    def encode(self, stream: int = 0, first: int = 0, count: int = 0):
        _check(library().mi355q_plan_encode(self.handle, stream, first, count))

    def graph_build(self, stream: int):
        _check(library().mi355q_plan_graph_build(self.handle, stream))

    def graph_launch(self, stream: int):
        _check(library().mi355q_plan_graph_launch(self.handle, stream))

    def destroy(self):
        if self.handle:
            _check(library().mi355q_plan_destroy(self.handle))
            self.handle = 0



# --------------------------------------------------------------------------------- STAF container
# STAFMetadataValueType
STAF_BOOL, STAF_UINT32, STAF_UINT64, STAF_FLOAT32, STAF_FLOAT64, STAF_STRING = 1, 2, 3, 4, 5, 6


@dataclass(frozen=True)
class STAFTensorEntry:
    """STAFTensorEntry (MC/STAF/STAFLoader.swift:299-311)."""
    name: str
    payload_offset: int
    payload_size: int
    scheme_identifier: int
    semantic_role: int
    original_dtype: int
    shape: tuple
    block_size: int
    group_size: int
    buffer_offset: int
    alignment: int
    checksum: int
    shard_index: int


def _entry_from_c(e: _StafEntry) -> STAFTensorEntry:
    name = C.string_at(e.name, e.name_length).decode("utf-8", "replace") if e.name else ""
    return STAFTensorEntry(name, e.payload_offset, e.payload_size, e.scheme_identifier, e.semantic_role,
                           e.original_dtype, tuple(e.shape[:e.dimension_count]), e.block_size, e.group_size,
                           e.buffer_offset, e.alignment, e.checksum, e.shard_index)


def _metadata_to_c(values: dict):
    """{key: (type, value)} -> array of mi355q_staf_metadata (plus the byte strings that back it)."""
    import struct
    arr = (_StafMetadata * max(1, len(values)))()
    keep = []
    for i, (key, (typ, value)) in enumerate(values.items()):
        kb = key.encode()
        keep.append(kb)
        arr[i].key, arr[i].type = kb, typ
        if typ == STAF_STRING:
            vb = value.encode()
            buf = C.create_string_buffer(vb, len(vb) + 1)
            keep.append(buf)
            arr[i].text, arr[i].text_length, arr[i].payload0 = C.addressof(buf), len(vb), 0
        elif typ == STAF_FLOAT32:
            arr[i].payload0 = struct.unpack("<I", struct.pack("<f", value))[0]
        elif typ == STAF_FLOAT64:
            arr[i].payload0 = struct.unpack("<Q", struct.pack("<d", value))[0]
        else:
            arr[i].payload0 = int(value)
    return arr, keep


class STAFFile:
    """An opened model.staf (STAFLoader.load + STAFWeightStore, MC/STAF/STAFLoader.swift:19-299)."""

    def __init__(self, path: str):
        h = C.c_void_p()
        _check(library().mi355q_staf_open(os.fsencode(path), C.byref(h)))
        self.handle = h.value

    def close(self):
        if self.handle:
            library().mi355q_staf_close(self.handle)
            self.handle = None

    @property
    def format_version(self) -> int:
        return library().mi355q_staf_format_version(self.handle)

    @property
    def entries(self) -> list:
        out = []
        for i in range(library().mi355q_staf_tensor_count(self.handle)):
            e = _StafEntry()
            _check(library().mi355q_staf_tensor_at(self.handle, i, C.byref(e)))
            out.append(_entry_from_c(e))
        return out

    def find(self, name: str) -> STAFTensorEntry:
        e = _StafEntry()
        _check(library().mi355q_staf_find(self.handle, name.encode(), C.byref(e)))
        return _entry_from_c(e)

    @property
    def metadata(self) -> dict:
        import struct
        out = {}
        for i in range(library().mi355q_staf_metadata_count(self.handle)):
            m = _StafMetadata()
            _check(library().mi355q_staf_metadata_at(self.handle, i, C.byref(m)))
            if m.type == STAF_STRING:
                v = C.string_at(m.text, m.text_length).decode("utf-8", "replace") if m.text else ""
            elif m.type == STAF_BOOL:
                v = m.payload0 != 0
            elif m.type == STAF_UINT32:
                v = m.payload0 & 0xFFFFFFFF
            elif m.type == STAF_FLOAT32:
                v = struct.unpack("<f", struct.pack("<I", m.payload0 & 0xFFFFFFFF))[0]
            elif m.type == STAF_FLOAT64:
                v = struct.unpack("<d", struct.pack("<Q", m.payload0))[0]
            else:
                v = m.payload0
            out[m.key.decode()] = (m.type, v)
        return out

    def payload_region(self) -> np.ndarray:
        """Copy of the payload region (first tensor to end of file) as bytes."""
        n = C.c_uint64()
        p = library().mi355q_staf_payload_region(self.handle, C.byref(n))
        return np.frombuffer(C.string_at(p, n.value), dtype=np.uint8)

    def payload(self, entry: STAFTensorEntry) -> np.ndarray:
        return self.payload_region()[entry.buffer_offset:entry.buffer_offset + entry.payload_size]

    def upload(self, ctx: "Context") -> "DeviceBuffer":
        """The single device buffer of the weight store; tensors live at .ptr + entry.buffer_offset."""
        p, n = C.c_void_p(), C.c_uint64()
        _check(library().mi355q_staf_upload(ctx.handle, self.handle, C.byref(p), C.byref(n)))
        return DeviceBuffer(ctx, p.value, n.value)

    def weight(self, ctx: "Context", name: str, layout: int = LAYOUT_STAF_BLOCKS,
               region: "DeviceBuffer | None" = None) -> "PackedWeight":
        h = C.c_void_p()
        _check(library().mi355q_staf_weight(ctx.handle, self.handle, region.ptr if region is not None else None,
                                            name.encode(), layout, C.byref(h)))
        return PackedWeight(ctx, h.value, keepalive=(region, self) if region is not None else (self,))


def staf_write(path: str, tensors: list, metadata: dict | None = None):
    """STAFWriter.write for converted payloads.  tensors: dicts with name, scheme_identifier, shape, payload
    (bytes-like) and optionally semantic_role, original_dtype, shard_index; metadata: {key: (type, value)}."""
    arr = (_StafTensor * max(1, len(tensors)))()
    keep = []
    for i, t in enumerate(tensors):
        nb = t["name"].encode()
        pb = np.ascontiguousarray(np.frombuffer(bytes(t["payload"]), dtype=np.uint8))
        keep += [nb, pb]
        arr[i].name, arr[i].scheme_identifier = nb, t["scheme_identifier"]
        arr[i].semantic_role, arr[i].original_dtype = t.get("semantic_role", 0), t.get("original_dtype", 0xFF)
        arr[i].dimension_count = len(t["shape"])
        for d, v in enumerate(t["shape"][:8]):
            arr[i].shape[d] = v
        arr[i].payload, arr[i].payload_size = pb.ctypes.data if pb.size else None, pb.size
        arr[i].shard_index = t.get("shard_index", 0)
    md, keep_md = _metadata_to_c(metadata or {})
    _check(library().mi355q_staf_write(os.fsencode(path), arr, len(tensors), md, len(metadata or {})))


def staf_is_valid(path: str, sources=(), expected: dict | None = None) -> bool:
    """STAFValidator.isValid (MC/STAF/STAFValidator.swift:5-78)."""
    src = (C.c_char_p * max(1, len(sources)))(*[os.fsencode(s) for s in sources])
    md, keep = _metadata_to_c(expected or {})
    ok = C.c_int32()
    _check(library().mi355q_staf_is_valid(os.fsencode(path), src, len(sources), md, len(expected or {}), C.byref(ok)))
    return bool(ok.value)



# --------------------------------------------------------------------------------- KV cache
KV_SEQUENCE_MAJOR, KV_HEAD_MAJOR = 0, 1      # KVCacheLayoutMode


def kv_scheme_is_supported(scheme_identifier: int) -> bool:
    return bool(library().mi355q_kv_scheme_is_supported(scheme_identifier))


def kv_bytes_per_head_slot(scheme_identifier: int, head_dimension: int) -> int:
    return library().mi355q_kv_bytes_per_head_slot(scheme_identifier, head_dimension)


@dataclass(frozen=True)
class KVCacheSpecification:
    """One layer's K or V cache (KVCacheSpecification, MC/Buffer/MetalGraphAllocator.swift:7-175)."""
    scheme_identifier: int
    layout_mode: int
    kv_head_count: int
    head_dimension: int
    maximum_sequence_length: int

    @property
    def bytes_per_head_slot(self) -> int:
        return kv_bytes_per_head_slot(self.scheme_identifier, self.head_dimension)

    @property
    def bytes_per_token_slot(self) -> int:
        return self.kv_head_count * self.bytes_per_head_slot

    @property
    def bytes_per_layer(self) -> int:
        return self.maximum_sequence_length * self.bytes_per_token_slot

    def offset(self, head: int, position: int) -> int:
        slot = self.bytes_per_head_slot
        if self.layout_mode == KV_SEQUENCE_MAJOR:
            return head * self.maximum_sequence_length * slot + position * slot
        return position * self.kv_head_count * slot + head * slot

    def _c(self) -> _KvLayout:
        return _KvLayout(self.scheme_identifier, self.layout_mode, 0, self.kv_head_count, self.head_dimension,
                         self.maximum_sequence_length, self.bytes_per_head_slot)


def shape_family(output_dimension: int, input_dimension: int):
    """DecodeProjectionShapeFamily.resolve -> (family, preferredSimdgroups, tileElements, kernelBaseName)."""
    fam, sg, tile = C.c_int32(), C.c_uint32(), C.c_uint32()
    name = C.create_string_buffer(48)
    _check(library().mi355q_shape_family_resolve(output_dimension, input_dimension, C.byref(fam), C.byref(sg),
                                                 C.byref(tile), name, 48))
    return FAMILY_NAMES[fam.value], sg.value, tile.value, name.value.decode()


class Context:
    """Device context (the MTLDevice + command queue stand-in).  Raises MI355QError when no GPU."""

    def __init__(self, device_index: int = 0):
        h = C.c_void_p()
        _check(library().mi355q_context_create(device_index, C.byref(h)))
        self.handle = h.value

    def close(self):
        if self.handle:
            library().mi355q_context_destroy(self.handle)
            self.handle = None

    def scratch_bytes(self):
        """Bytes of device scratch the context holds (partial results, split rows, gated sums)."""
        out = (C.c_uint64 * 3)()
        _check(library().mi355q_context_scratch_bytes(self.handle, out))
        return tuple(int(v) for v in out)

    @staticmethod
    def probe_wide_shape(tile_rows: int = 0, k_parts: int = 0):
        """A/B runs: tile height and K parts of the wide-tile prefill kernel for the whole process (0: the library chooses)."""
        library().mi355q_probe_wide_shape(tile_rows, k_parts)

    def set_library_use(self, enabled: bool):
        """Whether launches may hand a dense product to the platform's GEMM library (on by default)."""
        _check(library().mi355q_context_set_library_use(self.handle, 1 if enabled else 0))

    # ---- device info / memory / streams / events
    def device_info(self) -> _DeviceInfo:
        i = _DeviceInfo()
        _check(library().mi355q_device_query(self.handle, C.byref(i)))
        return i

    def alloc(self, nbytes: int) -> DeviceBuffer:
        p = C.c_void_p()
        _check(library().mi355q_buffer_alloc(self.handle, max(1, nbytes), C.byref(p)))
        return DeviceBuffer(self, p.value, nbytes)

    def upload(self, array: np.ndarray) -> DeviceBuffer:
        a = np.ascontiguousarray(array)
        b = self.alloc(a.nbytes)
        if a.nbytes:
            b.upload(a)
        return b

    def read_probe(self, src, nbytes: int, stream: int = 0):
        """One launch that only streams `nbytes` of `src` from HBM (the ceiling a decode launch is compared with)."""
        _check(library().mi355q_buffer_read_probe(self.handle, stream, self._ptr(src), nbytes))

    def copy(self, dst, src, nbytes: int, stream: int = 0):
        _check(library().mi355q_buffer_copy(self.handle, stream, self._ptr(dst), self._ptr(src), nbytes))

    def fill(self, buf: DeviceBuffer, word: int, stream: int = 0):
        _check(library().mi355q_buffer_fill(self.handle, stream, buf.ptr, word, buf.nbytes // 4))

    def stream_create(self) -> int:
        p = C.c_void_p()
        _check(library().mi355q_stream_create(self.handle, C.byref(p)))
        return p.value

    def stream_destroy(self, stream: int):
        _check(library().mi355q_stream_destroy(self.handle, stream))

    def synchronize(self, stream: int = 0):
        _check(library().mi355q_stream_synchronize(self.handle, stream))

    def event_create(self) -> int:
        p = C.c_void_p()
        _check(library().mi355q_event_create(self.handle, C.byref(p)))
        return p.value

    def event_destroy(self, ev: int):
        _check(library().mi355q_event_destroy(self.handle, ev))

    def event_record(self, ev: int, stream: int = 0):
        _check(library().mi355q_event_record(self.handle, ev, stream))

    def event_synchronize(self, ev: int):
        _check(library().mi355q_event_synchronize(self.handle, ev))

    def event_elapsed_ms(self, start: int, stop: int) -> float:
        ms = C.c_float()
        _check(library().mi355q_event_elapsed_ms(self.handle, start, stop, C.byref(ms)))
        return ms.value

    # ---- packed weights
    def weight_prepare_mlx(self, fmt: QuantizationFormat, codes, scales, biases, sb_dtype: int,
                           layout: int = LAYOUT_PLANES, k: int | None = None) -> PackedWeight:
        codes = np.ascontiguousarray(codes, dtype=np.uint32)
        n, packed = codes.shape
        k = packed * 32 // fmt.bits if k is None else k
        scales, biases = _np_sb(scales, sb_dtype), _np_sb(biases, sb_dtype)
        h = C.c_void_p()
        _check(library().mi355q_weight_prepare_mlx(self.handle, fmt.scheme_identifier, n, k, codes.ctypes.data,
                                                   scales.ctypes.data, biases.ctypes.data, sb_dtype, layout,
                                                   C.byref(h)))
        return PackedWeight(self, h.value)

    def weight_prepare_staf(self, fmt: QuantizationFormat, n: int, k: int, blocks,
                            layout: int = LAYOUT_STAF_BLOCKS) -> PackedWeight:
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        h = C.c_void_p()
        _check(library().mi355q_weight_prepare_staf(self.handle, fmt.scheme_identifier, n, k, blocks.ctypes.data,
                                                    blocks.size, layout, C.byref(h)))
        return PackedWeight(self, h.value)

    def clock_probe_ghz(self) -> float:
        """Shader clock of the last MFMA GEMM launched with FLAG_PROBE_CLOCK (0.0 if none ran)."""
        c, t = C.c_uint64(), C.c_uint64()
        _check(library().mi355q_clock_probe_read(self.handle, C.byref(c), C.byref(t)))
        return c.value / (t.value * 10.0) if t.value else 0.0

    def kv_cache_write(self, spec: "KVCacheSpecification", cache, src, src_dtype: int, first_position: int,
                       sequence_length: int, input_row_stride: int = 0, stream: int = 0):
        lay = spec._c()
        _check(library().mi355q_kv_cache_write(self.handle, stream, C.byref(lay), self._ptr(cache), self._ptr(src),
                                               src_dtype, input_row_stride, first_position, sequence_length))

    def kv_cache_read(self, spec: "KVCacheSpecification", cache, out, out_dtype: int, first_position: int,
                      sequence_length: int, out_row_stride: int = 0, stream: int = 0):
        lay = spec._c()
        _check(library().mi355q_kv_cache_read(self.handle, stream, C.byref(lay), self._ptr(cache), self._ptr(out),
                                              out_dtype, out_row_stride, first_position, sequence_length))

    def weight_wrap_staf(self, fmt: QuantizationFormat, n: int, k: int, blocks: DeviceBuffer,
                         byte_offset: int = 0, payload_bytes: int | None = None) -> PackedWeight:
        payload_bytes = fmt.weight_bytes(n, k) if payload_bytes is None else payload_bytes
        h = C.c_void_p()
        _check(library().mi355q_weight_wrap_staf(self.handle, fmt.scheme_identifier, n, k,
                                                 blocks.ptr + byte_offset, payload_bytes, C.byref(h)))
        return PackedWeight(self, h.value, keepalive=(blocks,))

    def weight_wrap_planes(self, fmt: QuantizationFormat, n: int, k: int, codes: DeviceBuffer,
                           scales: DeviceBuffer, biases: DeviceBuffer, sb_dtype: int) -> PackedWeight:
        h = C.c_void_p()
        _check(library().mi355q_weight_wrap_planes(self.handle, fmt.scheme_identifier, n, k, codes.ptr, scales.ptr,
                                                   biases.ptr, sb_dtype, C.byref(h)))
        return PackedWeight(self, h.value, keepalive=(codes, scales, biases))

    # ---- launches (device pointers as ints or DeviceBuffers)
    @staticmethod
    def _ptr(b):
        return b.ptr if isinstance(b, DeviceBuffer) else (0 if b is None else int(b))

    def qgemv(self, w: PackedWeight, x, x_dtype, y, y_dtype, m=1, x_row_stride=0, y_row_stride=0, flags=0,
              stream=0):
        _check(library().mi355q_qgemv(self.handle, stream, w.handle, self._ptr(x), x_dtype, self._ptr(y), y_dtype,
                                      m, x_row_stride, y_row_stride, flags))

    def qgemm(self, w: PackedWeight, x, x_dtype, y, y_dtype, m, x_row_stride=0, y_row_stride=0, flags=0,
              stream=0):
        _check(library().mi355q_qgemm(self.handle, stream, w.handle, self._ptr(x), x_dtype, self._ptr(y), y_dtype,
                                      m, x_row_stride, y_row_stride, flags))

    def batched_qgemm(self, weights, x, x_dtype, ys, y_dtype, m, x_row_stride=0, flags=0, stream=0):
        n = len(weights)
        wh = (C.c_void_p * n)(*[w.handle for w in weights])
        yh = (C.c_void_p * n)(*[self._ptr(y) for y in ys])
        _check(library().mi355q_batched_qgemm(self.handle, stream, n, wh, self._ptr(x), x_dtype, yh, y_dtype, m,
                                              x_row_stride, flags))

    def gated_qgemm(self, w_gate, w_up, x, x_dtype, y, y_dtype, m, activation=GATED_SILU, x_row_stride=0,
                    y_row_stride=0, flags=0, stream=0):
        """MLPFragment's gate_proj + up_proj + swiglu / gelu_gated as one call: y = act(x Wgate^T) * (x Wup^T)."""
        _check(library().mi355q_gated_qgemm(self.handle, stream, w_gate.handle, w_up.handle, self._ptr(x), x_dtype,
                                            self._ptr(y), y_dtype, m, x_row_stride, y_row_stride, activation, flags))

    def gated_activation(self, gate, up, out, dtype, dimension, sequence_length=1, row_stride=0,
                         activation=GATED_SILU, stream=0):
        """The elementwise step alone: out = act(gate) * up."""
        _check(library().mi355q_gated_activation_apply(self.handle, stream, self._ptr(gate), self._ptr(up),
                                                       self._ptr(out), dtype, dimension, sequence_length, row_stride,
                                                       activation))

    def dequant_bf16(self, w: PackedWeight, out, stream=0):
        _check(library().mi355q_dequant_bf16(self.handle, stream, w.handle, self._ptr(out)))

    def dequant_f32(self, w: PackedWeight, out, stream=0):
        """CPUWeightStore.decodeQuantized on the device: row-major fp32 [N, K], scale * q then + zero, two roundings."""
        _check(library().mi355q_dequant_f32(self.handle, stream, w.handle, self._ptr(out)))

    def gemm_bf16(self, a, a_dtype, b_bf16, c, c_dtype, m, n, k, a_row_stride=0, c_row_stride=0, stream=0):
        _check(library().mi355q_gemm_bf16(self.handle, stream, self._ptr(a), a_dtype, self._ptr(b_bf16),
                                          self._ptr(c), c_dtype, m, n, k, a_row_stride, c_row_stride))

    def embedding_lookup(self, table: PackedWeight, token_ids, sequence_length, out, out_dtype, out_row_stride=0,
                         embedding_scale=None, stream=0):
        """Gather dequantised rows of a packed [vocabulary, embeddingDim] table (GatherFragment)."""
        _check(library().mi355q_embedding_lookup(self.handle, stream, table.handle, self._ptr(token_ids),
                                                 sequence_length, self._ptr(out), out_dtype, out_row_stride,
                                                 0 if embedding_scale is None else 1,
                                                 0.0 if embedding_scale is None else float(embedding_scale)))

    def unpack_codes(self, w: PackedWeight, out, stream=0):
        _check(library().mi355q_unpack_codes(self.handle, stream, w.handle, self._ptr(out)))

    def argmax(self, logits, dtype, vocabulary_size, token_out, stream=0):
        _check(library().mi355q_argmax(self.handle, stream, self._ptr(logits), dtype, vocabulary_size,
                                       self._ptr(token_out)))

    def lmhead_argmax(self, w: PackedWeight, x, x_dtype, logits_f32, token_out, flags=0, stream=0):
        _check(library().mi355q_lmhead_argmax(self.handle, stream, w.handle, self._ptr(x), x_dtype,
                                              self._ptr(logits_f32), self._ptr(token_out), flags))

    def lmhead_argmax_static(self, w: PackedWeight, x, x_dtype, logits_f32, token_out, flags=0, stream=0):
        """The same head through the entry point that allocates nothing (its partial keys live in the library image)."""
        _check(library().mi355q_lmhead_argmax_static(self.handle, stream, w.handle, self._ptr(x), x_dtype,
                                                     self._ptr(logits_f32), self._ptr(token_out), flags))
