// Quantized KV cache: write (quantise one head vector per wavefront into its slot) and read (dequantise
// slots back to rows).  The slot format is the weight block format: per group f16 scale, f16 minimum,
// then 8-bit codes or 4-bit codes packed two to a byte, low nibble first.
//
// Restates write_kv_quantized_q8 / _q4, write_kv_element_dense and read_kv_element
// (Sources/MetalCompiler/Generator/MetalSourceGenerator+Attention.swift:2057-2157, 1958-1971, 1923-1956) and the
// slot addressing of the cache fill kernel (:762-769, 1233-1250).  HBM-bound and tiny: one launch moves
// positions x heads x (head_dim x source element + slot) bytes.
#include "device_utils.h"

namespace mi355q {

struct KvArgs {
    uint8_t* cache;
    const void* src;       // write: [count, row_stride] in dtype
    void* out;             // read:  [count, row_stride] in dtype
    uint32_t scheme, layout_mode, kv_heads, head_dim, max_positions, slot_bytes;
    uint32_t row_stride, first_position, count, dtype;
    uint32_t bits, group, bytes_per_block;     // 0 for the dense schemes
};

__device__ __forceinline__ size_t kv_slot_offset(const KvArgs& a, uint32_t head, uint32_t position) {
    return a.layout_mode == 0 ? ((size_t)head * a.max_positions + position) * a.slot_bytes
                              : ((size_t)position * a.kv_heads + head) * a.slot_bytes;
}

__device__ __forceinline__ float kv_load(const void* p, size_t i, uint32_t dtype) {
    if (dtype == MI355Q_F32) return ((const float*)p)[i];
    if (dtype == MI355Q_BF16) return __uint_as_float((uint32_t)((const uint16_t*)p)[i] << 16);
    return f16_to_f32(((const uint16_t*)p)[i]);
}

__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = fminf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

// One wavefront per (position, head) vector.
__global__ __launch_bounds__(256) void kv_cache_write_kernel(KvArgs a) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t v = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (v >= a.count * a.kv_heads) return;               // wavefront-uniform
    const uint32_t p = v / a.kv_heads, h = v - p * a.kv_heads;
    uint8_t* slot = a.cache + kv_slot_offset(a, h, a.first_position + p);
    const size_t src0 = (size_t)p * a.row_stride + (size_t)h * a.head_dim;
    if (a.bits == 0) {                                    // dense slot: one conversion per element
        for (uint32_t d = lane; d < a.head_dim; d += 64) {
            const float x = kv_load(a.src, src0 + d, a.dtype);
            if (a.scheme == 0x02) ((float*)slot)[d] = x;
            else if (a.scheme == 0x01) ((uint16_t*)slot)[d] = f32_to_bf16_rne(x);
            else ((uint16_t*)slot)[d] = f32_to_f16_rne(x);
        }
        return;
    }
    const float levels = a.bits == 8 ? 255.0f : 15.0f;
    const int top = a.bits == 8 ? 255 : 15;
    for (uint32_t start = 0, g = 0; start < a.head_dim; start += a.group, g++) {
        const uint32_t len = a.head_dim - start < a.group ? a.head_dim - start : a.group;
        float lo = INFINITY, hi = -INFINITY;
        for (uint32_t i = lane; i < len; i += 64) {
            const float x = kv_load(a.src, src0 + start + i, a.dtype);
            lo = fminf(lo, x);
            hi = fmaxf(hi, x);
        }
        lo = wave_min(lo);
        hi = wave_max(hi);
        float scale = __fdiv_rn(__fsub_rn(hi, lo), levels);
        if (scale < 1e-10f) scale = 1e-10f;
        uint8_t* block = slot + (size_t)g * a.bytes_per_block;
        if (lane == 0) {
            ((uint16_t*)block)[0] = f32_to_f16_rne(scale);
            ((uint16_t*)block)[1] = f32_to_f16_rne(lo);
        }
        auto code = [&](float x) {
            const int q = (int)roundf(__fdiv_rn(__fsub_rn(x, lo), scale));
            return q < 0 ? 0 : q > top ? top : q;
        };
        if (a.bits == 8) {
            for (uint32_t i = lane; i < len; i += 64)
                block[4 + i] = (uint8_t)code(kv_load(a.src, src0 + start + i, a.dtype));
        } else {
            for (uint32_t i = lane; 2 * i < len; i += 64) {
                const float x0 = kv_load(a.src, src0 + start + 2 * i, a.dtype);
                const float x1 = 2 * i + 1 < len ? kv_load(a.src, src0 + start + 2 * i + 1, a.dtype) : 0.0f;
                block[4 + i] = (uint8_t)(code(x0) | (code(x1) << 4));
            }
        }
    }
}

// The same quantiser for head vectors of exactly 128 elements (two per lane, read with one load) with all groups of
// the vector in flight at once: minimum and maximum are taken inside the run of group/2 lanes that holds a group,
// every lane then writes its own two codes.  Same operations per element as the kernel above, so the same bytes.
__global__ __launch_bounds__(256) void kv_cache_write_hd128_kernel(KvArgs a) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t v = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (v >= a.count * a.kv_heads) return;               // wavefront-uniform
    const uint32_t p = v / a.kv_heads, h = v - p * a.kv_heads;
    uint8_t* slot = a.cache + kv_slot_offset(a, h, a.first_position + p);
    const size_t src0 = (size_t)p * a.row_stride + (size_t)h * 128u + 2u * lane;
    float x0, x1;
    if (a.dtype == MI355Q_F32) {
        const float2 t = *(const float2*)((const float*)a.src + src0);
        x0 = t.x; x1 = t.y;
    } else {
        const uint32_t t = *(const uint32_t*)((const uint16_t*)a.src + src0);
        if (a.dtype == MI355Q_BF16) { x0 = __uint_as_float(t << 16); x1 = __uint_as_float(t & 0xFFFF0000u); }
        else { x0 = f16_to_f32((uint16_t)(t & 0xFFFFu)); x1 = f16_to_f32((uint16_t)(t >> 16)); }
    }
    float lo = fminf(x0, x1), hi = fmaxf(x0, x1);
    for (uint32_t o = a.group >> 2; o >= 1; o >>= 1) {    // group / 2 lanes hold one group
        lo = fminf(lo, __shfl_xor(lo, (int)o));
        hi = fmaxf(hi, __shfl_xor(hi, (int)o));
    }
    const float levels = a.bits == 8 ? 255.0f : 15.0f;
    const int top = a.bits == 8 ? 255 : 15;
    float scale = __fdiv_rn(__fsub_rn(hi, lo), levels);
    if (scale < 1e-10f) scale = 1e-10f;
    const uint32_t d = 2u * lane, g = d / a.group, i = d - g * a.group;
    uint8_t* block = slot + (size_t)g * a.bytes_per_block;
    if (i == 0) *(uint32_t*)block = (uint32_t)f32_to_f16_rne(scale) | ((uint32_t)f32_to_f16_rne(lo) << 16);
    auto code = [&](float x) {
        const int q = (int)roundf(__fdiv_rn(__fsub_rn(x, lo), scale));
        return (uint32_t)(q < 0 ? 0 : q > top ? top : q);
    };
    const uint32_t q0 = code(x0), q1 = code(x1);
    if (a.bits == 8) *(uint16_t*)(block + 4 + i) = (uint16_t)(q0 | (q1 << 8));
    else block[4 + (i >> 1)] = (uint8_t)(q0 | (q1 << 4));
}

// Head vectors of 128 elements, four per lane: a wavefront quantises two vectors (one per half), a lane reads its
// four elements with one load and writes its four codes with one store, and a group's minimum and maximum are
// taken inside the run of group/4 lanes that holds it.  Same operations per element again, so the same bytes.
__global__ __launch_bounds__(256) void kv_cache_write_hd128x4_kernel(KvArgs a) {
    const uint32_t lane = threadIdx.x & 63, l = lane & 31;
    const uint32_t total = a.count * a.kv_heads;
    const uint32_t v_raw = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 2 + (lane >> 5);
    const bool live = v_raw < total;                      // the last wavefront may hold a single vector
    const uint32_t v = live ? v_raw : total - 1;          // its other half repeats that vector and stores nothing
    const uint32_t p = v / a.kv_heads, h = v - p * a.kv_heads;
    uint8_t* slot = a.cache + kv_slot_offset(a, h, a.first_position + p);
    const size_t src0 = (size_t)p * a.row_stride + (size_t)h * 128u + 4u * l;
    float x[4];
    if (a.dtype == MI355Q_F32) {
        const float4 t = *(const float4*)((const float*)a.src + src0);
        x[0] = t.x; x[1] = t.y; x[2] = t.z; x[3] = t.w;
    } else {
        const uint2 t = *(const uint2*)((const uint16_t*)a.src + src0);
        if (a.dtype == MI355Q_BF16) {
            x[0] = __uint_as_float(t.x << 16); x[1] = __uint_as_float(t.x & 0xFFFF0000u);
            x[2] = __uint_as_float(t.y << 16); x[3] = __uint_as_float(t.y & 0xFFFF0000u);
        } else {
            x[0] = f16_to_f32((uint16_t)(t.x & 0xFFFFu)); x[1] = f16_to_f32((uint16_t)(t.x >> 16));
            x[2] = f16_to_f32((uint16_t)(t.y & 0xFFFFu)); x[3] = f16_to_f32((uint16_t)(t.y >> 16));
        }
    }
    float lo = fminf(fminf(x[0], x[1]), fminf(x[2], x[3])), hi = fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3]));
    for (uint32_t o = a.group >> 3; o >= 1; o >>= 1) {    // group / 4 lanes hold one group
        lo = fminf(lo, __shfl_xor(lo, (int)o));
        hi = fmaxf(hi, __shfl_xor(hi, (int)o));
    }
    const float levels = a.bits == 8 ? 255.0f : 15.0f;
    const int top = a.bits == 8 ? 255 : 15;
    float scale = __fdiv_rn(__fsub_rn(hi, lo), levels);
    if (scale < 1e-10f) scale = 1e-10f;
    const uint32_t d = 4u * l, g = d / a.group, i = d - g * a.group;
    uint8_t* block = slot + (size_t)g * a.bytes_per_block;
    if (!live) return;
    if (i == 0) *(uint32_t*)block = (uint32_t)f32_to_f16_rne(scale) | ((uint32_t)f32_to_f16_rne(lo) << 16);
    uint32_t q[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int c = (int)roundf(__fdiv_rn(__fsub_rn(x[e], lo), scale));
        q[e] = (uint32_t)(c < 0 ? 0 : c > top ? top : c);
    }
    if (a.bits == 8) *(uint32_t*)(block + 4 + i) = q[0] | (q[1] << 8) | (q[2] << 16) | (q[3] << 24);
    else *(uint16_t*)(block + 4 + (i >> 1)) = (uint16_t)(q[0] | (q[1] << 4) | (q[2] << 8) | (q[3] << 12));
}

// One thread per element of the output rows.
__global__ __launch_bounds__(256) void kv_cache_read_kernel(KvArgs a) {
    const uint32_t row_elems = a.kv_heads * a.head_dim;
    for (uint32_t p = blockIdx.y; p < a.count; p += gridDim.y)     // positions beyond the grid's y limit wrap round
    for (uint32_t e = blockIdx.x * 256 + threadIdx.x; e < row_elems; e += gridDim.x * 256) {
        const uint32_t h = e / a.head_dim, d = e - h * a.head_dim;
        const uint8_t* slot = a.cache + kv_slot_offset(a, h, a.first_position + p);
        float x;
        if (a.bits == 0) {
            x = a.scheme == 0x02 ? ((const float*)slot)[d]
              : a.scheme == 0x01 ? __uint_as_float((uint32_t)((const uint16_t*)slot)[d] << 16)
                                 : f16_to_f32(((const uint16_t*)slot)[d]);
        } else {
            const uint8_t* block = slot + (size_t)(d / a.group) * a.bytes_per_block;
            const uint32_t i = d % a.group;
            const float scale = f16_to_f32(((const uint16_t*)block)[0]), zero = f16_to_f32(((const uint16_t*)block)[1]);
            const uint32_t q = a.bits == 8 ? block[4 + i] : (i & 1 ? block[4 + i / 2] >> 4 : block[4 + i / 2] & 0x0Fu);
            x = __fadd_rn(__fmul_rn(scale, (float)q), zero);
        }
        const size_t o = (size_t)p * a.row_stride + e;
        if (a.dtype == MI355Q_F32) ((float*)a.out)[o] = x;
        else if (a.dtype == MI355Q_BF16) ((uint16_t*)a.out)[o] = f32_to_bf16_rne(x);
        else ((uint16_t*)a.out)[o] = f32_to_f16_rne(x);
    }
}

// Quantized slots, four consecutive elements of a head vector per thread (they share a group: groups and head
// dimensions are multiples of four here): one 32- or 16-bit load of codes, one header, one 8- or 16-byte store.
// Same arithmetic per element as the kernel above.
__global__ __launch_bounds__(256) void kv_cache_read_x4_kernel(KvArgs a) {
    const uint32_t row_elems = a.kv_heads * a.head_dim;
    for (uint32_t p = blockIdx.y; p < a.count; p += gridDim.y)
    for (uint32_t e = (blockIdx.x * 256 + threadIdx.x) * 4; e < row_elems; e += gridDim.x * 1024) {
        const uint32_t h = e / a.head_dim, d = e - h * a.head_dim;
        const uint8_t* slot = a.cache + kv_slot_offset(a, h, a.first_position + p);
        const uint8_t* block = slot + (size_t)(d / a.group) * a.bytes_per_block;
        const uint32_t i = d % a.group;
        const uint32_t hdr = *(const uint32_t*)block;
        const float scale = f16_to_f32((uint16_t)(hdr & 0xFFFFu)), zero = f16_to_f32((uint16_t)(hdr >> 16));
        uint32_t q[4];
        if (a.bits == 8) {
            const uint32_t w = *(const uint32_t*)(block + 4 + i);
            q[0] = w & 0xFFu; q[1] = (w >> 8) & 0xFFu; q[2] = (w >> 16) & 0xFFu; q[3] = w >> 24;
        } else {
            const uint32_t w = *(const uint16_t*)(block + 4 + (i >> 1));
            q[0] = w & 0xFu; q[1] = (w >> 4) & 0xFu; q[2] = (w >> 8) & 0xFu; q[3] = (w >> 12) & 0xFu;
        }
        float x[4];
#pragma unroll
        for (int j = 0; j < 4; j++) x[j] = __fadd_rn(__fmul_rn(scale, (float)q[j]), zero);
        const size_t o = (size_t)p * a.row_stride + e;
        if (a.dtype == MI355Q_F32) {
            float4 t; t.x = x[0]; t.y = x[1]; t.z = x[2]; t.w = x[3];
            *(float4*)((float*)a.out + o) = t;
        } else {
            uint2 t;
            if (a.dtype == MI355Q_BF16) {
                t.x = (uint32_t)f32_to_bf16_rne(x[0]) | ((uint32_t)f32_to_bf16_rne(x[1]) << 16);
                t.y = (uint32_t)f32_to_bf16_rne(x[2]) | ((uint32_t)f32_to_bf16_rne(x[3]) << 16);
            } else {
                t.x = (uint32_t)f32_to_f16_rne(x[0]) | ((uint32_t)f32_to_f16_rne(x[1]) << 16);
                t.y = (uint32_t)f32_to_f16_rne(x[2]) | ((uint32_t)f32_to_f16_rne(x[3]) << 16);
            }
            *(uint2*)((uint16_t*)a.out + o) = t;
        }
    }
}

namespace {

// kv_quant_bits / kv_quant_group_size / kv_quant_bytes_per_block (:1894-1921)
bool kv_block_layout(uint8_t scheme, uint32_t* bits, uint32_t* group) {
    switch (scheme) {
    case 0x10: *bits = 8; *group = 32; return true;
    case 0x11: *bits = 8; *group = 64; return true;
    case 0x12: *bits = 8; *group = 128; return true;
    case 0x40: *bits = 4; *group = 64; return true;
    case 0x41: case 0x42: *bits = 4; *group = 128; return true;
    default: *bits = 0; *group = 0; return false;
    }
}

mi355q_status kv_prepare(const mi355q_context* ctx, const mi355q_kv_layout* l, const void* cache, const void* rows,
                         int dtype, uint32_t row_stride, uint32_t first_position, uint32_t count, KvArgs* a) {
    if (!ctx) return fail(MI355Q_ERR_NULL_HANDLE, "context is null");
    if (!l || !cache || !rows) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null layout or buffer");
    if (!mi355q_kv_scheme_is_supported(l->scheme))
        return fail(MI355Q_ERR_UNSUPPORTED_FORMAT, "scheme 0x%02x has no KV cache kernels", (unsigned)l->scheme);
    if (dtype != MI355Q_F16 && dtype != MI355Q_BF16 && dtype != MI355Q_F32)
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "unknown element type %d", dtype);
    if (l->layout_mode > 1) return fail(MI355Q_ERR_INVALID_ARGUMENT, "layout mode is 0 (sequence-major) or 1 (head-major)");
    if (!l->kv_head_count || !l->head_dimension || !l->maximum_sequence_length || !count)
        return fail(MI355Q_ERR_SHAPE, "head count, head dimension, maximum sequence length and sequence length must be positive");
    if ((uint64_t)first_position + count > l->maximum_sequence_length)
        return fail(MI355Q_ERR_SHAPE, "positions [%u, %u) leave the cache of %u positions", first_position,
                    first_position + count, l->maximum_sequence_length);
    const uint32_t row = l->kv_head_count * l->head_dimension;
    if (row_stride == 0) row_stride = row;
    if (row_stride < row) return fail(MI355Q_ERR_SHAPE, "row stride %u is shorter than heads x head dimension = %u", row_stride, row);
    std::memset(a, 0, sizeof *a);
    kv_block_layout(l->scheme, &a->bits, &a->group);
    a->bytes_per_block = a->bits ? 4 + a->group * a->bits / 8 : 0;
    const uint32_t raw = a->bits ? (l->head_dimension + a->group - 1) / a->group * a->bytes_per_block
                                 : l->head_dimension * (l->scheme == 0x02 ? 4u : 2u);
    if (l->head_slot_bytes < raw || l->head_slot_bytes % 4)
        return fail(MI355Q_ERR_SIZE_MISMATCH, "head slot of %u bytes: need at least %u and a multiple of 4", l->head_slot_bytes, raw);
    if ((uintptr_t)cache % 4 || (uintptr_t)rows % 4) return fail(MI355Q_ERR_INVALID_ARGUMENT, "buffers must be 4-byte aligned");
    a->cache = (uint8_t*)const_cast<void*>(cache);
    a->scheme = l->scheme; a->layout_mode = l->layout_mode; a->kv_heads = l->kv_head_count; a->head_dim = l->head_dimension;
    a->max_positions = l->maximum_sequence_length; a->slot_bytes = l->head_slot_bytes;
    a->row_stride = row_stride; a->first_position = first_position; a->count = count; a->dtype = (uint32_t)dtype;
    return MI355Q_OK;
}

}  // namespace
}  // namespace mi355q

using namespace mi355q;

extern "C" {

int32_t mi355q_kv_scheme_is_supported(uint8_t scheme) {
    uint32_t bits, group;
    return scheme <= 0x02 || kv_block_layout(scheme, &bits, &group);
}

uint32_t mi355q_kv_bytes_per_head_slot(uint8_t scheme, uint32_t head_dim) {
    uint32_t weights = 1, bytes = 2, alignment = 256;
    if (scheme == 0x02) bytes = 4;
    else if (scheme > 0x01 && scheme != 0xFF) {
        if (scheme == 0x70) scheme = 0x10;               // rotor schemes size as their base scheme
        if (scheme == 0x71) scheme = 0x40;
        mi355q_format f;
        if (mi355q_format_for_scheme(scheme, &f) != MI355Q_OK || !f.in_reference_registry) return 0;
        weights = f.group_size; bytes = f.bytes_per_block; alignment = 64;
    }
    const uint32_t raw = (head_dim + weights - 1) / weights * bytes;
    return (raw + alignment - 1) / alignment * alignment;
}

mi355q_status mi355q_kv_cache_write(mi355q_context* ctx, void* stream, const mi355q_kv_layout* layout, void* cache_dev,
                                    const void* src_dev, mi355q_dtype src_dtype, uint32_t input_row_stride,
                                    uint32_t first_position, uint32_t sequence_length) {
    KvArgs a;
    if (mi355q_status st = kv_prepare(ctx, layout, cache_dev, src_dev, (int)src_dtype, input_row_stride, first_position,
                                      sequence_length, &a)) return st;
    a.src = src_dev;
    const uint64_t vectors = (uint64_t)a.count * a.kv_heads;
    const size_t esz = a.dtype == MI355Q_F32 ? 4 : 2;
    const bool two_per_lane = a.bits != 0 && a.head_dim == 128 && a.row_stride % 2 == 0 &&
                              (uintptr_t)src_dev % (2 * esz) == 0 && (a.group == 32 || a.group == 64 || a.group == 128);
    // four per lane needs 8- or 16-byte loads of the source and 4-byte aligned slots
    const bool four_per_lane = two_per_lane && a.row_stride % 4 == 0 && (uintptr_t)src_dev % (4 * esz) == 0 &&
                               a.slot_bytes % 4 == 0 && (uintptr_t)a.cache % 4 == 0;
    if (four_per_lane)
        kv_cache_write_hd128x4_kernel<<<dim3((unsigned)((vectors + 7) / 8)), dim3(256), 0, (hipStream_t)stream>>>(a);
    else if (two_per_lane)
        kv_cache_write_hd128_kernel<<<dim3((unsigned)((vectors + 3) / 4)), dim3(256), 0, (hipStream_t)stream>>>(a);
    else
        kv_cache_write_kernel<<<dim3((unsigned)((vectors + 3) / 4)), dim3(256), 0, (hipStream_t)stream>>>(a);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

mi355q_status mi355q_kv_cache_read(mi355q_context* ctx, void* stream, const mi355q_kv_layout* layout, const void* cache_dev,
                                   void* out_dev, mi355q_dtype out_dtype, uint32_t out_row_stride, uint32_t first_position,
                                   uint32_t sequence_length) {
    KvArgs a;
    if (mi355q_status st = kv_prepare(ctx, layout, cache_dev, out_dev, (int)out_dtype, out_row_stride, first_position,
                                      sequence_length, &a)) return st;
    a.out = out_dev;
    const uint32_t row = a.kv_heads * a.head_dim;
    const size_t esz = a.dtype == MI355Q_F32 ? 4 : 2;
    const uint32_t by = a.count < 65535u ? a.count : 65535u;     // grid y limit; the kernels stride over the rest
    // four elements per thread: whole groups of four, 4-byte aligned slots and blocks, 8- or 16-byte aligned output rows
    const bool four = a.bits != 0 && a.head_dim % 4 == 0 && a.group % 4 == 0 && a.slot_bytes % 4 == 0 &&
                      a.bytes_per_block % 4 == 0 && (uintptr_t)a.cache % 4 == 0 && a.row_stride % 4 == 0 &&
                      (uintptr_t)out_dev % (4 * esz) == 0;
    if (four) {
        uint32_t bx = (row / 4 + 255) / 256;
        if (bx > 64) bx = 64;
        kv_cache_read_x4_kernel<<<dim3(bx, by), dim3(256), 0, (hipStream_t)stream>>>(a);
        MI355Q_HIP(hipGetLastError());
        return MI355Q_OK;
    }
    uint32_t bx = (row + 255) / 256;
    if (bx > 64) bx = 64;
    kv_cache_read_kernel<<<dim3(bx, by), dim3(256), 0, (hipStream_t)stream>>>(a);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

}  // extern "C"
