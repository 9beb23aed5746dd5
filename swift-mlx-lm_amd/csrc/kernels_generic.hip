// Reference-shaped kernels: one code at a time, any registered format, either layout, any
// activation dtype and stride.  They are the always-available path (tiny shapes, odd strides,
// f16/f32 activations) and the A/B partner of the specialised kernels.
//
// Reference kernels these stand in for (Sources/MetalCompiler/Generator/):
//   generateUnifiedQuantizedGEMV      MetalSourceGenerator+Quantized.swift:496-575
//   generateQuantizedGEMM_Q4/_Q8      MetalSourceGenerator+Quantized.swift:22-156 (sequence signature)
//   generateUnifiedDequantToBFloat    MetalSourceGenerator+Quantized.swift:361-416
//   generateArgmax                    MetalSourceGenerator+Sampling.swift:62-107
#include "device_utils.h"

namespace mi355q {

// ------------------------------------------------------------------------------ unpack codes
__global__ __launch_bounds__(256) void unpack_codes_kernel(WView w, uint8_t* __restrict__ out) {
    const size_t total = (size_t)w.n * w.k;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < total; i += stride) {
        const uint32_t row = (uint32_t)(i / w.k), c = (uint32_t)(i % w.k);
        out[i] = (uint8_t)load_code(w, row, c);
    }
}

mi355q_status launch_unpack_codes(hipStream_t s, const WView& w, uint8_t* out) {
    const size_t total = (size_t)w.n * w.k;
    size_t blocks = (total + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    unpack_codes_kernel<<<dim3((unsigned)blocks), dim3(256), 0, s>>>(w, out);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

// ------------------------------------------------------------------- pack (scale, bias) words
// Split-plane weights keep one 32-bit word per group next to the two 16-bit planes:
// scale in the low half, bias in the high half, so the GEMV fetches both with one load.
__global__ __launch_bounds__(256) void pack_sz_kernel(const uint16_t* __restrict__ scales,
                                                      const uint16_t* __restrict__ biases,
                                                      uint32_t* __restrict__ sz, size_t groups,
                                                      uint32_t blocks_per_row, uint32_t sz_stride) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < groups; i += stride) {
        const size_t row = i / blocks_per_row, b = i - row * blocks_per_row;
        sz[row * sz_stride + b] = (uint32_t)scales[i] | ((uint32_t)biases[i] << 16);
    }
}

mi355q_status launch_pack_sz(hipStream_t s, const uint16_t* scales, const uint16_t* biases, uint32_t* sz,
                             size_t groups, uint32_t blocks_per_row, uint32_t sz_stride) {
    size_t blocks = (groups + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    if (blocks == 0) blocks = 1;
    pack_sz_kernel<<<dim3((unsigned)blocks), dim3(256), 0, s>>>(scales, biases, sz, groups, blocks_per_row, sz_stride);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

// TILE16 records from a split-plane weight (q4, group 64, K % 128 == 0): one thread per output word.
// Rows past N are zero (codes 0, scale 0, bias 0).  Layout: gemv_tile16.hip.
__global__ __launch_bounds__(256) void tile16_pack_kernel(WView w, uint32_t* __restrict__ tiles, size_t words) {
    const uint32_t kblocks = w.k >> 7;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += (size_t)gridDim.x * blockDim.x) {
        const size_t recno = i / 288u;
        const uint32_t o = (uint32_t)(i - recno * 288u);
        const uint32_t tile = (uint32_t)(recno / kblocks), kb = (uint32_t)(recno - (size_t)tile * kblocks);
        uint32_t out = 0;
        if (o < 256u) {
            const uint32_t lane = o >> 2, j = o & 3u, n = lane & 15u, kq = lane >> 4;
            const uint32_t row = tile * 16u + n;
            if (row < w.n) {
                const uint32_t code0 = kb * 128u + (j >> 1) * 64u + kq * 16u + (j & 1u) * 8u;   // first of 8 codes
                const uint32_t src = w.codes[(size_t)row * w.code_stride + (code0 >> 3)];
#pragma unroll
                for (uint32_t e = 0; e < 8; e++) {
                    const uint32_t nib = (e >> 1) + 4u * (e & 1u);
                    out |= ((src >> (4u * e)) & 0xFu) << (4u * nib);
                }
            }
        } else {
            const uint32_t q = o - 256u, n = q >> 1, g = q & 1u;
            const uint32_t row = tile * 16u + n;
            if (row < w.n) out = w.sz[(size_t)row * w.sz_stride + kb * 2u + g];
        }
        tiles[i] = out;
    }
}

mi355q_status launch_tile16_pack(hipStream_t s, const WView& planes, uint32_t* tiles) {
    const size_t words = (size_t)((planes.n + 15) / 16) * (planes.k / 128) * 288u;
    size_t blocks = (words + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    if (blocks == 0) blocks = 1;
    tile16_pack_kernel<<<dim3((unsigned)blocks), dim3(256), 0, s>>>(planes, tiles, words);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

// Codes c0 .. c0+7 of a row (c0 a multiple of 8) as one little-endian bit string: code i sits at bit
// i*bits.  A run of 8 codes starts on a byte boundary and spans at most 64 bits for every width.
__device__ __forceinline__ uint64_t load_codes8(const WView& w, uint32_t row, uint32_t c0) {
    uint64_t v = 0;
    if (w.layout == MI355Q_LAYOUT_PLANES) {
        const uint32_t* rowp = w.codes + (size_t)row * w.code_stride;
        const uint32_t bit = c0 * w.bits, word = bit >> 5, sh = bit & 31u;
        v = rowp[word];
        if (sh + 8u * w.bits > 32u) v |= (uint64_t)rowp[word + 1] << 32;
        v >>= sh;
    } else if (w.layout == MI355Q_LAYOUT_STAF_BLOCKS) {
        const uint32_t b = c0 / w.group, e = c0 - b * w.group;
        const uint8_t* qs =
            w.blocks + ((size_t)row * w.blocks_per_row + b) * w.bytes_per_block + 4 + ((e * w.bits) >> 3);
        if (((uintptr_t)qs & 3u) == 0 && (w.bits & 3u) == 0) {
            v = *(const uint32_t*)qs;
            if (w.bits == 8) v |= (uint64_t)((const uint32_t*)qs)[1] << 32;
        } else {
            for (uint32_t i = 0; i < w.bits; i++) v |= (uint64_t)qs[i] << (8u * i);
        }
    } else {
        // TILE16 (4-bit): the 8 codes are one record word, lane kq*16 + row%16, word j as in load_code; its nibbles are
        // stored as (c0,c2,c4,c6,c1,c3,c5,c7): even codes in the low half, odd ones in the high half
        const uint32_t o = c0 & 127u, g = o >> 6, in_g = o & 63u, kq = in_g >> 4, j = g * 2 + ((in_g >> 3) & 1u);
        const uint32_t* rec = w.tiles + ((size_t)(row >> 4) * (w.k >> 7) + (c0 >> 7)) * 288u;
        const uint32_t word = rec[(kq * 16u + (row & 15u)) * 4u + j];
        auto spread = [](uint32_t x) {                       // nibble i of the low 16 bits -> nibble 2i
            x = (x | (x << 8)) & 0x00FF00FFu;
            return (x | (x << 4)) & 0x0F0F0F0Fu;
        };
        v = spread(word & 0xFFFFu) | (spread(word >> 16) << 4);
    }
    return v;
}

// --------------------------------------------------------------------------- embedding lookup
// out[pos, d] = (float(q) * scale + zero) [* embeddingScale] of table row token_ids[pos], rounded once to
// the output type: embedding_lookup[_seq]_q{b}_g{g} of the reference
// (Sources/MetalCompiler/Generator/MetalSourceGenerator+Embedding.swift:79-153, 229-322).  Any layout and
// bit width; the two roundings (product, sum) are kept apart so the fp32 result is bit-identical to an
// unfused host evaluation.  A token id outside the table yields a row of zeros (the reference reads out
// of bounds there).
__global__ __launch_bounds__(256) void embedding_lookup_kernel(WView w, const int32_t* __restrict__ token_ids,
                                                               uint32_t sequence_length, void* __restrict__ out,
                                                               uint32_t out_dtype, uint32_t out_stride, int has_scale,
                                                               float embedding_scale) {
    const uint32_t pos = blockIdx.y;
    if (pos >= sequence_length) return;
    const int32_t tok = token_ids[pos];
    const bool valid = tok >= 0 && (uint32_t)tok < w.n;
    for (uint32_t d = blockIdx.x * 256u + threadIdx.x; d < w.k; d += gridDim.x * 256u) {
        float v = 0.0f;
        if (valid) {
            float scale, zero;
            load_scale_zero(w, (uint32_t)tok, d / w.group, scale, zero);
            const float q = (float)load_code(w, (uint32_t)tok, d);
            v = __fadd_rn(__fmul_rn(q, scale), zero);
            if (has_scale) v = __fmul_rn(v, embedding_scale);
        }
        const size_t o = (size_t)pos * out_stride + d;
        if (out_dtype == MI355Q_F32) ((float*)out)[o] = v;
        else if (out_dtype == MI355Q_BF16) ((uint16_t*)out)[o] = f32_to_bf16_rne(v);
        else ((uint16_t*)out)[o] = f32_to_f16_rne(v);
    }
}

// The same lookup with eight consecutive dimensions per thread (one or two code loads, one scale/zero
// pair, 128-bit stores): the variant for rows of whole 8-code runs and 16-byte aligned output rows.  The grid is
// (chunks of a row) x (positions) and the bit width a template argument: no 64-bit division, constant shifts.
template <int BITS>
__global__ __launch_bounds__(256) void embedding_lookup_x8_kernel(WView w, const int32_t* __restrict__ token_ids,
                                                                  uint32_t sequence_length, void* __restrict__ out,
                                                                  uint32_t out_dtype, uint32_t out_stride, int has_scale,
                                                                  float embedding_scale) {
    constexpr uint32_t mask = (1u << BITS) - 1u;
    const uint32_t d0 = (blockIdx.x * 256 + threadIdx.x) << 3;
    if (d0 >= w.k) return;
    for (uint32_t pos = blockIdx.y; pos < sequence_length; pos += gridDim.y) {
        const int32_t tok = token_ids[pos];
        float f[8];
#pragma unroll
        for (int i = 0; i < 8; i++) f[i] = 0.0f;
        if (tok >= 0 && (uint32_t)tok < w.n) {
            const uint64_t v = load_codes8(w, (uint32_t)tok, d0);
            float scale, zero;
            load_scale_zero(w, (uint32_t)tok, d0 / w.group, scale, zero);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float q = (float)((uint32_t)(v >> (i * BITS)) & mask);
                f[i] = __fadd_rn(__fmul_rn(q, scale), zero);
                if (has_scale) f[i] = __fmul_rn(f[i], embedding_scale);
            }
        }
        const size_t o = (size_t)pos * out_stride + d0;
        if (out_dtype == MI355Q_F32) {
            typedef float f32x4 __attribute__((ext_vector_type(4)));
            f32x4 a, b;
            a.x = f[0]; a.y = f[1]; a.z = f[2]; a.w = f[3];
            b.x = f[4]; b.y = f[5]; b.z = f[6]; b.w = f[7];
            ((f32x4*)((float*)out + o))[0] = a;
            ((f32x4*)((float*)out + o))[1] = b;
        } else {
            uint32_t h[8];
#pragma unroll
            for (int i = 0; i < 8; i++) h[i] = out_dtype == MI355Q_BF16 ? f32_to_bf16_rne(f[i]) : f32_to_f16_rne(f[i]);
            u32x4 st;
            st.x = h[0] | (h[1] << 16); st.y = h[2] | (h[3] << 16);
            st.z = h[4] | (h[5] << 16); st.w = h[6] | (h[7] << 16);
            *(u32x4*)((uint16_t*)out + o) = st;
        }
    }
}

mi355q_status launch_embedding_lookup(hipStream_t s, const WView& w, const int32_t* token_ids, uint32_t sequence_length,
                                      void* out, int out_dtype, uint32_t out_stride, int has_scale,
                                      float embedding_scale) {
    const size_t esz = out_dtype == MI355Q_F32 ? 4 : 2;
    if (w.k % 8 == 0 && (uintptr_t)out % 16 == 0 && ((size_t)out_stride * esz) % 16 == 0) {
        const dim3 grid((w.k / 8 + 255) / 256, sequence_length < 65535u ? sequence_length : 65535u), block(256);
#define MI355Q_EMBED_CASE(B)                                                                                        \
    case B:                                                                                                         \
        embedding_lookup_x8_kernel<B><<<grid, block, 0, s>>>(w, token_ids, sequence_length, out, (uint32_t)out_dtype, \
                                                             out_stride, has_scale, embedding_scale);               \
        break;
        switch (w.bits) {
            MI355Q_EMBED_CASE(2) MI355Q_EMBED_CASE(3) MI355Q_EMBED_CASE(4) MI355Q_EMBED_CASE(5) MI355Q_EMBED_CASE(6)
            MI355Q_EMBED_CASE(8)
        default: return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no embedding kernel for %u-bit codes", w.bits);
        }
#undef MI355Q_EMBED_CASE
    } else {
        uint32_t gx = (w.k + 255u) / 256u;
        if (gx > 64u) gx = 64u;
        embedding_lookup_kernel<<<dim3(gx, sequence_length), dim3(256), 0, s>>>(w, token_ids, sequence_length, out,
                                                                               (uint32_t)out_dtype, out_stride,
                                                                               has_scale, embedding_scale);
    }
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

// ------------------------------------------------------------------------------ gated activation (SwiGLU / GEGLU)
// out[s, i] = T(activation(float(gate[s, i])) * float(up[s, i])): the reference's swiglu / gelu_gated elementwise kernel
// (Sources/MetalCompiler/Generator/MetalSourceGenerator+NormAndElementwise.swift:196-249), one element per thread.
__global__ __launch_bounds__(256) void gated_activation_kernel(const void* __restrict__ gate, const void* __restrict__ up,
                                                              void* __restrict__ out, uint32_t dtype, uint32_t dimension,
                                                              uint32_t sequence_length, uint32_t gate_stride,
                                                              uint32_t up_stride, uint32_t out_stride, uint32_t activation) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= dimension) return;
    for (uint32_t sq = blockIdx.y; sq < sequence_length; sq += gridDim.y) {
        const size_t gi = (size_t)sq * gate_stride + i, ui = (size_t)sq * up_stride + i, oi = (size_t)sq * out_stride + i;
        float g, u;
        if (dtype == MI355Q_F32) { g = ((const float*)gate)[gi]; u = ((const float*)up)[ui]; }
        else if (dtype == MI355Q_BF16) { g = bf16_to_f32(((const uint16_t*)gate)[gi]); u = bf16_to_f32(((const uint16_t*)up)[ui]); }
        else { g = f16_to_f32(((const uint16_t*)gate)[gi]); u = f16_to_f32(((const uint16_t*)up)[ui]); }
        const float v = gated_value(g, u, activation, MI355Q_F32);
        if (dtype == MI355Q_F32) ((float*)out)[oi] = v;
        else if (dtype == MI355Q_BF16) ((uint16_t*)out)[oi] = f32_to_bf16_rne(v);
        else ((uint16_t*)out)[oi] = f32_to_f16_rne(v);
    }
}

mi355q_status launch_gated_activation(hipStream_t s, const void* gate, const void* up, void* out, int dtype, uint32_t dimension,
                                      uint32_t sequence_length, uint32_t gate_stride, uint32_t up_stride, uint32_t out_stride,
                                      int activation) {
    const dim3 grid((dimension + 255u) / 256u, sequence_length < 65535u ? sequence_length : 65535u);
    gated_activation_kernel<<<grid, dim3(256), 0, s>>>(gate, up, out, (uint32_t)dtype, dimension, sequence_length, gate_stride,
                                                       up_stride, out_stride, (uint32_t)activation);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

// ------------------------------------------------------------------------------ dequant to bf16 / fp32
// One workgroup per row, 256 threads striding over the row, as the reference kernel does.
// scale*q and +zero are kept as two roundings so the result is bit-identical to an unfused
// host evaluation (the order CPUWeightStore.decodeQuantized evaluates, Sources/SwiftLM/CPUWeightStore.swift:170).
// OUT (an mi355q_dtype): F32 stores the fp32 value itself, BF16 and F16 its rounding to nearest even.
template <int OUT>
__device__ __forceinline__ uint16_t dequant_round16(float v) {
    return OUT == MI355Q_BF16 ? f32_to_bf16_rne(v) : f32_to_f16_rne(v);
}

template <int OUT>
__global__ __launch_bounds__(256) void dequant_kernel(WView w, void* __restrict__ out) {
    constexpr bool F32 = OUT == MI355Q_F32;
    for (uint32_t row = blockIdx.x; row < w.n; row += gridDim.x) {
        for (uint32_t c = threadIdx.x; c < w.k; c += 256) {
            float scale, zero;
            load_scale_zero(w, row, c / w.group, scale, zero);
            const float q = (float)load_code(w, row, c);
            const float v = __fadd_rn(__fmul_rn(scale, q), zero);
            if constexpr (F32) ((float*)out)[(size_t)row * w.k + c] = v;
            else ((uint16_t*)out)[(size_t)row * w.k + c] = dequant_round16<OUT>(v);
        }
    }
}

// Eight consecutive codes per thread: one or two 32-bit loads of codes (a run of 8 codes starts on a
// byte boundary and spans at most 64 bits for every width), one scale/zero pair (groups are multiples
// of 8 codes), one 128-bit store.  Same arithmetic as the per-element kernel above.
// BITS is a template argument (constant shifts on the 64-bit field) and the grid is two-dimensional -- x over the
// 8-code chunks of a row, y over rows -- so that no thread divides a 64-bit index: with run-time width and a flat index
// the kernel was bound by its integer arithmetic (42 us for 4096 -> 14336, against 26 us for a plain copy of as many bytes).
template <int BITS, int OUT>
__global__ __launch_bounds__(256) void dequant_x8_kernel(WView w, void* __restrict__ out) {
    constexpr bool F32 = OUT == MI355Q_F32;
    const uint32_t c0 = (blockIdx.x * 256 + threadIdx.x) << 3;
    if (c0 >= w.k) return;
    constexpr uint32_t mask = (1u << BITS) - 1u;
    const uint32_t g = c0 / w.group;
#pragma unroll 2
    for (uint32_t row = blockIdx.y; row < w.n; row += gridDim.y) {
        const uint64_t v = load_codes8(w, row, c0);
        float scale, zero;
        load_scale_zero(w, row, g, scale, zero);
        float f[8];
#pragma unroll
        for (int i = 0; i < 8; i++) f[i] = __fadd_rn(__fmul_rn(scale, (float)((uint32_t)(v >> (i * BITS)) & mask)), zero);
        if constexpr (F32) {
            u32x4 lo, hi;
            lo.x = __float_as_uint(f[0]); lo.y = __float_as_uint(f[1]); lo.z = __float_as_uint(f[2]); lo.w = __float_as_uint(f[3]);
            hi.x = __float_as_uint(f[4]); hi.y = __float_as_uint(f[5]); hi.z = __float_as_uint(f[6]); hi.w = __float_as_uint(f[7]);
            u32x4* dst = (u32x4*)((float*)out + (size_t)row * w.k + c0);
            __builtin_nontemporal_store(lo, dst);
            __builtin_nontemporal_store(hi, dst + 1);
        } else {
            u32x4 st;
            st.x = dequant_round16<OUT>(f[0]) | ((uint32_t)dequant_round16<OUT>(f[1]) << 16);
            st.y = dequant_round16<OUT>(f[2]) | ((uint32_t)dequant_round16<OUT>(f[3]) << 16);
            st.z = dequant_round16<OUT>(f[4]) | ((uint32_t)dequant_round16<OUT>(f[5]) << 16);
            st.w = dequant_round16<OUT>(f[6]) | ((uint32_t)dequant_round16<OUT>(f[7]) << 16);
            __builtin_nontemporal_store(st, (u32x4*)((uint16_t*)out + (size_t)row * w.k + c0));
        }
    }
}

template <int OUT>
mi355q_status launch_dequant(hipStream_t s, const WView& w, void* out) {
    constexpr bool F32 = OUT == MI355Q_F32;
    if (w.k % 8 == 0 && (uintptr_t)out % 16 == 0 && (!F32 || w.k % 4 == 0)) {
        // two to four rows per thread, at most 65535 workgroups along y
        uint32_t gy = w.n > 4096 ? (w.n + 3) / 4 : (w.n + 1) / 2;
        if (gy > 65535u) gy = 65535u;
        const dim3 grid((w.k / 8 + 255) / 256, gy), block(256);
        switch (w.bits) {
        case 2: dequant_x8_kernel<2, OUT><<<grid, block, 0, s>>>(w, out); break;
        case 3: dequant_x8_kernel<3, OUT><<<grid, block, 0, s>>>(w, out); break;
        case 4: dequant_x8_kernel<4, OUT><<<grid, block, 0, s>>>(w, out); break;
        case 5: dequant_x8_kernel<5, OUT><<<grid, block, 0, s>>>(w, out); break;
        case 6: dequant_x8_kernel<6, OUT><<<grid, block, 0, s>>>(w, out); break;
        case 8: dequant_x8_kernel<8, OUT><<<grid, block, 0, s>>>(w, out); break;
        default: return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no dequantisation kernel for %u-bit codes", w.bits);
        }
    } else {
        unsigned blocks = w.n < 65535u * 16u ? w.n : 65535u * 16u;
        dequant_kernel<OUT><<<dim3(blocks), dim3(256), 0, s>>>(w, out);
    }
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

// fp32 activations as two bf16 matrices: hi = bf16(x), lo = bf16(x - hi), so that hi + lo carries sixteen bits of x
// (x - hi is exact in fp32).  Four elements per thread; x rows 16-byte aligned, K a multiple of 4.
__global__ __launch_bounds__(256) void split_f32_bf16x2_kernel(const float* __restrict__ x, uint32_t m, uint32_t k,
                                                               uint32_t x_stride, uint16_t* __restrict__ hi,
                                                               uint16_t* __restrict__ lo, uint32_t out_stride) {
    const uint32_t row = blockIdx.y;
    for (uint32_t c = (blockIdx.x * 256 + threadIdx.x) * 4; c < k; c += gridDim.x * 1024) {
        const float4 v = *(const float4*)(x + (size_t)row * x_stride + c);
        const float f[4] = {v.x, v.y, v.z, v.w};
        uint16_t h[4], l[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            h[i] = f32_to_bf16_rne(f[i]);
            // a finite value above the largest bf16 would round to infinity: the largest bf16 and a remainder instead;
            // a non-finite one stands alone
            const bool finite = f[i] - f[i] == 0.0f;
            if (finite && (h[i] & 0x7FFFu) == 0x7F80u) h[i] = (uint16_t)((h[i] & 0x8000u) | 0x7F7Fu);
            l[i] = finite ? f32_to_bf16_rne(f[i] - __uint_as_float((uint32_t)h[i] << 16)) : (uint16_t)0;
        }
        uint2 hv, lv;
        hv.x = h[0] | ((uint32_t)h[1] << 16); hv.y = h[2] | ((uint32_t)h[3] << 16);
        lv.x = l[0] | ((uint32_t)l[1] << 16); lv.y = l[2] | ((uint32_t)l[3] << 16);
        *(uint2*)(hi + (size_t)row * out_stride + c) = hv;
        *(uint2*)(lo + (size_t)row * out_stride + c) = lv;
    }
}

// Rows from one floating-point type to another, one element per thread (a handful of rows: the small-batch form of the
// two-dispatch route widens its activations to fp32 and narrows its fp32 result).
__global__ __launch_bounds__(256) void convert_rows_kernel(const void* __restrict__ src, int src_dtype, uint32_t src_stride,
                                                           void* __restrict__ dst, int dst_dtype, uint32_t dst_stride,
                                                           uint32_t cols) {
    const uint32_t row = blockIdx.y;
    for (uint32_t c = blockIdx.x * 256 + threadIdx.x; c < cols; c += gridDim.x * 256) {
        const size_t i = (size_t)row * src_stride + c, o = (size_t)row * dst_stride + c;
        const float v = src_dtype == MI355Q_F32 ? ((const float*)src)[i]
                      : src_dtype == MI355Q_BF16 ? __uint_as_float((uint32_t)((const uint16_t*)src)[i] << 16)
                                                 : f16_to_f32(((const uint16_t*)src)[i]);
        if (dst_dtype == MI355Q_F32) ((float*)dst)[o] = v;
        else if (dst_dtype == MI355Q_BF16) ((uint16_t*)dst)[o] = f32_to_bf16_rne(v);
        else ((uint16_t*)dst)[o] = f32_to_f16_rne(v);
    }
}

mi355q_status launch_convert_rows(hipStream_t s, const void* src, int src_dtype, uint32_t src_stride, void* dst, int dst_dtype,
                                  uint32_t dst_stride, uint32_t rows, uint32_t cols) {
    if (rows > 65535u) return fail(MI355Q_ERR_SHAPE, "more than 65535 rows");
    uint32_t gx = (cols + 255) / 256;
    if (gx > 256) gx = 256;
    convert_rows_kernel<<<dim3(gx, rows), dim3(256), 0, s>>>(src, src_dtype, src_stride, dst, dst_dtype, dst_stride, cols);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

// fp32 activations as three bf16 rows each whose sum is the activation exactly: hi = bf16(x), mid = bf16(x - hi),
// lo = x - hi - mid; both differences are exact in fp32 and the last one fits bf16 (24 significant bits = 8 + 8 + 8,
// rounding to nearest leaves at most 16, then at most 7).  A bf16 kernel run on the 3 M rows then computes the fp32
// projection with exact products.  out: [3][M][out_stride].  A non-finite activation stays in hi alone.
__global__ __launch_bounds__(256) void split_rows_bf16_kernel(const float* __restrict__ x, uint32_t m, uint32_t k,
                                                              uint32_t x_stride, uint16_t* __restrict__ out,
                                                              uint32_t out_stride) {
    const uint32_t row = blockIdx.y;
    for (uint32_t c = blockIdx.x * 256 + threadIdx.x; c < k; c += gridDim.x * 256) {
        const float v = x[(size_t)row * x_stride + c];
        uint16_t part[3] = {f32_to_bf16_rne(v), 0, 0};
        // a finite v above the largest bf16 would round to infinity: its high part is the largest bf16 instead, and the
        // remainder splits like any other
        if (v - v == 0.0f && (part[0] & 0x7FFFu) == 0x7F80u) part[0] = (uint16_t)((part[0] & 0x8000u) | 0x7F7Fu);
        const float high = __uint_as_float((uint32_t)part[0] << 16);
        if (v - v == 0.0f) {                                // finite
            float r = v - high;
#pragma unroll
            for (int p = 1; p < 3; p++) {
                part[p] = f32_to_bf16_rne(r);
                r -= __uint_as_float((uint32_t)part[p] << 16);
            }
        }
#pragma unroll
        for (int p = 0; p < 3; p++) out[((size_t)p * m + row) * out_stride + c] = part[p];
    }
}

// y[r] = the sum over the parts of split_rows_bf16_kernel of their partial projections, smallest part first
__global__ __launch_bounds__(256) void sum_parts_rows_kernel(const float* __restrict__ yp, uint32_t parts, uint32_t m, uint32_t n,
                                                             void* __restrict__ y, int y_dtype, uint32_t y_stride) {
    const uint32_t row = blockIdx.y;
    for (uint32_t c = blockIdx.x * 256 + threadIdx.x; c < n; c += gridDim.x * 256) {
        float v = yp[((size_t)(parts - 1) * m + row) * n + c];
        for (uint32_t p = parts - 1; p-- > 0;) v += yp[((size_t)p * m + row) * n + c];
        const size_t o = (size_t)row * y_stride + c;
        if (y_dtype == MI355Q_F32) ((float*)y)[o] = v;
        else if (y_dtype == MI355Q_BF16) ((uint16_t*)y)[o] = f32_to_bf16_rne(v);
        else ((uint16_t*)y)[o] = f32_to_f16_rne(v);
    }
}

mi355q_status launch_split_rows_bf16(hipStream_t s, const void* x, int x_dtype, uint32_t m, uint32_t k, uint32_t x_stride,
                                     uint16_t* out, uint32_t out_stride) {
    if (m > 65535u) return fail(MI355Q_ERR_SHAPE, "more than 65535 activation rows");
    uint32_t gx = (k + 255) / 256;
    if (gx > 256) gx = 256;
    if (x_dtype != MI355Q_F32) return fail(MI355Q_ERR_INVALID_ARGUMENT, "only fp32 rows are split into bf16 rows");
    split_rows_bf16_kernel<<<dim3(gx, m), dim3(256), 0, s>>>((const float*)x, m, k, x_stride, out, out_stride);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

mi355q_status launch_sum_parts_rows(hipStream_t s, const float* yp, uint32_t parts, uint32_t m, uint32_t n, void* y, int y_dtype,
                                    uint32_t y_stride) {
    if (m > 65535u) return fail(MI355Q_ERR_SHAPE, "more than 65535 rows");
    uint32_t gx = (n + 255) / 256;
    if (gx > 256) gx = 256;
    sum_parts_rows_kernel<<<dim3(gx, m), dim3(256), 0, s>>>(yp, parts, m, n, y, y_dtype, y_stride);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

mi355q_status launch_split_f32_bf16x2(hipStream_t s, const float* x, uint32_t m, uint32_t k, uint32_t x_stride, uint16_t* hi,
                                      uint16_t* lo, uint32_t out_stride) {
    if (out_stride == 0) out_stride = k;
    if (m > 65535u) return fail(MI355Q_ERR_SHAPE, "more than 65535 activation rows");
    uint32_t gx = (k / 4 + 255) / 256;
    if (gx > 64) gx = 64;
    split_f32_bf16x2_kernel<<<dim3(gx, m), dim3(256), 0, s>>>(x, m, k, x_stride, hi, lo, out_stride);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

mi355q_status launch_dequant_bf16(hipStream_t s, const WView& w, uint16_t* out) { return launch_dequant<MI355Q_BF16>(s, w, out); }
mi355q_status launch_dequant_f32(hipStream_t s, const WView& w, float* out) { return launch_dequant<MI355Q_F32>(s, w, out); }
mi355q_status launch_dequant_f16(hipStream_t s, const WView& w, uint16_t* out) { return launch_dequant<MI355Q_F16>(s, w, out); }

// ------------------------------------------------------------------------------ generic GEMV
// grid (ceil(N/4), M); one wavefront per output row, lanes stride over the codes of the row.
template <int XD, int YD>
__global__ __launch_bounds__(256) void gemv_generic_kernel(WView w, const void* __restrict__ x,
                                                           void* __restrict__ y, uint32_t x_stride,
                                                           uint32_t y_stride) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t row = blockIdx.x * 4 + wave;
    const uint32_t m = blockIdx.y;
    if (row >= w.n) return;  // whole wavefront leaves together
    const size_t xoff = (size_t)m * x_stride;
    float sum = 0.0f;
    for (uint32_t b = 0; b < w.blocks_per_row; b++) {
        float scale, zero;
        load_scale_zero(w, row, b, scale, zero);
        for (uint32_t e = lane; e < w.group; e += 64) {
            const uint32_t c = b * w.group + e;
            const float wt = scale * (float)load_code(w, row, c) + zero;
            sum += wt * load_act<XD>(x, xoff + c);
        }
    }
    sum = wave_reduce_sum(sum);
    if (lane == 0) store_out<YD>(y, (size_t)m * y_stride + row, sum);
}

template <int XD>
static mi355q_status launch_generic_y(hipStream_t s, const WView& w, const void* x, void* y,
                                      int y_dtype, uint32_t m, uint32_t xs, uint32_t ys) {
    dim3 grid((w.n + 3) / 4, m), block(256);
    switch (y_dtype) {
    case MI355Q_F16: gemv_generic_kernel<XD, MI355Q_F16><<<grid, block, 0, s>>>(w, x, y, xs, ys); break;
    case MI355Q_BF16: gemv_generic_kernel<XD, MI355Q_BF16><<<grid, block, 0, s>>>(w, x, y, xs, ys); break;
    default: gemv_generic_kernel<XD, MI355Q_F32><<<grid, block, 0, s>>>(w, x, y, xs, ys); break;
    }
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

mi355q_status launch_gemv_generic(hipStream_t s, const WView& w, const void* x, int x_dtype, void* y,
                                  int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride) {
    if (m > 65535u) return fail(MI355Q_ERR_INVALID_ARGUMENT, "generic kernel supports M <= 65535");
    switch (x_dtype) {
    case MI355Q_F16: return launch_generic_y<MI355Q_F16>(s, w, x, y, y_dtype, m, x_stride, y_stride);
    case MI355Q_BF16: return launch_generic_y<MI355Q_BF16>(s, w, x, y, y_dtype, m, x_stride, y_stride);
    default: return launch_generic_y<MI355Q_F32>(s, w, x, y, y_dtype, m, x_stride, y_stride);
    }
}

// ------------------------------------------------------------------------------------ argmax
// One workgroup of 1024 threads.  Each thread scans i = tid, tid+1024, ... with a strict '>'
// from (-inf, index 0); partial results merge with "greater value, or equal value and lower
// index", so the winner is the lowest index holding the maximum, and NaN never wins.
template <int D>
__global__ __launch_bounds__(1024) void argmax_kernel(const void* __restrict__ logits, uint32_t n,
                                                      int32_t* __restrict__ result) {
    __shared__ float s_val[16];
    __shared__ uint32_t s_idx[16];
    float best = -INFINITY;
    uint32_t bidx = 0;
    for (uint32_t i = threadIdx.x; i < n; i += 1024) {
        const float v = load_act<D>(logits, i);
        if (v > best) { best = v; bidx = i; }
    }
    wave_argmax(best, bidx);
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) { s_val[wave] = best; s_idx[wave] = bidx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        float bv = s_val[0];
        uint32_t bi = s_idx[0];
        for (int i = 1; i < 16; i++)
            if (s_val[i] > bv || (s_val[i] == bv && s_idx[i] < bi)) { bv = s_val[i]; bi = s_idx[i]; }
        result[0] = (int32_t)bi;
    }
}

// Second step of the fused output head: the maximum of the packed (ordered value, ~row) keys the projection's
// workgroups left behind, one key each; 0 means "no finite candidate".  Keys order by value first and by lower
// row second, so the plain maximum is the lowest index holding the maximum.
__global__ __launch_bounds__(1024) void argmax_finish_kernel(const unsigned long long* __restrict__ partial, uint32_t count,
                                                             int32_t* __restrict__ result) {
    __shared__ unsigned long long s_key[16];
    unsigned long long best = 0ull;
    for (uint32_t i = threadIdx.x; i < count; i += 1024) {
        const unsigned long long k = partial[i];
        best = k > best ? k : best;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const uint32_t hi = (uint32_t)__shfl_xor((int)(best >> 32), off, 64);
        const uint32_t lo = (uint32_t)__shfl_xor((int)(best & 0xFFFFFFFFull), off, 64);
        const unsigned long long o = ((unsigned long long)hi << 32) | lo;
        best = o > best ? o : best;
    }
    if ((threadIdx.x & 63) == 0) s_key[threadIdx.x >> 6] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < 16; i++) best = s_key[i] > best ? s_key[i] : best;
        result[0] = best ? (int32_t)(0xFFFFFFFFu - (uint32_t)(best & 0xFFFFFFFFull)) : 0;
    }
}

mi355q_status launch_argmax_finish(hipStream_t s, const unsigned long long* partial, uint32_t count, int32_t* token_out) {
    argmax_finish_kernel<<<dim3(1), dim3(1024), 0, s>>>(partial, count, token_out);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

// First step of the two-launch argmax for long vectors: one packed (ordered value, ~index) key per workgroup, the
// same key the fused output head leaves behind (-0 counts as +0, NaN and -inf never contribute).
template <int D>
__global__ __launch_bounds__(256) void argmax_partial_kernel(const void* __restrict__ logits, uint32_t n,
                                                             unsigned long long* __restrict__ partial) {
    __shared__ unsigned long long s_key[4];
    unsigned long long best = 0ull;
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += gridDim.x * 256u) {
        const float v = load_act<D>(logits, i);
        if (v > -INFINITY) {
            const uint32_t u = __float_as_uint(v + 0.0f);
            const uint32_t key = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
            const unsigned long long pk = ((unsigned long long)key << 32) | (unsigned long long)(0xFFFFFFFFu - i);
            best = pk > best ? pk : best;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const uint32_t hi = (uint32_t)__shfl_xor((int)(best >> 32), off, 64);
        const uint32_t lo = (uint32_t)__shfl_xor((int)(best & 0xFFFFFFFFull), off, 64);
        const unsigned long long o = ((unsigned long long)hi << 32) | lo;
        best = o > best ? o : best;
    }
    if ((threadIdx.x & 63) == 0) s_key[threadIdx.x >> 6] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < 4; i++) best = s_key[i] > best ? s_key[i] : best;
        partial[blockIdx.x] = best;
    }
}

// One workgroup for short vectors; for long ones (a vocabulary) up to 256 workgroups leave one key each in
// `partial` (at least 256 entries; may be null, then the single workgroup runs) and a second launch picks the token.
mi355q_status launch_argmax(hipStream_t s, const void* logits, int dtype, uint32_t n, int32_t* token_out,
                            unsigned long long* partial) {
    if (partial && n >= 16384) {
        uint32_t groups = (n + 1023) / 1024;
        if (groups > 256) groups = 256;
        switch (dtype) {
        case MI355Q_F16: argmax_partial_kernel<MI355Q_F16><<<dim3(groups), dim3(256), 0, s>>>(logits, n, partial); break;
        case MI355Q_BF16: argmax_partial_kernel<MI355Q_BF16><<<dim3(groups), dim3(256), 0, s>>>(logits, n, partial); break;
        default: argmax_partial_kernel<MI355Q_F32><<<dim3(groups), dim3(256), 0, s>>>(logits, n, partial); break;
        }
        MI355Q_HIP(hipGetLastError());
        return launch_argmax_finish(s, partial, groups, token_out);
    }
    switch (dtype) {
    case MI355Q_F16: argmax_kernel<MI355Q_F16><<<dim3(1), dim3(1024), 0, s>>>(logits, n, token_out); break;
    case MI355Q_BF16: argmax_kernel<MI355Q_BF16><<<dim3(1), dim3(1024), 0, s>>>(logits, n, token_out); break;
    default: argmax_kernel<MI355Q_F32><<<dim3(1), dim3(1024), 0, s>>>(logits, n, token_out); break;
    }
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

}  // namespace mi355q
