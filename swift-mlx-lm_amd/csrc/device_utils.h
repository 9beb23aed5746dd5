// Device helpers shared by the kernel translation units (gfx950, wave64).
#pragma once

#include <type_traits>
#include <utility>

#include "common.h"

namespace mi355q {

// Native vectors (not the HIP uint4 struct): register arrays of these are reliably kept in VGPRs.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
// Calls f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>): a loop whose index is a
// compile-time constant inside the body.
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// Code at compile-time bit position POS of a lane chunk held in WPL registers.
template <int POS, int BITS, int WPL>
__device__ __forceinline__ uint32_t extract_code(const uint32_t (&w)[WPL]) {
    constexpr int word = POS >> 5, sh = POS & 31;
    constexpr uint32_t mask = (1u << BITS) - 1u;
    if constexpr (sh + BITS <= 32) {
        return (w[word] >> sh) & mask;
    } else {
        return __builtin_amdgcn_alignbit(w[word + 1], w[word], sh) & mask;
    }
}


// ---- number formats ------------------------------------------------------------------------
__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
__device__ __forceinline__ float f16_to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }

// bits + 0x7FFF + lsb, >> 16: the reference's host/MSL rule
// (Sources/MetalCompiler/BFloat16.swift:25-32, Generator/MetalSourceGenerator.swift:50-56).
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    const uint32_t u = __float_as_uint(f);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ uint16_t f32_to_f16_rne(float f) {
    return __builtin_bit_cast(uint16_t, (_Float16)f);
}

// Eight f16 values (four words) as two bf16 vectors whose sum is each value exactly: hi = the upper eight significant
// bits (the fp32 form cut after its upper half), lo = value - hi (at most three significant bits, so its upper half is
// all of it).  Non-finite values stay in hi alone.
__device__ __forceinline__ void f16x8_to_bf16_hi_lo(const u32x4& v, u32x4& hi, u32x4& lo) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t h[4], l[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float f0 = f16_to_f32((uint16_t)(w[i] & 0xFFFFu)), f1 = f16_to_f32((uint16_t)(w[i] >> 16));
        const uint32_t h0 = __float_as_uint(f0) & 0xFFFF0000u, h1 = __float_as_uint(f1) & 0xFFFF0000u;
        float l0 = f0 - __uint_as_float(h0), l1 = f1 - __uint_as_float(h1);
        l0 = (f0 - f0 == 0.0f) ? l0 : 0.0f;
        l1 = (f1 - f1 == 0.0f) ? l1 : 0.0f;
        h[i] = __builtin_amdgcn_perm(h1, h0, 0x07060302u);
        l[i] = __builtin_amdgcn_perm(__float_as_uint(l1), __float_as_uint(l0), 0x07060302u);
    }
    hi.x = h[0]; hi.y = h[1]; hi.z = h[2]; hi.w = h[3];
    lo.x = l[0]; lo.y = l[1]; lo.z = l[2]; lo.w = l[3];
}

// activation(gate) * up of the gated MLP (SwiGLU: silu; GEGLU: tanh-approximated GELU), on a gate and an up value that
// are first rounded to the buffer type `dtype`, as the reference's elementwise kernel reads them from buffers of that
// type (Sources/MetalCompiler/Generator/MetalSourceGenerator+NormAndElementwise.swift:196-249); fp32 arithmetic, the
// caller rounds the product to the output type.
__device__ __forceinline__ float round_to_dtype(float v, uint32_t dtype) {
    if (dtype == MI355Q_BF16) return bf16_to_f32(f32_to_bf16_rne(v));
    if (dtype == MI355Q_F16) return f16_to_f32(f32_to_f16_rne(v));
    return v;
}
// 1 / (1 + exp(-t)) on the hardware's 2^x and reciprocal (one unit in the last place each); the rounding of the product
// t * log2(e), which would grow with |t|, is put back to first order.  Within 4e-7 relative of the formula; exp and
// an IEEE division (45 instructions an output with the roundings, against 20) were what the activation cost the
// epilogues of the matrix-core kernels.
__device__ __forceinline__ float sigmoid_f32(float t) {
    const float p = t * -1.4426950408889634f;
    const float lost = __builtin_fmaf(t, -1.4426950408889634f, -p);        // exact: what the product's rounding dropped
    const float e = __builtin_amdgcn_exp2f(p) * __builtin_fmaf(lost, 0.6931471805599453f, 1.0f);   // (inf stays inf)
    return __builtin_amdgcn_rcpf(1.0f + e);
}
// swiglu: g * sigmoid(g) * u.  gelu_gated: 0.5 g (1 + tanh(y)) u with y = 0.7978845608 (g + 0.044715 g^3), which is
// g * sigmoid(2 y) * u, the identity 0.5 (1 + tanh(y)) = sigmoid(2 y).
__device__ __forceinline__ float gated_value(float gate, float up, uint32_t activation, uint32_t dtype) {
    const float g = round_to_dtype(gate, dtype), u = round_to_dtype(up, dtype);
    const float t = activation == MI355Q_GATED_GELU_TANH ? 1.5957691216f * (g + 0.044715f * g * g * g) : g;
    return g * sigmoid_f32(t) * u;
}

__device__ __forceinline__ float sb_to_f32(uint16_t h, uint32_t sb_dtype) {
    return sb_dtype == MI355Q_BF16 ? bf16_to_f32(h) : f16_to_f32(h);
}

template <int D>
__device__ __forceinline__ float load_act(const void* p, size_t i) {
    if constexpr (D == MI355Q_F16) return f16_to_f32(((const uint16_t*)p)[i]);
    else if constexpr (D == MI355Q_BF16) return bf16_to_f32(((const uint16_t*)p)[i]);
    else return ((const float*)p)[i];
}

template <int D>
__device__ __forceinline__ void store_out(void* p, size_t i, float v) {
    if constexpr (D == MI355Q_F16) ((uint16_t*)p)[i] = f32_to_f16_rne(v);
    else if constexpr (D == MI355Q_BF16) ((uint16_t*)p)[i] = f32_to_bf16_rne(v);
    else ((float*)p)[i] = v;
}

// ---- one code / one block header, either layout ---------------------------------------------
// q_k = (stream >> k*bits) & mask over the LSB-first bit stream
// (Sources/MetalCompiler/STAF/QuantizationFormat.swift:1044-1257).
__device__ __forceinline__ uint32_t load_code(const WView& w, uint32_t row, uint32_t c) {
    const uint32_t mask = (1u << w.bits) - 1u;
    if (w.layout == MI355Q_LAYOUT_PLANES) {
        const uint32_t* rowp = w.codes + (size_t)row * w.code_stride;
        const uint64_t bit = (uint64_t)c * w.bits;
        const uint32_t word = (uint32_t)(bit >> 5), sh = (uint32_t)(bit & 31);
        uint32_t v = rowp[word] >> sh;
        if (sh + w.bits > 32) v |= rowp[word + 1] << (32 - sh);
        return v & mask;
    }
    if (w.layout == MI355Q_LAYOUT_TILE16) {
        // record (row / 16, c / 128): lane kq*16 + row%16 holds word j = codes (j/2)*64 + kq*16 + (j%2)*8 .. +8
        // with nibbles stored as (c0,c2,c4,c6,c1,c3,c5,c7)
        const uint32_t o = c & 127u, g = o >> 6, in_g = o & 63u, kq = in_g >> 4, j = g * 2 + ((in_g >> 3) & 1u);
        const uint32_t e = in_g & 7u, nib = (e >> 1) + 4u * (e & 1u);
        const uint32_t* rec = w.tiles + ((size_t)(row >> 4) * (w.k >> 7) + (c >> 7)) * 288u;
        return (rec[(kq * 16u + (row & 15u)) * 4u + j] >> (4u * nib)) & 0xFu;
    }
    const uint32_t b = c / w.group, e = c - b * w.group;
    const uint8_t* qs = w.blocks + ((size_t)row * w.blocks_per_row + b) * w.bytes_per_block + 4;
    const uint32_t bit = e * w.bits, byte = bit >> 3, sh = bit & 7;
    uint32_t v = qs[byte];
    if (sh + w.bits > 8) v |= (uint32_t)qs[byte + 1] << 8;
    return (v >> sh) & mask;
}

__device__ __forceinline__ void load_scale_zero(const WView& w, uint32_t row, uint32_t b, float& scale,
                                                float& zero) {
    if (w.layout == MI355Q_LAYOUT_PLANES) {
        const size_t g = (size_t)row * w.blocks_per_row + b;
        scale = sb_to_f32(w.scales[g], w.sb_dtype);
        zero = sb_to_f32(w.biases[g], w.sb_dtype);
    } else if (w.layout == MI355Q_LAYOUT_TILE16) {
        const uint32_t* rec = w.tiles + ((size_t)(row >> 4) * (w.k >> 7) + (b >> 1)) * 288u;
        const uint32_t szw = rec[256u + (row & 15u) * 2u + (b & 1u)];
        scale = sb_to_f32((uint16_t)(szw & 0xFFFFu), w.sb_dtype);
        zero = sb_to_f32((uint16_t)(szw >> 16), w.sb_dtype);
    } else {
        const uint16_t* hdr =
            (const uint16_t*)(w.blocks + ((size_t)row * w.blocks_per_row + b) * w.bytes_per_block);
        scale = f16_to_f32(hdr[0]);
        zero = f16_to_f32(hdr[1]);
    }
}

// ---- wavefront reductions (all 64 lanes must be active) -------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

// Sum over the 64 lanes; every lane returns the total.  Four DPP steps inside each row of 16
// lanes (quad swap, quad-pair swap, half-row mirror, row mirror), then the four row totals are
// read with readlane.
__device__ __forceinline__ float wave_reduce_sum(float v) {
    v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_f32<0x141>(v);  // row_half_mirror
    v += dpp_f32<0x140>(v);  // row_mirror
    const int iv = __float_as_int(v);
    return (__int_as_float(__builtin_amdgcn_readlane(iv, 0)) + __int_as_float(__builtin_amdgcn_readlane(iv, 16))) +
           (__int_as_float(__builtin_amdgcn_readlane(iv, 32)) + __int_as_float(__builtin_amdgcn_readlane(iv, 48)));
}

// Value of lane (lane ^ MASK).  Quad permutes and the 8-lane rotation are DPP modifiers, 4 and 16
// go through the swizzle crossbar, 32 through the permute crossbar; none touches LDS memory.
template <int MASK>
__device__ __forceinline__ float lane_xor(float v) {
    if constexpr (MASK == 1) return dpp_f32<0xB1>(v);        // quad_perm [1,0,3,2]
    else if constexpr (MASK == 2) return dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
    else if constexpr (MASK == 8) return dpp_f32<0x128>(v);  // row_ror:8
    else if constexpr (MASK == 4) return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x101F));
    else if constexpr (MASK == 16) return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F));
    else return __shfl_xor(v, 32, 64);
}

// Reduces B per-lane partial sums (B rows, B a power of two <= 64) across the wavefront at once:
// each stage halves the number of live values by letting the two lanes of a pair each keep one
// row and hand the other over.  On return, lane l holds the complete sum of row (l & (B-1)).
// About 3B operations instead of the 12B of B separate reductions.
template <int B, int MASK = 1>
__device__ __forceinline__ float transpose_reduce(float (&p)[B], uint32_t lane) {
    if constexpr (B == 1) {
        float v = p[0];
        if constexpr (MASK <= 1) v += lane_xor<1>(v);
        if constexpr (MASK <= 2) v += lane_xor<2>(v);
        if constexpr (MASK <= 4) v += lane_xor<4>(v);
        if constexpr (MASK <= 8) v += lane_xor<8>(v);
        if constexpr (MASK <= 16) v += lane_xor<16>(v);
        if constexpr (MASK <= 32) v += lane_xor<32>(v);
        return v;
    } else {
        float q[B / 2];
        const bool odd = (lane & MASK) != 0;
#pragma unroll
        for (int i = 0; i < B / 2; i++) {
            const float keep = odd ? p[2 * i + 1] : p[2 * i];
            const float send = odd ? p[2 * i] : p[2 * i + 1];
            q[i] = keep + lane_xor<MASK>(send);
        }
        return transpose_reduce<B / 2, MASK * 2>(q, lane);
    }
}

// (value, index) maximum with "greater, or equal and lower index"; every lane ends with the result.
__device__ __forceinline__ void wave_argmax(float& v, uint32_t& idx) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(v, off, 64);
        const uint32_t oi = (uint32_t)__shfl_xor((int)idx, off, 64);
        if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
    }
}

}  // namespace mi355q
