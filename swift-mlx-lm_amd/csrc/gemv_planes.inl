// Decode GEMV over the split-plane layout (uint32 code words + scale plane + bias plane),
// bf16 activations, 1 <= M <= 8.  HBM-bound by design:
//
//   * every lane owns one "lane chunk" of a row per K-step: WPL consecutive code words
//     (128-bit load for 2/4/8-bit, 96-bit for 3/6-bit, so straddling codes never cross lanes);
//     a wavefront therefore reads 64*WPL*4 contiguous bytes of one row per load instruction;
//   * a wavefront carries R rows at once and prefetches the next K-step while it computes;
//   * activations are staged once per workgroup in LDS, already permuted into the pair order
//     the unpacker produces, laid out [m][k-step][piece][lane] so reads are conflict-free b128;
//   * 2/4-bit codes become bf16 pairs (128+q) with one and-or each and go through
//     v_dot2_f32_bf16 against the bf16 activation pairs (fp32 accumulate); other widths are
//     extracted with bit-field/funnel ops and accumulated with fp32 FMA;
//   * the affine form is applied per lane chunk:  sum (s*q+z)*x = s*sum(q*x) + z*sum(x), with
//     sum(x) per lane chunk precomputed at staging time;
//   * one DPP/readlane reduction per output row at the end (split-K across the 64 lanes).
//
// Replaces gemv_q{b}_g{g} (Sources/MetalCompiler/Generator/MetalSourceGenerator+Quantized.swift:496-575)
// and, for M > 1, the sequence signature of gemm_q*_g* (:22-156) at small M.
#pragma once

#include <type_traits>
#include <utility>

#include "device_utils.h"

namespace mi355q {

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

struct GemvArgs {
    const uint32_t* codes;
    const uint16_t* scales;
    const uint16_t* biases;
    const uint16_t* x;       // bf16 [M, x_stride]
    void* y;                 // [M, y_stride] in y_dtype (may be null when only logits are wanted)
    float* logits;           // optional fp32 [N] copy (M == 1)
    int32_t* token_out;      // ARGMAX only
    unsigned long long* scratch;  // ARGMAX only: [0] packed max, [1] ticket
    uint32_t n, k, m;
    uint32_t x_stride, y_stride;
    uint32_t words_per_row, blocks_per_row;
    uint32_t nc;             // K-steps per row = ceil(K / (64*CPL))
    uint32_t nrb;            // row blocks = ceil(N / (4*R))
    uint32_t y_dtype, sb_dtype;
};

template <int BITS> struct GemvGeo;
template <> struct GemvGeo<2> { static constexpr int WPL = 4, CPL = 64; static constexpr bool PAIRS = true; };
template <> struct GemvGeo<4> { static constexpr int WPL = 4, CPL = 32; static constexpr bool PAIRS = true; };
template <> struct GemvGeo<8> { static constexpr int WPL = 4, CPL = 16; static constexpr bool PAIRS = false; };
template <> struct GemvGeo<3> { static constexpr int WPL = 3, CPL = 32; static constexpr bool PAIRS = false; };
template <> struct GemvGeo<6> { static constexpr int WPL = 3, CPL = 16; static constexpr bool PAIRS = false; };
template <> struct GemvGeo<5> { static constexpr int WPL = 5, CPL = 32; static constexpr bool PAIRS = false; };

// Element (within a lane chunk) that lands in half `which` of staged pair `i`.
template <int BITS>
__host__ __device__ constexpr int pair_elem(int i, int which) {
    if (BITS == 4) return 8 * (i / 4) + (i % 4) + 4 * which;    // word j: (c_p, c_{p+4})
    if (BITS == 2) return 16 * (i / 8) + (i % 8) + 8 * which;   // word j: (c_p, c_{p+8})
    return 2 * i + which;                                       // natural order
}

typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;

__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), acc,
                                           false);
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

template <int BITS, int GROUP, int R, int MT, bool ARGMAX>
__global__ __launch_bounds__(256) void gemv_planes_kernel(GemvArgs a) {
    using G = GemvGeo<BITS>;
    constexpr int WPL = G::WPL, CPL = G::CPL;
    constexpr int Q = CPL / 8;                          // uint4 pieces (8 codes) per lane chunk
    constexpr int SR = CPL < GROUP ? CPL : GROUP;       // codes of one group inside a lane chunk
    constexpr int NSR = CPL / SR;                       // sub-runs (groups touched) per lane chunk
    constexpr int KC = 64 * CPL;                        // codes per wavefront K-step
    constexpr float OFS = G::PAIRS ? 128.0f : 0.0f;     // magic offset carried by the bf16 codes

    extern __shared__ uint4 smem[];
    const uint32_t NC = a.nc;
    uint4* xs = smem;                                       // [MT][NC][Q][64]
    float* sxs = (float*)(smem + (size_t)MT * NC * Q * 64); // [MT][NC][NSR][64]

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    struct Pref {
        uint32_t w[R][WPL];
        uint16_t s[R][NSR], z[R][NSR];
    };

    auto issue = [&](uint32_t rb, uint32_t c, Pref& p) {
        const uint32_t chunk = c * 64 + lane;               // lane-chunk index inside the row
        const bool live = (uint64_t)chunk * CPL < a.k;
#pragma unroll
        for (int r = 0; r < R; r++) {
            uint32_t row = rb * (4 * R) + wave * R + r;
            row = row < a.n ? row : a.n - 1;                // clamp: results of such rows are dropped
            if (live) {
                const uint32_t* src = a.codes + (size_t)row * a.words_per_row + (size_t)chunk * WPL;
                if constexpr (WPL == 4) {
                    const uint4 v = *(const uint4*)src;
                    p.w[r][0] = v.x; p.w[r][1] = v.y; p.w[r][2] = v.z; p.w[r][3] = v.w;
                } else {
#pragma unroll
                    for (int i = 0; i < WPL; i++) p.w[r][i] = src[i];
                }
#pragma unroll
                for (int sr = 0; sr < NSR; sr++) {
                    const size_t g = (size_t)row * a.blocks_per_row + ((size_t)chunk * CPL + sr * SR) / GROUP;
                    p.s[r][sr] = a.scales[g];
                    p.z[r][sr] = a.biases[g];
                }
            } else {
#pragma unroll
                for (int i = 0; i < WPL; i++) p.w[r][i] = 0;
#pragma unroll
                for (int sr = 0; sr < NSR; sr++) { p.s[r][sr] = 0; p.z[r][sr] = 0; }
            }
        }
    };

    // ---- first weight loads go out before the activations are staged ------------------------
    uint32_t rb = blockIdx.x, c = 0;
    bool have = rb < a.nrb;
    Pref nxt;
    if (have) issue(rb, 0, nxt);

    // ---- stage activations: one task = one lane chunk of one activation row -----------------
    for (uint32_t task = tid; task < (uint32_t)MT * NC * 64; task += 256) {
        const uint32_t l = task & 63, cc = (task >> 6) % NC, m = (task >> 6) / NC;
        const uint64_t kbase = (uint64_t)cc * KC + (uint64_t)l * CPL;
        uint32_t d[CPL / 2];
        if (m < a.m && kbase < a.k) {
            const uint4* src = (const uint4*)(a.x + (size_t)m * a.x_stride + kbase);
#pragma unroll
            for (int i = 0; i < Q; i++) {
                const uint4 v = src[i];
                d[4 * i + 0] = v.x; d[4 * i + 1] = v.y; d[4 * i + 2] = v.z; d[4 * i + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int i = 0; i < CPL / 2; i++) d[i] = 0;
        }
        auto elem = [&](int e) -> uint32_t { return (e & 1) ? (d[e >> 1] >> 16) : (d[e >> 1] & 0xFFFFu); };
#pragma unroll
        for (int i = 0; i < Q; i++) {
            uint4 o;
            o.x = elem(pair_elem<BITS>(4 * i + 0, 0)) | (elem(pair_elem<BITS>(4 * i + 0, 1)) << 16);
            o.y = elem(pair_elem<BITS>(4 * i + 1, 0)) | (elem(pair_elem<BITS>(4 * i + 1, 1)) << 16);
            o.z = elem(pair_elem<BITS>(4 * i + 2, 0)) | (elem(pair_elem<BITS>(4 * i + 2, 1)) << 16);
            o.w = elem(pair_elem<BITS>(4 * i + 3, 0)) | (elem(pair_elem<BITS>(4 * i + 3, 1)) << 16);
            xs[((size_t)(m * NC + cc) * Q + i) * 64 + l] = o;
        }
#pragma unroll
        for (int sr = 0; sr < NSR; sr++) {
            float sx = 0.0f;
#pragma unroll
            for (int e = 0; e < SR; e++) sx += __uint_as_float(elem(sr * SR + e) << 16);
            sxs[((size_t)(m * NC + cc) * NSR + sr) * 64 + l] = sx;
        }
    }
    __syncthreads();

    float acc[R][MT];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int m = 0; m < MT; m++) acc[r][m] = 0.0f;

    unsigned long long best = 0ull;  // ARGMAX: packed (ordered value, ~row); 0 = nothing seen

    while (have) {
        Pref cur = nxt;
        uint32_t c2 = c + 1, rb2 = rb;
        if (c2 == NC) { c2 = 0; rb2 = rb + gridDim.x; }
        const bool have2 = rb2 < a.nrb;
        if (have2) issue(rb2, c2, nxt);

        // ---- one K-step of R rows ----------------------------------------------------------
        float dot[R][MT][NSR];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int m = 0; m < MT; m++)
#pragma unroll
                for (int sr = 0; sr < NSR; sr++) dot[r][m][sr] = 0.0f;

        static_for<Q>([&](auto P) {
            constexpr int p = decltype(P)::value;
            constexpr int sr = (p * 8) / SR;
            uint4 xv[MT];
#pragma unroll
            for (int m = 0; m < MT; m++) xv[m] = xs[((size_t)(m * NC + c) * Q + p) * 64 + lane];

            if constexpr (G::PAIRS) {
#pragma unroll
                for (int r = 0; r < R; r++) {
                    uint32_t pr[4];
                    if constexpr (BITS == 4) {
                        const uint32_t wv = cur.w[r][p];
                        pr[0] = (wv & 0x000F000Fu) | 0x43004300u;
                        pr[1] = ((wv >> 4) & 0x000F000Fu) | 0x43004300u;
                        pr[2] = ((wv >> 8) & 0x000F000Fu) | 0x43004300u;
                        pr[3] = ((wv >> 12) & 0x000F000Fu) | 0x43004300u;
                    } else {  // BITS == 2: word p/2, shifts 2*(4*(p&1) + i)
                        const uint32_t wv = cur.w[r][p >> 1] >> (8 * (p & 1));
                        pr[0] = (wv & 0x00030003u) | 0x43004300u;
                        pr[1] = ((wv >> 2) & 0x00030003u) | 0x43004300u;
                        pr[2] = ((wv >> 4) & 0x00030003u) | 0x43004300u;
                        pr[3] = ((wv >> 6) & 0x00030003u) | 0x43004300u;
                    }
#pragma unroll
                    for (int m = 0; m < MT; m++) {
                        float dsum = dot[r][m][sr];
                        dsum = dot2_bf16(pr[0], xv[m].x, dsum);
                        dsum = dot2_bf16(pr[1], xv[m].y, dsum);
                        dsum = dot2_bf16(pr[2], xv[m].z, dsum);
                        dsum = dot2_bf16(pr[3], xv[m].w, dsum);
                        dot[r][m][sr] = dsum;
                    }
                }
            } else {
                float xf[MT][8];
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    xf[m][0] = __uint_as_float(xv[m].x << 16); xf[m][1] = __uint_as_float(xv[m].x & 0xFFFF0000u);
                    xf[m][2] = __uint_as_float(xv[m].y << 16); xf[m][3] = __uint_as_float(xv[m].y & 0xFFFF0000u);
                    xf[m][4] = __uint_as_float(xv[m].z << 16); xf[m][5] = __uint_as_float(xv[m].z & 0xFFFF0000u);
                    xf[m][6] = __uint_as_float(xv[m].w << 16); xf[m][7] = __uint_as_float(xv[m].w & 0xFFFF0000u);
                }
#pragma unroll
                for (int r = 0; r < R; r++) {
                    float qf[8];
                    qf[0] = (float)extract_code<(p * 8 + 0) * BITS, BITS, WPL>(cur.w[r]);
                    qf[1] = (float)extract_code<(p * 8 + 1) * BITS, BITS, WPL>(cur.w[r]);
                    qf[2] = (float)extract_code<(p * 8 + 2) * BITS, BITS, WPL>(cur.w[r]);
                    qf[3] = (float)extract_code<(p * 8 + 3) * BITS, BITS, WPL>(cur.w[r]);
                    qf[4] = (float)extract_code<(p * 8 + 4) * BITS, BITS, WPL>(cur.w[r]);
                    qf[5] = (float)extract_code<(p * 8 + 5) * BITS, BITS, WPL>(cur.w[r]);
                    qf[6] = (float)extract_code<(p * 8 + 6) * BITS, BITS, WPL>(cur.w[r]);
                    qf[7] = (float)extract_code<(p * 8 + 7) * BITS, BITS, WPL>(cur.w[r]);
#pragma unroll
                    for (int m = 0; m < MT; m++) {
                        float dsum = dot[r][m][sr];
#pragma unroll
                        for (int e = 0; e < 8; e++) dsum = __builtin_fmaf(qf[e], xf[m][e], dsum);
                        dot[r][m][sr] = dsum;
                    }
                }
            }
        });

        // ---- affine form per sub-run: s*dot + (z - OFS*s)*sum(x) -----------------------------
#pragma unroll
        for (int sr = 0; sr < NSR; sr++) {
            float sx[MT];
#pragma unroll
            for (int m = 0; m < MT; m++) sx[m] = sxs[((size_t)(m * NC + c) * NSR + sr) * 64 + lane];
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float s = sb_to_f32(cur.s[r][sr], a.sb_dtype);
                const float z = sb_to_f32(cur.z[r][sr], a.sb_dtype);
                const float zc = z - OFS * s;
#pragma unroll
                for (int m = 0; m < MT; m++) acc[r][m] += s * dot[r][m][sr] + zc * sx[m];
            }
        }

        // ---- row block complete: reduce across the wavefront and store ----------------------
        if (c == NC - 1) {
#pragma unroll
            for (int r = 0; r < R; r++) {
                const uint32_t row = rb * (4 * R) + wave * R + r;
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    const float tot = wave_reduce_sum(acc[r][m]);
                    acc[r][m] = 0.0f;
                    if (row < a.n && (uint32_t)m < a.m) {
                        if (lane == 0) {
                            if (a.y) {
                                const size_t o = (size_t)m * a.y_stride + row;
                                if (a.y_dtype == MI355Q_F32) ((float*)a.y)[o] = tot;
                                else if (a.y_dtype == MI355Q_BF16) ((uint16_t*)a.y)[o] = f32_to_bf16_rne(tot);
                                else ((uint16_t*)a.y)[o] = f32_to_f16_rne(tot);
                            }
                            if (a.logits && m == 0) a.logits[row] = tot;
                        }
                        if constexpr (ARGMAX) {
                            if (m == 0 && tot > -INFINITY) {  // NaN and -inf never contribute
                                const uint32_t u = __float_as_uint(tot + 0.0f);  // -0 -> +0
                                const uint32_t key = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
                                const unsigned long long pk =
                                    ((unsigned long long)key << 32) | (unsigned long long)(0xFFFFFFFFu - row);
                                best = pk > best ? pk : best;
                            }
                        }
                    }
                }
            }
        }
        rb = rb2; c = c2; have = have2;
    }

    if constexpr (ARGMAX) {
        // `best` is wavefront-uniform.  One atomic per wavefront, then a ticket: the workgroup that
        // draws the last ticket publishes the token and leaves the scratch cells zeroed again.
        __shared__ uint32_t s_last;
        if (lane == 0 && best) atomicMax(&a.scratch[0], best);
        __threadfence();
        __syncthreads();
        if (tid == 0) {
            const unsigned long long t = atomicAdd(&a.scratch[1], 1ull);
            s_last = (t == (unsigned long long)gridDim.x - 1ull) ? 1u : 0u;
        }
        __syncthreads();
        if (s_last && tid == 0) {
            __threadfence();
            const unsigned long long pk = atomicExch(&a.scratch[0], 0ull);
            a.token_out[0] = pk ? (int32_t)(0xFFFFFFFFu - (uint32_t)(pk & 0xFFFFFFFFull)) : 0;
            atomicExch(&a.scratch[1], 0ull);
        }
    }
}

}  // namespace mi355q
