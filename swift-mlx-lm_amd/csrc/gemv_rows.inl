// Decode GEMV over the split-plane layout for one activation row (M = 1) when a row is a small, known number
// of K-steps: the fast path of gemv_q{b}_g{g}
// (Sources/MetalCompiler/Generator/MetalSourceGenerator+Quantized.swift:496-575).
//
// Same arithmetic as gemv_planes_kernel (lane chunks, magic-offset code pairs into v_dot2, affine form per
// sub-run, fp32 accumulation); what differs is the shape of the instruction stream:
//   * NCT, the K-steps per row, is a template argument, and a wavefront walks its rows BR at a time ("pass"),
//     so which ring slot holds which (row, K-step) is known at compile time: the steady loop has no index
//     arithmetic, no selects and no branches besides its back edge.  The general kernel spends more scalar
//     instructions and branches per K-step than vector ones, and the scalar unit issues one instruction per
//     wavefront slot just like the vector unit: that bookkeeping, not the unpack, was its ceiling;
//   * a wavefront whose share is at most eight K-steps issues ALL its weight loads before anything else
//     (one pass).  Wavefronts are served oldest first, so the youngest ones get their first bytes late;
//     with every load already in flight they need one memory round trip, not one per pass;
//   * the activation loads are pinned ahead of the weight loads (vector loads return in issue order) and
//     staged in LDS once per workgroup; rows re-read them from LDS (conflict-free 128-bit reads);
//   * row sums are reduced BR at a time (transpose-reduce) and parked one per lane for one coalesced store.
#pragma once

#include "gemv_planes.inl"

namespace mi355q {

// 3-bit codes with bf16 arithmetic, used where they lie.  A field whose lowest bit is bit a <= 4 of its half-word
// stays inside the mantissa of the magic 0x4300, so (w & mask) | magic is the bf16 pair (128 + 2^a0 q0, 128 + 2^a1 q1)
// with no shift; the activations are staged multiplied by 2^-a (exact), and
//   sum (128 + 2^a q) (2^-a x) = sum q x + 128 sum 2^-a x,
// the last sum computed once at staging.  One shift then serves every field it brings to a <= 4.  The 32 codes of a
// lane chunk (three words) pair up as in the table below: thirteen pairs from eight shifts of the three words, one pair
// from the outer half-words of words 0 and 2 (one byte permute), and the codes that straddle a half-word or word
// boundary from two funnel shifts, which bring 5 and 10, 21 and 26 to bits 1 and 16: 27 instructions for 16 pairs
// where extracting code by code took about 4 per pair more (4096 -> 14336: 8.4 -> 7.75 us).  (2-bit codes gain
// nothing from the same treatment -- two shifts instead of seven per word, measured 7.6 us either way -- and pay for
// the scaled staging: they keep their shifts.)
struct InplacePair { int e0, a0, e1, a1; };                 // chunk elements of the low and high half, their bit positions
__host__ __device__ constexpr InplacePair inplace_pair3(int i) {
    constexpr InplacePair t[16] = {{1, 3, 6, 2},   {2, 3, 7, 2},   {3, 3, 8, 2},   {4, 3, 9, 2},      // word 0 >> 0, 3, 6, 9
                                   {11, 1, 16, 0}, {12, 4, 17, 3}, {13, 1, 18, 0}, {14, 4, 19, 3},    // word 1 >> 0, 0, 6, 6
                                   {15, 1, 20, 0}, {22, 2, 28, 4}, {23, 2, 29, 4}, {24, 2, 30, 4},    // word 1 >> 12; word 2 >> 0, 3, 6
                                   {25, 2, 31, 4}, {0, 0, 27, 1},  {5, 1, 10, 0},  {21, 1, 26, 0}};   // word 2 >> 9; permute; funnel shifts
    return t[i & 15];
}

// XA = 0: bf16 activations, bf16 code pairs (128 + q).  XA = 1: f16 activations, f16 code pairs (1024 + mult q,
// fields of 2- and 4-bit codes used where they sit in the half-word, see f16_classes).
// GATED: the launch covers two matrices of equal shape (gate_proj, up_proj: MLPFragment's batched projection,
// Sources/MetalCompiler/Compilable/MLPFragment.swift:7-27).  A wavefront's rows are then "virtual rows" 2 r (row r of
// the first matrix) and 2 r + 1 (row r of the second), so a wavefront that owns a gate row owns the up row of the same
// index, their sums are parked in neighbouring lanes, and the epilogue stores activation(gate) * up: one output
// vector instead of two, and no elementwise launch (generateGatedActivation,
// Generator/MetalSourceGenerator+NormAndElementwise.swift:196-249).
// MT: activation rows (1 to 4).  They share every unpacked code pair: the unpack, the scale / bias conversion and the
// bookkeeping are paid once, the dot products per row, so a further row costs about a fifth of the first.
template <int BITS, int GROUP, int NCT, int BR, int WAVES, int XA, bool SBBF16, bool ARGMAX, bool GATED = false, int MT = 1>
__global__ __launch_bounds__(WAVES * 64) void gemv_rows_kernel(GemvArgs a) {
    static_assert(!(GATED && ARGMAX), "the gated epilogue has no arg-max tail");
    static_assert(MT == 1 || (!GATED && !ARGMAX), "batches have neither the gated epilogue nor the arg-max tail");
    using G = GemvGeo<BITS>;
    constexpr int WPL = G::WPL, CPL = G::CPL;
    constexpr int Q = CPL / 8;
    constexpr int SR = CPL < GROUP ? CPL : GROUP;
    constexpr int NSR = CPL / SR;
    constexpr int KC = 64 * CPL;
    constexpr bool SMALL_FIELD = BITS == 3 || BITS == 5 || BITS == 6;
    constexpr bool DOT2 = XA == 1 || G::PAIRS || SMALL_FIELD;
    constexpr bool MULTI = XA == 1 && G::PAIRS;
    constexpr bool INPLACE = XA == 0 && BITS == 3;                        // see inplace_pair3
    static_assert(!INPLACE || CPL <= GROUP, "fields used in place: one group per lane chunk");
    constexpr int NCLS = MULTI ? f16_classes<BITS>() : 1;
    constexpr int NF = MULTI || INPLACE ? 2 : 1;
    constexpr float OFS = XA == 1 ? 1024.0f : DOT2 ? 128.0f : 0.0f;
    static_assert(BR == 1 || BR == 2 || BR == 4 || BR == 8, "rows per pass: a power of two up to 8");

    extern __shared__ u32x4 smem[];
    u32x4* xs = smem;                                              // [MT][NCT][Q][64]
    float* sxs = (float*)(smem + (size_t)MT * NCT * Q * 64);        // [MT][NCT][NSR][NF][64]

#ifdef MI355Q_GEMV_TIMELINE
    const unsigned long long tl_entry = __builtin_amdgcn_s_memrealtime();
    unsigned long long tl_staged = 0, tl_first = 0;
#endif
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    // matrix of this wavefront (up to three share a launch), then its rows inside that matrix
    const uint32_t gw = blockIdx.x * WAVES + wave;
    const bool in1 = gw >= a.wave_end[0], in2 = gw >= a.wave_end[1];
    const uint32_t* const seg_codes = in2 ? a.codes[2] : in1 ? a.codes[1] : a.codes[0];
    const uint32_t* const seg_sz = in2 ? a.sz[2] : in1 ? a.sz[1] : a.sz[0];
    void* const seg_y = in2 ? a.y[2] : in1 ? a.y[1] : a.y[0];
    const uint32_t seg_n = in2 ? a.seg_rows[2] : in1 ? a.seg_rows[1] : a.seg_rows[0];
    const uint32_t row0 = (gw - (in2 ? a.wave_end[1] : in1 ? a.wave_end[0] : 0u)) * a.rows_per_wave;
    // rows this wavefront owns (0 for the wavefronts past the end of a matrix: they still stage and meet the barrier)
    const uint32_t nrows = row0 < seg_n ? (seg_n - row0 < a.rows_per_wave ? seg_n - row0 : a.rows_per_wave) : 0u;
    const uint32_t last = nrows ? nrows - 1 : 0u;                  // loads past the last row repeat it
    const uint32_t rbase = nrows ? row0 : seg_n - 1;
    const uint32_t cs_bytes = a.code_stride * 4, ss_bytes = a.sz_stride * 4;

    struct Slot {
        uint32_t w[WPL];
        uint32_t sz[NSR];
    };
    // per-lane byte offsets of the lane chunk of every K-step (chunks past K are clamped: they meet activations staged as zero)
    uint32_t voff[NCT], vsz[NCT][NSR];
#pragma unroll
    for (int c = 0; c < NCT; c++) {
        uint32_t chunk = c * 64 + lane;
        chunk = (uint64_t)chunk * CPL < a.k ? chunk : 0;
        voff[c] = chunk * (WPL * 4);
#pragma unroll
        for (int sr = 0; sr < NSR; sr++) vsz[c][sr] = ((chunk * CPL + sr * SR) / GROUP) * 4;
    }
    auto row_ptrs = [&](uint32_t r, const char*& cp, const char*& zp) {    // r: row inside the wavefront's share (scalar)
        r = r < last ? r : last;
        if constexpr (GATED) {
            const uint32_t vrow = rbase + r;
            const uint64_t row = vrow >> 1;
            cp = (const char*)((vrow & 1u) ? a.codes[1] : a.codes[0]) + row * cs_bytes;
            zp = (const char*)((vrow & 1u) ? a.sz[1] : a.sz[0]) + row * ss_bytes;
            return;
        }
        const uint64_t row = rbase + r;
        cp = (const char*)seg_codes + row * cs_bytes;
        zp = (const char*)seg_sz + row * ss_bytes;
    };
    auto issue = [&](const char* cp, const char* zp, int c, Slot& s) {
        if constexpr (WPL == 4) {
            const u32x4 v = MI355Q_STREAM_LOAD((const u32x4*)(cp + voff[c]));
            s.w[0] = v.x; s.w[1] = v.y; s.w[2] = v.z; s.w[3] = v.w;
        } else {
#pragma unroll
            for (int i = 0; i < WPL; i++) s.w[i] = MI355Q_STREAM_LOAD((const uint32_t*)(cp + voff[c]) + i);
        }
#pragma unroll
        for (int sr = 0; sr < NSR; sr++) s.sz[sr] = MI355Q_STREAM_LOAD((const uint32_t*)(zp + vsz[c][sr]));
    };

    // ---- staging: task cc = the 64 lane chunks of K-step cc % NCT of activation row cc / NCT, dealt to wavefronts whole
    auto stage_load = [&](uint32_t cc, uint32_t (&d)[CPL / 2]) {
        const uint32_t xrow = MT == 1 ? 0u : cc / (uint32_t)NCT, step_of = MT == 1 ? cc : cc % (uint32_t)NCT;
        const uint64_t kbase = (uint64_t)step_of * KC + (uint64_t)lane * CPL;
        const bool valid = cc < (uint32_t)(MT * NCT) && kbase < a.k;
        const u32x4* src = (const u32x4*)(a.x + (valid ? (uint64_t)xrow * a.x_stride + kbase : 0));
#pragma unroll
        for (int i = 0; i < Q; i++) {
            const u32x4 v = src[i];                         // clamped address: always readable
            d[4 * i + 0] = valid ? v.x : 0; d[4 * i + 1] = valid ? v.y : 0;
            d[4 * i + 2] = valid ? v.z : 0; d[4 * i + 3] = valid ? v.w : 0;
        }
    };
    auto stage_store = [&](uint32_t cc, const uint32_t (&d)[CPL / 2]) {
        if (cc >= (uint32_t)(MT * NCT)) return;
        uint32_t pw[CPL / 2];                               // staged pairs in the order the unpacker produces them
        float sx_true = 0.0f;                               // INPLACE: sum of the activations before they are scaled
        static_for<CPL / 2>([&](auto I) {
            constexpr int i = decltype(I)::value;
            constexpr int e0 = INPLACE ? inplace_pair3(i).e0 : pair_elem<BITS>(i, 0);
            constexpr int e1 = INPLACE ? inplace_pair3(i).e1 : pair_elem<BITS>(i, 1);
            if constexpr (e1 == e0 + 1 && (e0 & 1) == 0) pw[i] = d[e0 >> 1];
            else {
                constexpr uint32_t h0 = 2 * (e0 & 1), h1 = 4 + 2 * (e1 & 1);      // first byte of each half in the permute
                pw[i] = __builtin_amdgcn_perm(d[e1 >> 1], d[e0 >> 1], ((h1 + 1) << 24) | (h1 << 16) | ((h0 + 1) << 8) | h0);
            }
            if constexpr (INPLACE) {
                sx_true = dot2_x<XA>(pw[i], 0x3F803F80u, sx_true);
                constexpr int a0 = inplace_pair3(i).a0, a1 = inplace_pair3(i).a1;
                if constexpr (a0 != 0 || a1 != 0) {
                    const float lo = __uint_as_float(pw[i] << 16) * (1.0f / (float)(1 << a0));
                    const float hi = __uint_as_float(pw[i] & 0xFFFF0000u) * (1.0f / (float)(1 << a1));
                    pw[i] = __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
                }
            }
        });
        static_for<Q>([&](auto P) {
            constexpr int i = decltype(P)::value;
            u32x4 o;
            o.x = pw[4 * i + 0]; o.y = pw[4 * i + 1]; o.z = pw[4 * i + 2]; o.w = pw[4 * i + 3];
            xs[((size_t)cc * Q + i) * 64 + lane] = o;
        });
        constexpr uint32_t kOnes = XA == 1 ? 0x3C003C00u : 0x3F803F80u;
        if constexpr (INPLACE) {                            // one group per lane chunk: sum x, and 128 sum 2^-a x
            float px = 0.0f;
            static_for<CPL / 2>([&](auto I) { px = dot2_x<XA>(pw[decltype(I)::value], 0x43004300u, px); });
            float* const cell = sxs + (size_t)cc * NF * 64 + lane;
            cell[0] = sx_true;
            cell[64] = px;
        } else
        static_for<NSR>([&](auto S) {
            constexpr int sr = decltype(S)::value;
            float sx = 0.0f, px = 0.0f;
            static_for<CPL / 2>([&](auto I) {
                constexpr int i = decltype(I)::value;
                if constexpr (pair_elem<BITS>(i, 0) / SR == sr) {
                    sx = dot2_x<XA>(pw[i], kOnes, sx);
                    if constexpr (MULTI) {
                        constexpr uint32_t h = 0x6400u - ((uint32_t)f16_class_shift<BITS>(f16_pair_class<BITS>(i)) << 10);
                        px = dot2_f16(pw[i], h | (h << 16), px);
                    }
                }
            });
            float* const cell = sxs + ((size_t)cc * NSR + sr) * NF * 64 + lane;
            cell[0] = sx;
            if constexpr (MULTI) cell[64] = px;
        });
    };

    // ---- 1. activation loads, pinned ahead of the weight loads --------------------------------------------
    uint32_t dearly[CPL / 2];
    stage_load(wave, dearly);
    __builtin_amdgcn_sched_barrier(0);

    // ---- 2. the first pass of weight loads (for most launches: every load of this wavefront) ---------------
    Slot ring[BR][NCT];
    {
        const char *cp[BR], *zp[BR];
#pragma unroll
        for (int j = 0; j < BR; j++) row_ptrs((uint32_t)j, cp[j], zp[j]);
#pragma unroll
        for (int j = 0; j < BR; j++)
            static_for<NCT>([&](auto C) { issue(cp[j], zp[j], decltype(C)::value, ring[j][decltype(C)::value]); });
    }

    // ---- 3. stage the activations behind an LDS-only barrier ----------------------------------------------
    stage_store(wave, dearly);
    for (uint32_t cc = wave + WAVES; cc < (uint32_t)(MT * NCT); cc += WAVES) {
        uint32_t dl[CPL / 2];
        stage_load(cc, dl);
        stage_store(cc, dl);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
#ifdef MI355Q_GEMV_TIMELINE
    tl_staged = __builtin_amdgcn_s_memrealtime();
#endif

    uint32_t k_magic = XA == 1 ? 0x64006400u : 0x43004300u;
    asm volatile("" : "+v"(k_magic));
    uint32_t k_mask[NCLS];
#pragma unroll
    for (int c = 0; c < NCLS; c++) {
        k_mask[c] = (BITS == 4 ? 0x000F000Fu : 0x00030003u) << (MULTI ? f16_class_shift<BITS>(c) : 0);
        asm volatile("" : "+s"(k_mask[c]));
    }
    // INPLACE: the masks of the (low, high) field positions in use
    auto ip_mask_value = [](int a0, int a1) constexpr -> uint32_t { return (7u << a0) | (7u << (16 + a1)); };
    uint32_t m_a = ip_mask_value(3, 2), m_b = ip_mask_value(1, 0), m_c = ip_mask_value(4, 3);
    uint32_t m_d = ip_mask_value(2, 4), m_e = ip_mask_value(0, 1);
    if constexpr (INPLACE) {
        asm volatile("" : "+s"(m_a)); asm volatile("" : "+s"(m_b)); asm volatile("" : "+s"(m_c));
        asm volatile("" : "+s"(m_d)); asm volatile("" : "+s"(m_e));
    }

    // contribution of one K-step of one row: sum over its sub-runs of s * sum(q x) + z * sum(x)
    // (added to out[m] for each of the MT activation rows)
    auto step = [&](const Slot& cur, auto C, float (&out)[MT]) {
        constexpr int c = decltype(C)::value;
        float dot[MT][NSR][NCLS];
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int sr = 0; sr < NSR; sr++)
#pragma unroll
                for (int cl = 0; cl < NCLS; cl++) dot[m][sr][cl] = 0.0f;
        static_for<Q>([&](auto P) {
            constexpr int p = decltype(P)::value;
            constexpr int sr = (p * 8) / SR;
            if constexpr (DOT2) {
                uint32_t pr[4];
                if constexpr (MULTI && BITS == 4) {
                    const uint32_t wv = cur.w[p], w8 = wv >> 8;
                    pr[0] = (wv & k_mask[0]) | k_magic; pr[1] = (wv & k_mask[1]) | k_magic;
                    pr[2] = (w8 & k_mask[0]) | k_magic; pr[3] = (w8 & k_mask[1]) | k_magic;
                } else if constexpr (MULTI && BITS == 2) {
                    const uint32_t wv = cur.w[p >> 1];
                    if constexpr ((p & 1) == 0) {
                        pr[0] = (wv & k_mask[0]) | k_magic; pr[1] = (wv & k_mask[1]) | k_magic;
                        pr[2] = (wv & k_mask[2]) | k_magic; pr[3] = (wv & k_mask[3]) | k_magic;
                    } else {
                        const uint32_t w10 = wv >> 10;
                        pr[0] = (wv & k_mask[4]) | k_magic; pr[1] = (w10 & k_mask[0]) | k_magic;
                        pr[2] = (w10 & k_mask[1]) | k_magic; pr[3] = (w10 & k_mask[2]) | k_magic;
                    }
                } else if constexpr (BITS == 4) {
                    const uint32_t wv = cur.w[p];
                    pr[0] = (wv & k_mask[0]) | k_magic;
                    pr[1] = ((wv >> 4) & k_mask[0]) | k_magic;
                    pr[2] = ((wv >> 8) & k_mask[0]) | k_magic;
                    pr[3] = ((wv >> 12) & k_mask[0]) | k_magic;
                } else if constexpr (BITS == 2) {
                    const uint32_t wv = cur.w[p >> 1] >> (8 * (p & 1));
                    pr[0] = (wv & k_mask[0]) | k_magic;
                    pr[1] = ((wv >> 2) & k_mask[0]) | k_magic;
                    pr[2] = ((wv >> 4) & k_mask[0]) | k_magic;
                    pr[3] = ((wv >> 6) & k_mask[0]) | k_magic;
                } else if constexpr (INPLACE) {
                    const uint32_t w0 = cur.w[0], w1 = cur.w[1], w2 = cur.w[2];
                    if constexpr (p == 0) {
                        pr[0] = (w0 & m_a) | k_magic; pr[1] = ((w0 >> 3) & m_a) | k_magic;
                        pr[2] = ((w0 >> 6) & m_a) | k_magic; pr[3] = ((w0 >> 9) & m_a) | k_magic;
                    } else if constexpr (p == 1) {
                        const uint32_t w6 = w1 >> 6;
                        pr[0] = (w1 & m_b) | k_magic; pr[1] = (w1 & m_c) | k_magic;
                        pr[2] = (w6 & m_b) | k_magic; pr[3] = (w6 & m_c) | k_magic;
                    } else if constexpr (p == 2) {
                        pr[0] = ((w1 >> 12) & m_b) | k_magic; pr[1] = (w2 & m_d) | k_magic;
                        pr[2] = ((w2 >> 3) & m_d) | k_magic; pr[3] = ((w2 >> 6) & m_d) | k_magic;
                    } else {
                        pr[0] = ((w2 >> 9) & m_d) | k_magic;
                        pr[1] = (__builtin_amdgcn_perm(w2, w0, 0x07060100u) & m_e) | k_magic;
                        pr[2] = (__builtin_amdgcn_alignbit(w1, w0, 14) & m_b) | k_magic;
                        pr[3] = (__builtin_amdgcn_alignbit(w2, w1, 30) & m_b) | k_magic;
                    }
                } else if constexpr (BITS == 8) {
                    const uint32_t w0 = cur.w[2 * p], w1 = cur.w[2 * p + 1];
                    pr[0] = __builtin_amdgcn_perm(k_magic, w0, 0x05010500u);
                    pr[1] = __builtin_amdgcn_perm(k_magic, w0, 0x05030502u);
                    pr[2] = __builtin_amdgcn_perm(k_magic, w1, 0x05010500u);
                    pr[3] = __builtin_amdgcn_perm(k_magic, w1, 0x05030502u);
                } else {
                    static_for<4>([&](auto I) {
                        constexpr int i = decltype(I)::value;
                        const uint32_t qa = extract_code<(p * 8 + 2 * i) * BITS, BITS, WPL>(cur.w);
                        const uint32_t qb = extract_code<(p * 8 + 2 * i + 1) * BITS, BITS, WPL>(cur.w);
                        pr[i] = ((qb << 16) | qa) | k_magic;
                    });
                }
                constexpr int c0 = MULTI ? f16_pair_class<BITS>(4 * p + 0) : 0, c1 = MULTI ? f16_pair_class<BITS>(4 * p + 1) : 0;
                constexpr int c2 = MULTI ? f16_pair_class<BITS>(4 * p + 2) : 0, c3 = MULTI ? f16_pair_class<BITS>(4 * p + 3) : 0;
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    const u32x4 xv = xs[((size_t)(m * NCT + c) * Q + p) * 64 + lane];
                    dot[m][sr][c0] = dot2_x<XA>(pr[0], xv.x, dot[m][sr][c0]);
                    dot[m][sr][c1] = dot2_x<XA>(pr[1], xv.y, dot[m][sr][c1]);
                    dot[m][sr][c2] = dot2_x<XA>(pr[2], xv.z, dot[m][sr][c2]);
                    dot[m][sr][c3] = dot2_x<XA>(pr[3], xv.w, dot[m][sr][c3]);
                }
            } else {
                // 8-bit codes with bf16 activations: (128 + q) is not exact in bf16, so fp32 FMA on converted codes
                float qf[8];
                static_for<8>([&](auto E) {
                    constexpr int e = decltype(E)::value;
                    qf[e] = (float)extract_code<(p * 8 + e) * BITS, BITS, WPL>(cur.w);
                });
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    const u32x4 xv = xs[((size_t)(m * NCT + c) * Q + p) * 64 + lane];
                    const float xf[8] = {__uint_as_float(xv.x << 16), __uint_as_float(xv.x & 0xFFFF0000u),
                                         __uint_as_float(xv.y << 16), __uint_as_float(xv.y & 0xFFFF0000u),
                                         __uint_as_float(xv.z << 16), __uint_as_float(xv.z & 0xFFFF0000u),
                                         __uint_as_float(xv.w << 16), __uint_as_float(xv.w & 0xFFFF0000u)};
                    float dsum = dot[m][sr][0];
#pragma unroll
                    for (int e = 0; e < 8; e++) dsum = __builtin_fmaf(qf[e], xf[e], dsum);
                    dot[m][sr][0] = dsum;
                }
            }
        });
#pragma unroll
        for (int sr = 0; sr < NSR; sr++) {
            float s, z;
            const uint32_t szw = cur.sz[sr];
            if constexpr (SBBF16) { s = __uint_as_float(szw << 16); z = __uint_as_float(szw & 0xFFFF0000u); }
            else { s = f16_to_f32((uint16_t)(szw & 0xFFFFu)); z = f16_to_f32((uint16_t)(szw >> 16)); }
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const float* const cell = sxs + ((size_t)(m * NCT + c) * NSR + sr) * NF * 64 + lane;
                const float sx = cell[0];
                if constexpr (INPLACE) {
                    out[m] = __builtin_fmaf(s, dot[m][sr][0] - cell[64], __builtin_fmaf(z, sx, out[m]));
                } else if constexpr (MULTI) {
                    float t = dot[m][sr][0];
#pragma unroll
                    for (int cl = 1; cl < NCLS; cl++)
                        t = __builtin_fmaf(dot[m][sr][cl], 1.0f / (float)(1 << f16_class_shift<BITS>(cl)), t);
                    t -= cell[64];
                    out[m] = __builtin_fmaf(s, t, __builtin_fmaf(z, sx, out[m]));
                } else {
                    out[m] += s * dot[m][sr][0] + (z - OFS * s) * sx;
                }
            }
        }
    };

    float resm[MT];                                          // lane i parks the results of the wavefront's i-th row
#pragma unroll
    for (int m = 0; m < MT; m++) resm[m] = 0.0f;
    auto pass_body = [&](uint32_t pass, auto ISSUE_T) {
        constexpr bool ISSUE = decltype(ISSUE_T)::value;
        float acc[MT][BR];
#pragma unroll
        for (int j = 0; j < BR; j++) {
            const char *cp = nullptr, *zp = nullptr;
            if constexpr (ISSUE) row_ptrs((pass + 1) * BR + j, cp, zp);
            float o[MT];
#pragma unroll
            for (int m = 0; m < MT; m++) o[m] = 0.0f;
            static_for<NCT>([&](auto C) {
                step(ring[j][decltype(C)::value], C, o);
                if constexpr (ISSUE) issue(cp, zp, decltype(C)::value, ring[j][decltype(C)::value]);
            });
#pragma unroll
            for (int m = 0; m < MT; m++) acc[m][j] = o[m];
            asm volatile("" ::: "memory");                  // the next row reads the activations from LDS again (registers stay free)
        }
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const float v = transpose_reduce<BR>(acc[m], lane);    // lane l holds the sum of row (l & (BR - 1)) of this pass
            resm[m] = ((lane & ~(uint32_t)(BR - 1)) == pass * BR) ? v : resm[m];
        }
    };
    const uint32_t passes = (nrows + BR - 1) / BR;
#ifdef MI355Q_GEMV_TIMELINE
    {   // when the first weight words of this wavefront are there
        uint32_t first_word = ring[0][0].w[0];
        asm volatile("s_waitcnt vmcnt(0)" : "+v"(first_word));
        tl_first = __builtin_amdgcn_s_memrealtime();
    }
#endif
    for (uint32_t pass = 0; pass + 1 < passes; pass++) pass_body(pass, std::true_type{});
    if (passes) pass_body(passes - 1, std::false_type{});
#ifdef MI355Q_GEMV_TIMELINE
    if (a.timeline && wave == 0 && lane == 0) {
        unsigned long long* const t = a.timeline + (size_t)blockIdx.x * 6;
        uint32_t hw_id, xcc_id;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw_id));
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc_id));
        t[0] = tl_entry; t[1] = tl_staged; t[2] = tl_first; t[3] = __builtin_amdgcn_s_memrealtime();
        t[4] = hw_id; t[5] = xcc_id;
    }
#endif

    // ---- one coalesced store of the parked results (rows_per_wave <= 64) ------------------------------------
    const float res = resm[0];
    if constexpr (MT > 1) {
        const uint32_t ys = in2 ? a.y_stride[2] : in1 ? a.y_stride[1] : a.y_stride[0];
        if (lane < nrows && seg_y) {
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const size_t o = (size_t)m * ys + row0 + lane;
                if (a.y_dtype == MI355Q_F32) ((float*)seg_y)[o] = resm[m];
                else if (a.y_dtype == MI355Q_BF16) ((uint16_t*)seg_y)[o] = f32_to_bf16_rne(resm[m]);
                else ((uint16_t*)seg_y)[o] = f32_to_f16_rne(resm[m]);
            }
        }
        return;
    }
    if constexpr (GATED) {
        // lanes 2 r and 2 r + 1 hold the gate and the up sum of output row (row0 / 2 + r): both are rounded to the
        // output type first, as the reference's elementwise kernel reads them back from buffers of that type
        const float up_sum = __shfl_down(res, 1, 64);
        if (lane < nrows && !(lane & 1u)) {
            const uint32_t row = (row0 + lane) >> 1;
            const float v = gated_value(res, up_sum, a.gated, a.y_dtype);
            if (a.y_dtype == MI355Q_F32) ((float*)seg_y)[row] = v;
            else if (a.y_dtype == MI355Q_BF16) ((uint16_t*)seg_y)[row] = f32_to_bf16_rne(v);
            else ((uint16_t*)seg_y)[row] = f32_to_f16_rne(v);
        }
        return;
    }
    unsigned long long best = 0ull;
    if (lane < nrows) {
        const uint32_t row = row0 + lane;
        if (seg_y) {
            if (a.y_dtype == MI355Q_F32) ((float*)seg_y)[row] = res;
            else if (a.y_dtype == MI355Q_BF16) ((uint16_t*)seg_y)[row] = f32_to_bf16_rne(res);
            else ((uint16_t*)seg_y)[row] = f32_to_f16_rne(res);
        }
        if (a.logits) a.logits[row] = res;
        if constexpr (ARGMAX) {
            if (res > -INFINITY) {                           // NaN and -inf never contribute
                const uint32_t u = __float_as_uint(res + 0.0f);     // -0 -> +0
                const uint32_t key = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
                best = ((unsigned long long)key << 32) | (unsigned long long)(0xFFFFFFFFu - row);
            }
        }
    }
    if constexpr (ARGMAX) {
        // wavefront maximum of the packed (ordered value, ~row) key, workgroup maximum through LDS, one plain store
        // per workgroup; argmax_finish_kernel picks the token from the partial keys
        __shared__ unsigned long long s_best[WAVES];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const uint32_t hi = (uint32_t)__shfl_xor((int)(best >> 32), off, 64);
            const uint32_t lo = (uint32_t)__shfl_xor((int)(best & 0xFFFFFFFFull), off, 64);
            const unsigned long long o = ((unsigned long long)hi << 32) | lo;
            best = o > best ? o : best;
        }
        if (lane == 0) s_best[wave] = best;
        __syncthreads();
        if (tid == 0) {
            unsigned long long m = s_best[0];
#pragma unroll
            for (int w2 = 1; w2 < WAVES; w2++) m = s_best[w2] > m ? s_best[w2] : m;
            a.scratch[blockIdx.x] = m;
        }
    }
}

}  // namespace mi355q
