// Decode GEMV over the split-plane layout (uint32 code words + scale plane + bias plane),
// bf16 or f16 activations, 1 <= M <= 8.  HBM-bound by design:
//
//   * every lane owns one "lane chunk" of a row per K-step: WPL consecutive code words
//     (128-bit load for 2/4/8-bit, 96-bit for 3/6-bit, so straddling codes never cross lanes);
//     a wavefront therefore reads 64*WPL*4 contiguous bytes of one row per load instruction;
//   * a wavefront owns a run of consecutive rows, carries R of them at once and keeps its loads
//     D pipeline steps ahead of the arithmetic in a register ring;
//   * activations are staged once per workgroup in LDS, already permuted into the pair order
//     the unpacker produces, laid out [m][k-step][piece][lane] so reads are conflict-free b128;
//   * codes become 16-bit float pairs carrying a magic offset, with no int->float conversion, and go
//     through v_dot2 against the staged activation pairs (fp32 accumulate).  XA = 0: bf16 pairs
//     (128 + q) for bf16 activations.  XA = 1: f16 pairs for f16 activations.  In f16 a 4-bit field
//     needs no shift when it sits in bits
//     0-3 or 4-7 of a half-word ((w & 0x00F000F0) | 0x6400 is 1024 + 16 q), so a word of eight
//     codes costs one shift and four and-ors instead of three and four; 2-bit fields take five
//     positions per half-word unshifted; 8-bit codes become pairs with one byte permute;
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

// Weights are read exactly once per launch: non-temporal loads keep them from displacing the
// activations and each other in the caches.
#ifdef MI355Q_GEMV_NO_NT
#define MI355Q_STREAM_LOAD(p) (*(p))
#else
#define MI355Q_STREAM_LOAD(p) __builtin_nontemporal_load(p)
#endif

namespace mi355q {

constexpr int kGemvMaxSegments = 3;

// One launch covers up to three weight matrices that share K, format and activations (q+k+v,
// gate+up).  Wavefronts are dealt to the matrices whole: matrix i owns the wavefronts
// [wave_end[i-1], wave_end[i]), so a wavefront resolves its matrix once and then runs the
// single-matrix code on that matrix's rows.
struct GemvArgs {
    const uint32_t* codes[kGemvMaxSegments];
    const uint32_t* sz[kGemvMaxSegments];      // packed (scale | bias << 16) word per group
    void* y[kGemvMaxSegments];                 // [M, y_stride[i]] in y_dtype (may be null when only logits are wanted)
    uint32_t wave_end[kGemvMaxSegments];       // cumulative wavefront counts; unused entries repeat the last
    uint32_t seg_rows[kGemvMaxSegments];       // N_i
    uint32_t y_stride[kGemvMaxSegments];
    const uint16_t* x;       // bf16 or f16 [M, x_stride]
    float* logits;           // optional fp32 [N] copy (M == 1, single segment)
    int32_t* token_out;      // ARGMAX only
    unsigned long long* scratch;  // ARGMAX only: one packed (ordered value, ~row) key per workgroup; 0 = no candidate
    uint32_t k, m;
    uint32_t x_stride;
    uint32_t code_stride, sz_stride;   // 32-bit words between consecutive rows
    uint32_t nc;             // K-steps per row = ceil(K / (64*CPL))
    uint32_t rows_per_wave;  // consecutive rows owned by one wavefront
    uint32_t y_dtype, sb_dtype;
    uint32_t x_dtype;        // MI355Q_BF16 or MI355Q_F16 (f16 needs XA = 1)
    uint32_t gated;          // gated launches (GATED kernels): mi355q_gated_activation of the epilogue
#ifdef MI355Q_GEMV_TIMELINE
    unsigned long long* timeline;   // measurement build only: five 100 MHz time stamps and the hardware id per workgroup
#endif
};

// Host-side choice of kernel variant and launch shape.
struct GemvCfg {
    int r, mt;          // rows per pipeline step, activation rows (1, 2, 4, 8)
    bool argmax;
    int waves, depth;   // wavefronts per workgroup, prefetch ring depth
    int xreg;           // 0: activations read from LDS each step; 1/2: register-resident (K-steps per row)
    int xa;             // 0: bf16 activations and arithmetic; 1: f16
    bool rows;          // the static-structure kernel (gemv_rows_kernel) with `nct` K-steps per row, `br` rows per pass
    int nct, br;
    bool gated;         // rows kernel over (gate, up) row pairs with the gated activation as epilogue
    uint32_t grid, rows_per_wave, nc;
    size_t lds;
};

// Which instantiations of the static-structure kernel exist: the formats of the reference's default kernel set
// plus the group-64 widths of the bit-width sweep; f16 activations for the default set; the fused arg-max tail
// for rows of one or two K-steps (output heads have short rows and many of them).
constexpr bool gemv_rows_has_format(int bits, int group) {
    return (bits == 4 && (group == 64 || group == 128)) || (bits == 8 && (group == 32 || group == 64)) ||
           ((bits == 2 || bits == 3 || bits == 6) && group == 64);
}
constexpr bool gemv_rows_has_f16(int bits, int group) { return (bits == 4 || bits == 8) && gemv_rows_has_format(bits, group); }
constexpr bool gemv_rows_has_argmax(int nct, int br) { return (nct == 1 && br >= 4) || (nct == 2 && br >= 2); }
constexpr bool gemv_rows_has_shape(int nct, int br) {
    return (nct == 1 && (br == 1 || br == 2 || br == 4 || br == 8)) || (nct == 2 && (br == 1 || br == 2 || br == 4)) ||
           ((nct == 3 || nct == 4) && (br == 1 || br == 2)) || (nct == 7 && br == 1);
}
// Two to four activation rows on the static-structure kernel: 4-bit codes with bf16 activations.  Two rows: the shapes
// the chooser gives whole matrices (one pass of four rows of one K-step, of two rows of two to four, one row of seven;
// one row of two K-steps for matrices of few rows).  Three and four rows: rows of two K-steps (K up to 4096), where
// matrices are small enough for this kernel's short start to beat the matrix-core kernel.
constexpr bool gemv_rows_has_batch(int bits, int group, int nct, int br, int mt) {
    if (bits != 4 || (group != 64 && group != 128)) return false;
    if (mt == 2) return (nct == 1 && br == 4) || (nct >= 2 && nct <= 4 && br == 2) || (nct == 2 && br == 1) || (nct == 7 && br == 1);
    if (mt == 3 || mt == 4) return nct == 2 && (br == 1 || br == 2);
    return false;
}
// wavefronts per workgroup: four (measured best for rows of up to four K-steps at every bit width: with eight or
// sixteen, more wavefronts wait at the staging barrier), eight for rows of seven K-steps, whose staged copy is 28 KiB
constexpr int gemv_rows_waves(int nct) { return nct <= 4 ? 4 : 8; }

template <int BITS> struct GemvGeo;
template <> struct GemvGeo<2> { static constexpr int WPL = 4, CPL = 64; static constexpr bool PAIRS = true; };
template <> struct GemvGeo<4> { static constexpr int WPL = 4, CPL = 32; static constexpr bool PAIRS = true; };
template <> struct GemvGeo<8> { static constexpr int WPL = 4, CPL = 16; static constexpr bool PAIRS = false; };
template <> struct GemvGeo<3> { static constexpr int WPL = 3, CPL = 32; static constexpr bool PAIRS = false; };
template <> struct GemvGeo<6> { static constexpr int WPL = 3, CPL = 16; static constexpr bool PAIRS = false; };
template <> struct GemvGeo<5> { static constexpr int WPL = 5, CPL = 32; static constexpr bool PAIRS = false; };

// Small batches (MT = 2 or 4 activation rows): weight rows carried per pipeline step and ring depth.
// Two rows per step halve the LDS reads of the activations, but only 4- and 6-bit codes leave room
// for them in the register file at MT = 4 (the other widths would spill to scratch memory).
constexpr int gemv_batch_rows(int bits, int group, int mt) {
    if (mt == 2) return (bits == 2 && group == 16) ? 1 : 2;
    return (bits == 4 || bits == 6) ? 2 : 1;
}
constexpr int gemv_batch_depth(int bits, int group, int mt) {
    return (mt == 2 || gemv_batch_rows(bits, group, mt) == 1) ? 4 : 2;
}

// Element (within a lane chunk) that lands in half `which` of staged pair `i`.
template <int BITS>
__host__ __device__ constexpr int pair_elem(int i, int which) {
    if (BITS == 4) return 8 * (i / 4) + (i % 4) + 4 * which;    // word j: (c_p, c_{p+4})
    if (BITS == 2) return 16 * (i / 8) + (i % 8) + 8 * which;   // word j: (c_p, c_{p+8})
    return 2 * i + which;                                       // natural order
}

// f16 arithmetic on 2- and 4-bit codes: the field of staged pair i is used where it sits in its half-word, so
// the f16 pair reads 1024 + mult * q.  mult by pair: 4-bit (1, 16, 1, 16); 2-bit (1, 4, 16, 64, 256, 1, 4, 16),
// the last three after one shift by ten.  The dot products of pairs with the same mult share an accumulator
// ("class"), and  sum q x = sum_c (dot_c - 1024 Sx_c) / mult_c.
template <int BITS> __host__ __device__ constexpr int f16_classes() { return BITS == 4 ? 2 : BITS == 2 ? 5 : 1; }
template <int BITS> __host__ __device__ constexpr int f16_pair_class(int i) {
    if (BITS == 4) return i & 1;
    if (BITS == 2) return (i % 8) < 5 ? (i % 8) : (i % 8) - 5;
    return 0;
}
template <int BITS> __host__ __device__ constexpr int f16_class_shift(int c) { return BITS == 4 ? 4 * c : BITS == 2 ? 2 * c : 0; }

typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2_t;

__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), acc,
                                           false);
}
__device__ __forceinline__ float dot2_f16(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, a), __builtin_bit_cast(f16x2_t, b), acc, false);
}
template <int XA>
__device__ __forceinline__ float dot2_x(uint32_t a, uint32_t b, float acc) {
    if constexpr (XA == 1) return dot2_f16(a, b, acc);
    else return dot2_bf16(a, b, acc);
}

// One wavefront owns `rows_per_wave` consecutive rows and walks them R at a time, one K-step
// (64 lane chunks) per pipeline step.  Every wavefront runs the same number of steps (rows past
// the end are clamped for loading and masked for storing), so the kernel has no data-dependent
// control flow around its loads:
//   1. the activation loads are issued first (vector loads return in issue order, so they must
//      not queue behind the weight stream),
//   2. then D steps of weight loads -- for short rows that is the wavefront's whole share --
//   3. the activations are permuted into LDS behind an LDS-only barrier while the weights are
//      still in flight,
//   4. a software pipeline (prologue / steady loop / epilogue over a register ring of D steps)
//      does the arithmetic as the data lands,
//   5. row results are parked one per lane and written with a single coalesced store at the end:
//      a store inside the loop would share the wait counter with the loads and drain the ring.
// XREG = 1 or 2 means rows are exactly that many K-steps long and the wavefront keeps its
// activation slice in registers; XREG = 0 re-reads the slice from LDS at every step
// (conflict-free 128-bit reads shared by the R rows).
// XA = 0: bf16 activations and bf16 code pairs; XA = 1: f16 activations and f16 code pairs.
template <int BITS, int GROUP, int R, int MT, bool ARGMAX, int WAVES, int D, int XREG, int XA>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(MT == 1 ? 4 : 2)))
void gemv_planes_kernel(GemvArgs a) {
    using G = GemvGeo<BITS>;
    constexpr int WPL = G::WPL, CPL = G::CPL;
    constexpr int Q = CPL / 8;                          // uint4 pieces (8 codes) per lane chunk
    constexpr int SR = CPL < GROUP ? CPL : GROUP;       // codes of one group inside a lane chunk
    constexpr int NSR = CPL / SR;                       // sub-runs (groups touched) per lane chunk
    constexpr int KC = 64 * CPL;                        // codes per wavefront K-step
    // 3-, 5- and 6-bit codes are fed to v_dot2 like the others: the field fits the mantissa next to the magic offset
    constexpr bool SMALL_FIELD = BITS == 3 || BITS == 5 || BITS == 6;
    constexpr bool DOT2 = XA == 1 || G::PAIRS || SMALL_FIELD;             // else (8-bit, bf16 arithmetic): fp32 FMA
    constexpr bool MULTI = XA == 1 && G::PAIRS;                           // f16 arithmetic on fields used in place
    constexpr int NCLS = MULTI ? f16_classes<BITS>() : 1;
    constexpr int NF = MULTI ? 2 : 1;                   // staged floats per sub-run: Sx [, 1024 * sum_c Sx_c / mult_c]
    constexpr float OFS = XA == 1 ? 1024.0f : DOT2 ? 128.0f : 0.0f;       // magic offset carried by the code pairs
    constexpr int XC = XREG ? XREG : 1;                 // K-steps cached in registers
    static_assert(XREG == 0 || (MT == 1 && R == 1), "register-resident activations are for M == 1, R == 1");
    static_assert(XREG == 0 || D % XREG == 0, "ring depth must be a multiple of the K-steps per row");

    extern __shared__ u32x4 smem[];
    const uint32_t NC = a.nc;
    u32x4* xs = smem;                                      // [MT][NC][Q][64]
    float* sxs = (float*)(smem + (size_t)MT * NC * Q * 64); // [MT][NC][NSR][NF][64]

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    // the wavefront index is uniform: keep it (and everything derived from it) in scalar registers
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    // matrix of this wavefront (scalar select chain, once), then rows local to that matrix
    const uint32_t gw = blockIdx.x * WAVES + wave;
    const bool in1 = gw >= a.wave_end[0], in2 = gw >= a.wave_end[1];
    const uint32_t* const seg_codes = in2 ? a.codes[2] : in1 ? a.codes[1] : a.codes[0];
    const uint32_t* const seg_sz = in2 ? a.sz[2] : in1 ? a.sz[1] : a.sz[0];
    void* const seg_y = in2 ? a.y[2] : in1 ? a.y[1] : a.y[0];
    const uint32_t seg_ys = in2 ? a.y_stride[2] : in1 ? a.y_stride[1] : a.y_stride[0];
    const uint32_t seg_n = in2 ? a.seg_rows[2] : in1 ? a.seg_rows[1] : a.seg_rows[0];
    const uint32_t row0 = (gw - (in2 ? a.wave_end[1] : in1 ? a.wave_end[0] : 0u)) * a.rows_per_wave;
    const uint32_t nsteps = (a.rows_per_wave / R) * NC;     // same for every wavefront, >= 1

    struct Pref {
        uint32_t w[R][WPL];
        uint32_t sz[R][NSR];
    };

    // Unconditional loads: rows past N and lane chunks past K are clamped to valid addresses.
    // A clamped lane chunk meets activations staged as zero, a clamped row is never stored.
    // Addresses are "scalar row base + per-lane offset": the row part is wavefront-uniform.
    auto lane_offsets = [&](uint32_t c, uint32_t& code_off, uint32_t (&sz_off)[NSR]) {
        uint32_t chunk = c * 64 + lane;                     // lane-chunk index inside the row
        chunk = (uint64_t)chunk * CPL < a.k ? chunk : 0;
        code_off = chunk * WPL;
#pragma unroll
        for (int sr = 0; sr < NSR; sr++) sz_off[sr] = (chunk * CPL + sr * SR) / GROUP;
    };
    auto issue_at = [&](uint32_t rg, uint32_t code_off, const uint32_t (&sz_off)[NSR], Pref& p) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            uint32_t row = row0 + rg * R + r;
            row = row < seg_n ? row : seg_n - 1;
            const uint32_t* rowp = seg_codes + (size_t)row * a.code_stride;    // scalar
            const uint32_t* szp = seg_sz + (size_t)row * a.sz_stride;          // scalar
            if constexpr (WPL == 4) {
                const u32x4 v = MI355Q_STREAM_LOAD((const u32x4*)(rowp + code_off));
                p.w[r][0] = v.x; p.w[r][1] = v.y; p.w[r][2] = v.z; p.w[r][3] = v.w;
            } else {
#pragma unroll
                for (int i = 0; i < WPL; i++) p.w[r][i] = MI355Q_STREAM_LOAD(rowp + code_off + i);
            }
#pragma unroll
            for (int sr = 0; sr < NSR; sr++) p.sz[r][sr] = MI355Q_STREAM_LOAD(szp + sz_off[sr]);
        }
    };
    // per-lane offsets of the K-steps a ring slot can hold, precomputed when rows are XREG steps long
    uint32_t pre_code_off[XC];
    uint32_t pre_sz_off[XC][NSR];
    if constexpr (XREG != 0) {
#pragma unroll
        for (int cc = 0; cc < XC; cc++) lane_offsets((uint32_t)cc, pre_code_off[cc], pre_sz_off[cc]);
    }
    // CJ: compile-time K-step of the slot (XREG != 0); c: run-time K-step otherwise
    auto issue = [&](uint32_t rg, uint32_t c, Pref& p, auto CJ) {
        if constexpr (XREG != 0) {
            constexpr int cj = decltype(CJ)::value % XC;
            issue_at(rg, pre_code_off[cj], pre_sz_off[cj], p);
        } else {
            uint32_t code_off, sz_off[NSR];
            lane_offsets(c, code_off, sz_off);
            issue_at(rg, code_off, sz_off, p);
        }
    };

    // ---- staging helpers: one task = one lane chunk of one activation row ---------------------
    // Tasks are dealt to wavefronts whole: wave task tw = m * NC + cc covers the 64 lane chunks of
    // K-step cc of activation row m, so (m, cc) and every bound check on them stay scalar.
    const uint32_t nwt = (uint32_t)MT * NC;
    auto task_coords = [&](uint32_t tw, uint32_t& m, uint32_t& cc) {
        if constexpr (MT == 1) { m = 0; cc = tw; }
        else { m = tw / NC; cc = tw - m * NC; }
    };
    auto stage_load = [&](uint32_t tw, uint32_t (&d)[CPL / 2]) {
        uint32_t m, cc;
        task_coords(tw, m, cc);
        const uint64_t kbase = (uint64_t)cc * KC + (uint64_t)lane * CPL;
        const bool valid = tw < nwt && m < a.m && kbase < a.k;
        const u32x4* src = (const u32x4*)(a.x + (valid ? (size_t)m * a.x_stride + kbase : 0));
#pragma unroll
        for (int i = 0; i < Q; i++) {
            const u32x4 v = src[i];                         // clamped address: always readable
            d[4 * i + 0] = valid ? v.x : 0; d[4 * i + 1] = valid ? v.y : 0;
            d[4 * i + 2] = valid ? v.z : 0; d[4 * i + 3] = valid ? v.w : 0;
        }
    };
    auto stage_store = [&](uint32_t tw, const uint32_t (&d)[CPL / 2]) {
        if (tw >= nwt) return;                              // LDS writes only inside this (scalar) branch
        uint32_t m, cc;
        task_coords(tw, m, cc);
        uint32_t pw[CPL / 2];                               // staged pairs, in the order the unpacker produces them
        {
            // 16-bit elements as they are: staged pair i = (element e0, element e1), one byte permute of two dwords
            static_for<CPL / 2>([&](auto I) {
                constexpr int i = decltype(I)::value;
                constexpr int e0 = pair_elem<BITS>(i, 0), e1 = pair_elem<BITS>(i, 1);
                static_assert((e0 & 1) == (e1 & 1) || e1 == e0 + 1, "pair halves come from the same half-word");
                if constexpr (e1 == e0 + 1 && (e0 & 1) == 0) pw[i] = d[e0 >> 1];
                else pw[i] = __builtin_amdgcn_perm(d[e1 >> 1], d[e0 >> 1], (e0 & 1) ? 0x07060302u : 0x05040100u);
            });
        }
        static_for<Q>([&](auto P) {
            constexpr int i = decltype(P)::value;
            u32x4 o;
            o.x = pw[4 * i + 0]; o.y = pw[4 * i + 1]; o.z = pw[4 * i + 2]; o.w = pw[4 * i + 3];
            xs[((size_t)(m * NC + cc) * Q + i) * 64 + lane] = o;
        });
        // per sub-run: the sum of its activations (dot2 against the pair (1, 1)) and, for fields used in place,
        // 1024 * sum_c Sx_c / mult_c (dot2 against the pair (1024 / mult, 1024 / mult) of each staged pair)
        constexpr uint32_t kOnes = XA == 1 ? 0x3C003C00u : 0x3F803F80u;
        static_for<NSR>([&](auto S) {
            constexpr int sr = decltype(S)::value;
            float sx = 0.0f, px = 0.0f;
            static_for<CPL / 2>([&](auto I) {
                constexpr int i = decltype(I)::value;
                if constexpr (pair_elem<BITS>(i, 0) / SR == sr) {
                    sx = dot2_x<XA>(pw[i], kOnes, sx);
                    if constexpr (MULTI) {
                        // 1024 >> shift as an f16 pair: 1024 = 0x6400, each halving lowers the exponent field by one
                        constexpr uint32_t h = 0x6400u - ((uint32_t)f16_class_shift<BITS>(f16_pair_class<BITS>(i)) << 10);
                        px = dot2_f16(pw[i], h | (h << 16), px);
                    }
                }
            });
            float* const cell = sxs + ((size_t)(m * NC + cc) * NSR + sr) * NF * 64 + lane;
            cell[0] = sx;
            if constexpr (MULTI) cell[64] = px;
        });
    };
    auto lds_barrier = [&]() {      // LDS-only: the weight loads in flight must not be waited for here
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    };

    // ---- 1. activation loads first ------------------------------------------------------------
    constexpr int TE = 1;                                   // early staging tasks per wavefront
    uint32_t dearly[TE][CPL / 2];
#pragma unroll
    for (int t = 0; t < TE; t++) stage_load(wave + t * WAVES, dearly[t]);
    __builtin_amdgcn_sched_barrier(0);                      // pinned: the scheduler must not sink them below the weight loads

    // ---- 2. the first D steps of weight loads -------------------------------------------------
    // Steps past the last one repeat it (same addresses, so they hit in L2 and their data is
    // never used); this keeps every load unconditional.
    Pref ring[D];
    uint32_t irg = 0, ic = 0, istep = 0;                    // next step to issue
    auto advance = [&]() {
        if (istep + 1 < nsteps) {
            istep++;
            if (++ic == NC) { ic = 0; irg++; }
        }
    };
    static_for<D>([&](auto J) {
        constexpr int j = decltype(J)::value;
        issue(irg, ic, ring[j], J);
        advance();
    });

    // ---- 3. permute the activations into LDS (waits only for the loads of step 1) -------------
#pragma unroll
    for (int t = 0; t < TE; t++) stage_store(wave + t * WAVES, dearly[t]);
    for (uint32_t tw = wave + TE * WAVES; tw < nwt; tw += WAVES) {
        uint32_t dl[CPL / 2];                               // long rows / batches: the remaining tasks
        stage_load(tw, dl);
        stage_store(tw, dl);
    }
    lds_barrier();

    // ---- optional register-resident activation slice (M == 1, rows of XREG K-steps) -----------
    u32x4 xr[XC][Q];
    float sxr[XC][NSR][NF];
    if constexpr (XREG != 0) {
#pragma unroll
        for (int cc = 0; cc < XC; cc++) {
#pragma unroll
            for (int p = 0; p < Q; p++) xr[cc][p] = xs[((size_t)cc * Q + p) * 64 + lane];
#pragma unroll
            for (int sr = 0; sr < NSR; sr++)
#pragma unroll
                for (int f = 0; f < NF; f++) sxr[cc][sr][f] = sxs[(((size_t)cc * NSR + sr) * NF + f) * 64 + lane];
        }
    }

    // The pair masks live in SGPRs and the magic pair in a VGPR, all opaque to the optimiser, so that
    // (w & mask) | magic is one v_and_or_b32 instead of an AND and an OR with literals (a VOP3
    // instruction takes no literal and a single scalar operand on this target).
    uint32_t k_magic = XA == 1 ? 0x64006400u : 0x43004300u;
    asm volatile("" : "+v"(k_magic));
    uint32_t k_mask[NCLS];
#pragma unroll
    for (int c = 0; c < NCLS; c++) {
        k_mask[c] = (BITS == 4 ? 0x000F000Fu : 0x00030003u) << (MULTI ? f16_class_shift<BITS>(c) : 0);
        asm volatile("" : "+s"(k_mask[c]));
    }

    float acc[R][MT];
    float res[MT];                   // lane i parks the result of the wavefront's i-th row
#pragma unroll
    for (int m = 0; m < MT; m++) {
        res[m] = 0.0f;
#pragma unroll
        for (int r = 0; r < R; r++) acc[r][m] = 0.0f;
    }

    unsigned long long best = 0ull;  // ARGMAX, per lane: packed (ordered value, ~row); 0 = nothing seen
    uint32_t rg = 0, c = 0;          // step being computed
    constexpr int BR = XREG ? D / XC : 1;   // rows completed per ring pass when rows are XREG steps long
    float part[BR];                  // their per-lane partial sums, reduced together
#pragma unroll
    for (int i = 0; i < BR; i++) part[i] = 0.0f;

    auto flush = [&](uint32_t first_local, uint32_t count) {   // rows [first_local, +count) -> memory
        const uint32_t row = row0 + first_local + lane;
        if (lane < count && row < seg_n) {
            void* const yb = seg_y;
            const uint32_t ys = seg_ys, lrow = row;
#pragma unroll
            for (int m = 0; m < MT; m++) {
                if ((uint32_t)m < a.m) {
                    const float v = res[m];
                    if (yb) {
                        const size_t o = (size_t)m * ys + lrow;
                        if (a.y_dtype == MI355Q_F32) ((float*)yb)[o] = v;
                        else if (a.y_dtype == MI355Q_BF16) ((uint16_t*)yb)[o] = f32_to_bf16_rne(v);
                        else ((uint16_t*)yb)[o] = f32_to_f16_rne(v);
                    }
                    if (a.logits && m == 0) a.logits[row] = v;
                }
            }
            if constexpr (ARGMAX) {
                const float v = res[0];
                if (v > -INFINITY) {                         // NaN and -inf never contribute
                    const uint32_t u = __float_as_uint(v + 0.0f);   // -0 -> +0
                    const uint32_t key = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
                    const unsigned long long pk =
                        ((unsigned long long)key << 32) | (unsigned long long)(0xFFFFFFFFu - row);
                    best = pk > best ? pk : best;
                }
            }
        }
    };

    // J: ring slot.  When rows are XREG steps long the K-step index of a slot is a compile-time
    // constant (cj) and so is the slot at which a row completes.
    auto compute = [&](const Pref& cur, auto J) {
        constexpr int cj = XREG ? decltype(J)::value % XC : 0;
        // ---- one K-step of R rows ----------------------------------------------------------
        float dot[R][MT][NSR][NCLS];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int m = 0; m < MT; m++)
#pragma unroll
                for (int sr = 0; sr < NSR; sr++)
#pragma unroll
                    for (int cl = 0; cl < NCLS; cl++) dot[r][m][sr][cl] = 0.0f;

        static_for<Q>([&](auto P) {
            constexpr int p = decltype(P)::value;
            constexpr int sr = (p * 8) / SR;
            u32x4 xv[MT];
            if constexpr (XREG != 0) {
                xv[0] = xr[cj][p];
            } else {
#pragma unroll
                for (int m = 0; m < MT; m++) xv[m] = xs[((size_t)(m * NC + c) * Q + p) * 64 + lane];
            }

            if constexpr (DOT2) {
#pragma unroll
                for (int r = 0; r < R; r++) {
                    uint32_t pr[4];
                    if constexpr (MULTI && BITS == 4) {
                        // fields 0 and 1 of each half-word in place, fields 2 and 3 after one shift
                        const uint32_t wv = cur.w[r][p], w8 = wv >> 8;
                        pr[0] = (wv & k_mask[0]) | k_magic; pr[1] = (wv & k_mask[1]) | k_magic;
                        pr[2] = (w8 & k_mask[0]) | k_magic; pr[3] = (w8 & k_mask[1]) | k_magic;
                    } else if constexpr (MULTI && BITS == 2) {
                        // word p/2; even pieces: fields 0..3 in place; odd pieces: field 4 in place, 5..7 after one shift
                        const uint32_t wv = cur.w[r][p >> 1];
                        if constexpr ((p & 1) == 0) {
                            pr[0] = (wv & k_mask[0]) | k_magic; pr[1] = (wv & k_mask[1]) | k_magic;
                            pr[2] = (wv & k_mask[2]) | k_magic; pr[3] = (wv & k_mask[3]) | k_magic;
                        } else {
                            const uint32_t w10 = wv >> 10;
                            pr[0] = (wv & k_mask[4]) | k_magic; pr[1] = (w10 & k_mask[0]) | k_magic;
                            pr[2] = (w10 & k_mask[1]) | k_magic; pr[3] = (w10 & k_mask[2]) | k_magic;
                        }
                    } else if constexpr (BITS == 4) {
                        const uint32_t wv = cur.w[r][p];
                        pr[0] = (wv & k_mask[0]) | k_magic;
                        pr[1] = ((wv >> 4) & k_mask[0]) | k_magic;
                        pr[2] = ((wv >> 8) & k_mask[0]) | k_magic;
                        pr[3] = ((wv >> 12) & k_mask[0]) | k_magic;
                    } else if constexpr (BITS == 2) {   // word p/2, shifts 2*(4*(p&1) + i)
                        const uint32_t wv = cur.w[r][p >> 1] >> (8 * (p & 1));
                        pr[0] = (wv & k_mask[0]) | k_magic;
                        pr[1] = ((wv >> 2) & k_mask[0]) | k_magic;
                        pr[2] = ((wv >> 4) & k_mask[0]) | k_magic;
                        pr[3] = ((wv >> 6) & k_mask[0]) | k_magic;
                    } else if constexpr (BITS == 8) {
                        // f16 arithmetic: bytes (b0, 0x64, b1, 0x64), the 0x64 taken from the magic word, are the f16 pair (1024 + b0, 1024 + b1)
                        const uint32_t w0 = cur.w[r][2 * p], w1 = cur.w[r][2 * p + 1];
                        pr[0] = __builtin_amdgcn_perm(k_magic, w0, 0x05010500u);
                        pr[1] = __builtin_amdgcn_perm(k_magic, w0, 0x05030502u);
                        pr[2] = __builtin_amdgcn_perm(k_magic, w1, 0x05010500u);
                        pr[3] = __builtin_amdgcn_perm(k_magic, w1, 0x05030502u);
                    } else {
                        // 3-, 5-, 6-bit: codes 2i and 2i+1 of this piece side by side: two field extracts (funnel
                        // shifts where a code straddles words), one shift-or and the magic
                        static_for<4>([&](auto I) {
                            constexpr int i = decltype(I)::value;
                            const uint32_t qa = extract_code<(p * 8 + 2 * i) * BITS, BITS, WPL>(cur.w[r]);
                            const uint32_t qb = extract_code<(p * 8 + 2 * i + 1) * BITS, BITS, WPL>(cur.w[r]);
                            pr[i] = ((qb << 16) | qa) | k_magic;
                        });
                    }
                    // accumulator of each of the piece's four pairs (its class; one accumulator otherwise)
                    constexpr int c0 = MULTI ? f16_pair_class<BITS>(4 * p + 0) : 0, c1 = MULTI ? f16_pair_class<BITS>(4 * p + 1) : 0;
                    constexpr int c2 = MULTI ? f16_pair_class<BITS>(4 * p + 2) : 0, c3 = MULTI ? f16_pair_class<BITS>(4 * p + 3) : 0;
#pragma unroll
                    for (int m = 0; m < MT; m++) {
                        dot[r][m][sr][c0] = dot2_x<XA>(pr[0], xv[m].x, dot[r][m][sr][c0]);
                        dot[r][m][sr][c1] = dot2_x<XA>(pr[1], xv[m].y, dot[r][m][sr][c1]);
                        dot[r][m][sr][c2] = dot2_x<XA>(pr[2], xv[m].z, dot[r][m][sr][c2]);
                        dot[r][m][sr][c3] = dot2_x<XA>(pr[3], xv[m].w, dot[r][m][sr][c3]);
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
                        float dsum = dot[r][m][sr][0];
#pragma unroll
                        for (int e = 0; e < 8; e++) dsum = __builtin_fmaf(qf[e], xf[m][e], dsum);
                        dot[r][m][sr][0] = dsum;
                    }
                }
            }
        });

        // ---- affine form per sub-run: s * sum(q x) + z * sum(x) ---------------------------------
#pragma unroll
        for (int sr = 0; sr < NSR; sr++) {
            float sx[MT], px[MT];
            if constexpr (XREG != 0) {
                sx[0] = sxr[cj][sr][0];
                px[0] = MULTI ? sxr[cj][sr][NF - 1] : 0.0f;
            } else {
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    const float* const cell = sxs + ((size_t)(m * NC + c) * NSR + sr) * NF * 64 + lane;
                    sx[m] = cell[0];
                    px[m] = MULTI ? cell[(NF - 1) * 64] : 0.0f;
                }
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                float s, z;
                const uint32_t szw = cur.sz[r][sr];
                if (a.sb_dtype == MI355Q_BF16) {            // wavefront-uniform: keep it a real branch
                    asm volatile("" ::: "memory");
                    s = __uint_as_float(szw << 16); z = __uint_as_float(szw & 0xFFFF0000u);
                } else {
                    asm volatile("" ::: "memory");
                    s = f16_to_f32((uint16_t)(szw & 0xFFFFu)); z = f16_to_f32((uint16_t)(szw >> 16));
                }
                if constexpr (MULTI) {
                    // sum q x = sum_c dot_c / mult_c - px
#pragma unroll
                    for (int m = 0; m < MT; m++) {
                        float t = dot[r][m][sr][0];
#pragma unroll
                        for (int cl = 1; cl < NCLS; cl++)
                            t = __builtin_fmaf(dot[r][m][sr][cl], 1.0f / (float)(1 << f16_class_shift<BITS>(cl)), t);
                        t -= px[m];
                        acc[r][m] = __builtin_fmaf(s, t, __builtin_fmaf(z, sx[m], acc[r][m]));
                    }
                } else {
                    const float zc = z - OFS * s;
#pragma unroll
                    for (int m = 0; m < MT; m++) acc[r][m] += s * dot[r][m][sr][0] + zc * sx[m];
                }
            }
        }
        if constexpr (XREG != 0) {
            // ---- row complete at a known slot: keep its per-lane partial for the batched reduce -----
            if constexpr (cj == XC - 1) {
                part[decltype(J)::value / XC] = acc[0][0];
                acc[0][0] = 0.0f;
            }
        } else {
            // ---- rows complete: reduce across the wavefront, park the result in its lane ---------
            if (c == NC - 1) {
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const uint32_t local = rg * R + r;
#pragma unroll
                    for (int m = 0; m < MT; m++) {
                        const float tot = wave_reduce_sum(acc[r][m]);
                        acc[r][m] = 0.0f;
                        res[m] = (lane == (local & 63u)) ? tot : res[m];
                    }
                    // a wavefront that owns more than 64 rows empties its lanes every 64 rows
                    if ((local & 63u) == 63u && local + 1 < a.rows_per_wave) flush(local - 63u, 64u);
                }
            }
            if (++c == NC) { c = 0; rg++; }
        }
    };

    // After a ring pass over rows of XREG steps: BR rows are complete; reduce them together and
    // park row (pass*BR + i) in lane ((pass*BR + i) & 63).
    auto finish_pass = [&](uint32_t pass) {
        if constexpr (XREG != 0) {
            const float v = transpose_reduce<BR>(part, lane);
            const uint32_t base = (pass * BR) & 63u;
            res[0] = ((lane & ~(uint32_t)(BR - 1)) == base) ? v : res[0];
            const uint32_t done = (pass + 1) * BR;
            if ((done & 63u) == 0u && done < a.rows_per_wave) flush(done - 64u, 64u);
        }
    };

    // ---- 4. software pipeline: steady loop (compute a slot, refill it), then drain ------------
    const uint32_t groups = (nsteps + D - 1) / D;
    for (uint32_t it = 0; it + 1 < groups; it++) {
        static_for<D>([&](auto J) {
            constexpr int j = decltype(J)::value;
            compute(ring[j], J);
            issue(irg, ic, ring[j], J);
            advance();
        });
        finish_pass(it);
    }
    const uint32_t tail = nsteps - (groups - 1) * D;        // 1..D steps left in the ring
    static_for<D>([&](auto J) {
        constexpr int j = decltype(J)::value;
        if ((uint32_t)j < tail) compute(ring[j], J);
    });
    finish_pass(groups - 1);

    // ---- 5. one coalesced store of the parked results -----------------------------------------
    {
        const uint32_t done = a.rows_per_wave;
        const uint32_t first = (done - 1) & ~63u;           // start of the last (partial) block of 64
        flush(first, done - first);
    }

    if constexpr (ARGMAX) {
        // Per-lane candidates -> wavefront maximum (butterfly on the packed 64-bit key) -> workgroup maximum
        // through LDS -> one plain store per workgroup into the partial-key array.  A one-workgroup launch
        // (argmax_finish_kernel) then picks the token: same-address atomics from thousands of workgroups
        // serialise across the XCDs and would cost more than the projection itself.
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
