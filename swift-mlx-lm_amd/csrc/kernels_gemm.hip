// Prefill GEMM on the matrix cores:  Y[M,N] = X[M,K] * W[N,K]^T  with W either group-affine
// packed codes (dequantised to bf16 on the way into LDS) or a dense bf16 matrix.
//
// Stands in for the reference's two prefill routes in one kernel
//   gemm_q4_g64_f32s / gemm_q8_g32_f32s                      (direct, scalar FMA)
//   dequant_q{b}_g{g}_bf16  +  gemm_bf16_f32s (matmul2d)     (two dispatches + a bf16 scratch)
// (Sources/MetalCompiler/Generator/MetalSourceGenerator+Quantized.swift:22-156,361-416 and
//  MetalSourceGenerator+Linear.swift:18-81), without the scratch round trip.
//
// Shape of the kernel
//   * workgroup tile BM x BN x 64 (one K-tile = one 64-code run, so every row needs at most a
//     couple of (scale, bias) words per K-tile), 4 wavefronts in a 2 x 2 arrangement, each
//     owning a (BM/2) x (BN/2) block of 32x32 accumulators fed by v_mfma_f32_32x32x16_bf16;
//   * LDS holds two stages of [rows][64] bf16 for both operands; a row is 128 bytes = 8 chunks
//     of 16 bytes and chunk c of row r lives at position c ^ (r & 7), which makes both the
//     128-bit stores and the MFMA operand loads (32 rows x one chunk) bank-conflict free;
//   * the next K-tile is fetched into registers while the current one is multiplied; weight
//     words are unpacked, scaled (fp32 fma), rounded to bf16 (v_cvt_pk_bf16_f32) and stored to
//     the other LDS stage, so there is one barrier per K-tile;
//   * workgroup ids are remapped so that the workgroups of one XCD (id % 8) walk the N-tiles of
//     the same M-tile: the activation rows they share stay in that XCD's L2;
//   * fp32 accumulators are rounded once, to the output type, in the epilogue.
#include "device_utils.h"
#include <atomic>

namespace mi355q {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16_t;
typedef __bf16 bf16x2_v __attribute__((ext_vector_type(2)));
typedef float float2_v __attribute__((ext_vector_type(2)));

struct GemmArgs {
    const uint32_t* codes;   // QUANT: [N, K*bits/32]
    const uint32_t* tiles;   // QUANT on the TILE16 layout: records of 16 rows x 128 codes + 32 (scale, bias) words
    const uint32_t* sz;      // QUANT: packed (scale | bias << 16) per group
    const uint16_t* bdense;  // !QUANT: bf16 [N, K]
    const uint16_t* x;       // bf16 [M, xs]
    void* y;
    uint32_t m, n, k, xs, ys;
    uint32_t code_stride, sz_stride;   // 32-bit words between consecutive rows
    uint32_t y_dtype, sb_dtype;
    uint32_t tiles_m, tiles_n;
    uint32_t kblocks;        // TILE16: K / 128
    float* partial;          // split-K: fp32 [splits][M][N] partial results (null when K is not split)
    uint32_t kt_per_split;   // K-tiles per split (blockIdx.y indexes the split)
    unsigned long long* probe;   // optional: [0] shader cycles, [1] 100 MHz ticks that workgroup 0 spent in the kernel
};

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    float2_v v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_v));
}

constexpr int kTileK = 64;            // codes (and bf16 elements) per K-tile
constexpr int kRowBytes = kTileK * 2; // one LDS row

// Byte offset of 16-byte chunk `chunk` of tile row `row`.  The LDS has 64 banks of 4 bytes: a row
// of 128 bytes covers half of them, so two consecutive rows fill all banks and the chunk position
// is rotated by (row / 2) % 8: any 16 consecutive rows reading (or writing) the same logical chunk
// touch 16 different bank groups.
__device__ __forceinline__ uint32_t lds_off(uint32_t row, uint32_t chunk) {
    return row * kRowBytes + ((chunk ^ ((row >> 1) & 7u)) << 4);
}

// STAGES = 2: double-buffered LDS, one barrier per K-tile, one workgroup per CU for the big tiles.
// STAGES = 1: one LDS stage and two barriers per K-tile, sized so that two workgroups share a CU
// (and each SIMD holds two wavefronts): one workgroup's matrix-core phase covers the other's
// dequantisation, LDS fill and barrier.
// WAVES = 4: wavefronts 2 x 2 over the tile, one per SIMD.  WAVES = 8: 2 x 4, two per SIMD, so that
// one wavefront's LDS waits and barrier skew are covered by the other's MFMAs.
template <int BITS, int GROUP, int BM, int BN, bool QUANT, int STAGES, bool SB_BF16, int WAVES, bool T16>
__global__ __launch_bounds__(WAVES * 64, (STAGES == 1 ? 2 : 1)) void qgemm_mfma_kernel(GemmArgs a) {
    constexpr int NT = WAVES * 64;                        // threads
    constexpr int WN = WAVES / 2;                         // wavefronts along N (2 along M)
    constexpr int TM = BM / 2 / 32, TN = BN / WN / 32;    // 32x32 accumulators per wavefront
    constexpr int A_BYTES = BM * kRowBytes, B_BYTES = BN * kRowBytes, STAGE = A_BYTES + B_BYTES;
    constexpr int RPP = NT / 8;                           // tile rows covered by one pass of 16-byte chunks
    constexpr int A_PASSES = BM / RPP;                    // 16-byte chunks per thread for the X tile
    constexpr int TPR = NT / BN;                          // threads per weight row
    constexpr int CPT = kTileK / TPR;                     // codes per thread per K-tile
    constexpr int WPT = QUANT ? CPT * BITS / 32 : 0;      // code words per thread per K-tile
    constexpr int NGT = QUANT ? (CPT > GROUP ? CPT / GROUP : 1) : 0;   // groups a thread touches
    constexpr int B_DENSE_PASSES = BN / RPP;
    static_assert(TPR >= 1 && CPT % 8 == 0, "weight tile does not split over the threads");
    // TILE16 operand: 4-bit g64 records; a thread takes 32 codes (two 16-code quarters) of one row per K-tile
    static_assert(!T16 || (QUANT && BITS == 4 && GROUP == 64 && CPT == 32), "the TILE16 fetch is written for q4 g64, 32 codes per thread");

    extern __shared__ uint4 smem_q[];
    char* lds = (char*)smem_q;

    // ---- tile of this workgroup (XCD-aware order) --------------------------------------------
    const uint32_t total = a.tiles_m * a.tiles_n;
    const uint32_t per_xcd = (total + 7) / 8;
    const uint32_t t_id = (blockIdx.x % 8u) * per_xcd + blockIdx.x / 8u;
    if (t_id >= total) return;
    const uint32_t tm = t_id / a.tiles_n, tn = t_id % a.tiles_n;
    const uint32_t m0 = tm * BM, n0 = tn * BN;

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t wm = wave / WN, wn = wave % WN;
    // clock probe: the first wavefront of workgroup 0 times itself with the shader-clock counter and the
    // constant 100 MHz counter; their ratio is the clock the matrix cores actually ran at
    const bool probing = a.probe != nullptr && blockIdx.x == 0 && blockIdx.y == 0 && wave == 0;
    unsigned long long probe_c0 = 0, probe_r0 = 0;
    if (probing) { probe_c0 = __builtin_readcyclecounter(); probe_r0 = __builtin_amdgcn_s_memrealtime(); }

    // ---- global -> register fetch and register -> LDS fill of one K-tile, in NP parts -----------
    // Part p covers X-tile passes [p*AP, (p+1)*AP) and weight chunks [p*BC, (p+1)*BC) (a chunk is 8
    // codes, 16 bytes of bf16).  The packed weight words of a whole K-tile are fetched together.
    constexpr int NP = kTileK / 16;                        // one part per MFMA k-step
    constexpr int AP = A_PASSES / NP;
    constexpr int BC = QUANT ? (CPT / 8) / NP : B_DENSE_PASSES / NP;
    static_assert(AP >= 1 && BC >= 1, "tile too small to split into parts");
    u32x4 xa[A_PASSES];
    uint32_t wreg[QUANT ? WPT : 1], wnext[QUANT ? WPT : 1];
    uint32_t szreg[QUANT ? NGT : 1], sznext[QUANT ? NGT : 1];
    u32x4 bd[QUANT ? 1 : B_DENSE_PASSES];

    const uint32_t a_row = tid >> 3, a_chunk = tid & 7;       // X tile: 8 threads per row
    const uint32_t b_row = tid / TPR, b_part = tid % TPR;     // W tile: TPR threads per row
    uint32_t b_grow = n0 + b_row;
    b_grow = b_grow < a.n ? b_grow : a.n - 1;

    auto fetch_x = [&](auto P, uint32_t kt) __attribute__((always_inline)) {
        constexpr int part = decltype(P)::value;
        static_for<AP>([&](auto Q) __attribute__((always_inline)) {
            constexpr int p = part * AP + decltype(Q)::value;
            uint32_t gr = m0 + p * RPP + a_row;
            gr = gr < a.m ? gr : a.m - 1;
            xa[p] = *(const u32x4*)(a.x + (size_t)gr * a.xs + kt * kTileK + a_chunk * 8);
        });
    };
    auto fetch_dense = [&](auto P, uint32_t kt) __attribute__((always_inline)) {
        constexpr int part = decltype(P)::value;
        if constexpr (!QUANT) {
            static_for<BC>([&](auto Q) __attribute__((always_inline)) {
                constexpr int p = part * BC + decltype(Q)::value;
                uint32_t gr = n0 + p * RPP + a_row;
                gr = gr < a.n ? gr : a.n - 1;
                bd[p] = *(const u32x4*)(a.bdense + (size_t)gr * a.k + kt * kTileK + a_chunk * 8);
            });
        }
    };
    // packed words + (scale, bias) words of K-tile kt into (w, sz)
    auto fetch_codes = [&](uint32_t kt, uint32_t (&w)[QUANT ? WPT : 1], uint32_t (&sz)[QUANT ? NGT : 1])
                           __attribute__((always_inline)) {
        if constexpr (T16) {
            // K-tile kt is half h of record kt / 2; row b_grow is row n of row tile rt.  Quarter kq of the half
            // sits with lane kq * 16 + n: its words 2h and 2h + 1 hold codes kq * 16 .. + 16 of the K-tile.
            const uint32_t rt = b_grow >> 4, n = b_grow & 15u, h = kt & 1u;
            const uint32_t* rec = a.tiles + ((size_t)rt * a.kblocks + (kt >> 1)) * 288u;
#pragma unroll
            for (int q = 0; q < 2; q++) {
                const u32x2 v = *(const u32x2*)(rec + ((b_part * 2 + q) * 16 + n) * 4 + h * 2);
                w[2 * q] = v.x; w[2 * q + 1] = v.y;
            }
            sz[0] = rec[256 + n * 2 + h];
        } else if constexpr (QUANT) {
            const uint32_t k0 = kt * kTileK;
            const uint32_t* src = a.codes + (size_t)b_grow * a.code_stride + (size_t)kt * (kTileK * BITS / 32) +
                                  b_part * WPT;
            if constexpr (WPT % 4 == 0) {
                static_for<WPT / 4>([&](auto I) __attribute__((always_inline)) {
                    constexpr int i = decltype(I)::value;
                    const u32x4 v = ((const u32x4*)src)[i];
                    w[4 * i + 0] = v.x; w[4 * i + 1] = v.y; w[4 * i + 2] = v.z; w[4 * i + 3] = v.w;
                });
            } else if constexpr (WPT % 2 == 0) {
                static_for<WPT / 2>([&](auto I) __attribute__((always_inline)) {
                    constexpr int i = decltype(I)::value;
                    const u32x2 v = ((const u32x2*)src)[i];
                    w[2 * i + 0] = v.x; w[2 * i + 1] = v.y;
                });
            } else {
                static_for<WPT>([&](auto I) __attribute__((always_inline)) {
                    constexpr int i = decltype(I)::value;
                    w[i] = src[i];
                });
            }
            static_for<NGT>([&](auto G) __attribute__((always_inline)) {
                constexpr int g = decltype(G)::value;
                sz[g] = a.sz[(size_t)b_grow * a.sz_stride + (k0 + b_part * CPT + g * GROUP) / GROUP];
            });
        }
    };
    auto fetch = [&](uint32_t kt) __attribute__((always_inline)) {
        static_for<NP>([&](auto P) __attribute__((always_inline)) { fetch_x(P, kt); fetch_dense(P, kt); });
        fetch_codes(kt, wreg, szreg);
    };

    // ---- register -> LDS (with dequantisation of the weight words) ----------------------------
    auto stash_part = [&](auto P, uint32_t stage) __attribute__((always_inline)) {
        constexpr int part = decltype(P)::value;
        char* As = lds + stage * STAGE;
        char* Bs = As + A_BYTES;
        static_for<AP>([&](auto Q) __attribute__((always_inline)) {
            constexpr int p = part * AP + decltype(Q)::value;
            *(u32x4*)(As + lds_off(p * RPP + a_row, a_chunk)) = xa[p];
        });
        if constexpr (QUANT) {
            static_for<BC>([&](auto C) __attribute__((always_inline)) {
                constexpr int ci = part * BC + decltype(C)::value;     // chunk of 8 codes
                constexpr int g = NGT > 1 ? (ci * 8) / GROUP : 0;
                float s, z;
                const uint32_t szw = szreg[g];
                if constexpr (SB_BF16) {     // compile-time: a branch here would split the pipelined loop body
                    s = __uint_as_float(szw << 16); z = __uint_as_float(szw & 0xFFFF0000u);
                } else {
                    s = f16_to_f32((uint16_t)(szw & 0xFFFFu)); z = f16_to_f32((uint16_t)(szw >> 16));
                }
                float f[8];
                if constexpr (BITS == 4) {
                    // byte-lane conversion: even codes sit in the low nibbles, odd ones in the high
                    const uint32_t w = wreg[ci];
                    const uint32_t lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu;
                    float q[8];
                    asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(q[0]) : "v"(lo));
                    asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(q[1]) : "v"(hi));
                    asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(q[2]) : "v"(lo));
                    asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(q[3]) : "v"(hi));
                    asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(q[4]) : "v"(lo));
                    asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(q[5]) : "v"(hi));
                    asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(q[6]) : "v"(lo));
                    asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(q[7]) : "v"(hi));
                    if constexpr (T16) {
                        // q[i] is nibble i of the word; record words keep their nibbles in the order
                        // (c0,c2,c4,c6,c1,c3,c5,c7), so code e sits in nibble at[e]
                        constexpr int at[8] = {0, 4, 1, 5, 2, 6, 3, 7};
#pragma unroll
                        for (int e = 0; e < 8; e++) f[e] = __builtin_fmaf(s, q[at[e]], z);
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; e++) f[e] = __builtin_fmaf(s, q[e], z);
                    }
                } else {
                    f[0] = __builtin_fmaf(s, (float)extract_code<(ci * 8 + 0) * BITS, BITS, (WPT ? WPT : 1)>(wreg), z);
                    f[1] = __builtin_fmaf(s, (float)extract_code<(ci * 8 + 1) * BITS, BITS, (WPT ? WPT : 1)>(wreg), z);
                    f[2] = __builtin_fmaf(s, (float)extract_code<(ci * 8 + 2) * BITS, BITS, (WPT ? WPT : 1)>(wreg), z);
                    f[3] = __builtin_fmaf(s, (float)extract_code<(ci * 8 + 3) * BITS, BITS, (WPT ? WPT : 1)>(wreg), z);
                    f[4] = __builtin_fmaf(s, (float)extract_code<(ci * 8 + 4) * BITS, BITS, (WPT ? WPT : 1)>(wreg), z);
                    f[5] = __builtin_fmaf(s, (float)extract_code<(ci * 8 + 5) * BITS, BITS, (WPT ? WPT : 1)>(wreg), z);
                    f[6] = __builtin_fmaf(s, (float)extract_code<(ci * 8 + 6) * BITS, BITS, (WPT ? WPT : 1)>(wreg), z);
                    f[7] = __builtin_fmaf(s, (float)extract_code<(ci * 8 + 7) * BITS, BITS, (WPT ? WPT : 1)>(wreg), z);
                }
                u32x4 o;
                o.x = pack_bf16(f[0], f[1]); o.y = pack_bf16(f[2], f[3]);
                o.z = pack_bf16(f[4], f[5]); o.w = pack_bf16(f[6], f[7]);
                *(u32x4*)(Bs + lds_off(b_row, b_part * (CPT / 8) + ci)) = o;
            });
        } else {
            static_for<BC>([&](auto Q) __attribute__((always_inline)) {
                constexpr int p = part * BC + decltype(Q)::value;
                *(u32x4*)(Bs + lds_off(p * RPP + a_row, a_chunk)) = bd[p];
            });
        }
    };
    auto stash = [&](uint32_t stage) __attribute__((always_inline)) {
        static_for<NP>([&](auto P) __attribute__((always_inline)) { stash_part(P, stage); });
    };

    floatx16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // K range of this workgroup: all of K, or one of the splits (blockIdx.y)
    const uint32_t KT_all = a.k / kTileK;
    const uint32_t kt0 = blockIdx.y * a.kt_per_split;
    const uint32_t KT = kt0 + a.kt_per_split < KT_all ? kt0 + a.kt_per_split : KT_all;   // end (exclusive)
    const uint32_t frag_row = lane & 31, frag_half = lane >> 5;
    bf16x8_t af[2][TM], bf[2][TN];
    auto load_frags = [&](auto KK, uint32_t stage) __attribute__((always_inline)) {
        constexpr int kk = decltype(KK)::value;
        const char* As = lds + stage * STAGE;
        const char* Bs = As + A_BYTES;
#pragma unroll
        for (int i = 0; i < TM; i++)
            af[kk & 1][i] = *(const bf16x8_t*)(As + lds_off(wm * (BM / 2) + i * 32 + frag_row, kk * 2 + frag_half));
#pragma unroll
        for (int j = 0; j < TN; j++)
            bf[kk & 1][j] = *(const bf16x8_t*)(Bs + lds_off(wn * (BN / WN) + j * 32 + frag_row, kk * 2 + frag_half));
    };
    auto mfmas = [&](auto KK) __attribute__((always_inline)) {
        constexpr int kk = decltype(KK)::value;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[kk & 1][i], bf[kk & 1][j], acc[i][j], 0, 0, 0);
    };
    // Matrix-core phase of one K-tile: the operand fragments of k-step kk+1 are read from LDS while
    // the MFMAs of k-step kk run (two register sets), so only the first read of a K-tile is exposed.
    auto multiply = [&](uint32_t stage) __attribute__((always_inline)) {
        load_frags(std::integral_constant<int, 0>{}, stage);
        static_for<NP>([&](auto KK) __attribute__((always_inline)) {
            constexpr int kk = decltype(KK)::value;
            if constexpr (kk + 1 < NP) load_frags(std::integral_constant<int, kk + 1>{}, stage);
            __builtin_amdgcn_sched_barrier(0);   // keep the reads of kk+1 ahead of the MFMAs of kk
            mfmas(KK);
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    fetch(kt0);
    if constexpr (STAGES == 2) {
        // Software pipeline over K-tiles, all inside one wavefront's instruction stream: while the
        // MFMAs of K-tile kt run, K-tile kt+1 moves from registers to the other LDS stage (part by
        // part, dequantising) and K-tile kt+2 is fetched into the registers just freed.  Tile
        // indices past the end are clamped: the extra fetches and the extra LDS fill are never read.
        stash(0);
        __syncthreads();
        fetch(kt0 + 1 < KT ? kt0 + 1 : kt0);
        for (uint32_t kt = kt0; kt < KT; kt++) {
            const uint32_t stage = (kt - kt0) & 1;
            const uint32_t k2 = kt + 2 < KT ? kt + 2 : KT - 1;
            load_frags(std::integral_constant<int, 0>{}, stage);
            static_for<NP>([&](auto KK) __attribute__((always_inline)) {
                constexpr int kk = decltype(KK)::value;
                if constexpr (kk + 1 < NP) load_frags(std::integral_constant<int, kk + 1>{}, stage);
                stash_part(KK, stage ^ 1);
                fetch_x(KK, k2);
                fetch_dense(KK, k2);
                if constexpr (kk == 0) fetch_codes(k2, wnext, sznext);
                mfmas(KK);
                // Issue order inside this k-step: the LDS reads for the next k-step first, then the
                // MFMAs with the fill of the other stage (VALU, LDS writes) and the global loads
                // spread between them.
                __builtin_amdgcn_sched_group_barrier(0x100, TM + TN, 0);
#pragma unroll
                for (int q = 0; q < TM * TN; q++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);     // one MFMA
                    __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);     // a few VALU
                    if (q % 2 == 0) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);   // an LDS write
                    if (q % 4 == 1) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // a global load
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            if constexpr (QUANT) {
#pragma unroll
                for (int i = 0; i < WPT; i++) wreg[i] = wnext[i];
#pragma unroll
                for (int g = 0; g < NGT; g++) szreg[g] = sznext[g];
            }
            __syncthreads();
        }
    } else {
        for (uint32_t kt = kt0; kt < KT; kt++) {
            stash(0);
            __syncthreads();
            if (kt + 1 < KT) fetch(kt + 1);      // in flight during the matrix-core phase
            multiply(0);
            __syncthreads();                     // every wavefront is done reading before the next fill
        }
    }

    if (probing) {
        const unsigned long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
        if (lane == 0) { a.probe[0] = c1 - probe_c0; a.probe[1] = r1 - probe_r0; }
    }
    // ---- epilogue: one rounding, to the output type --------------------------------------------
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const uint32_t col = n0 + wn * (BN / WN) + j * 32 + frag_row;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t row = m0 + wm * (BM / 2) + i * 32 + 8 * (r / 4) + 4 * frag_half + (r % 4);
                if (row < a.m && col < a.n) {
                    const float v = acc[i][j][r];
                    if (a.partial) {                        // split-K: fp32 partial, summed by splitk_reduce_kernel
                        a.partial[((size_t)blockIdx.y * a.m + row) * a.n + col] = v;
                        continue;
                    }
                    const size_t o = (size_t)row * a.ys + col;
                    if (a.y_dtype == MI355Q_F32) ((float*)a.y)[o] = v;
                    else if (a.y_dtype == MI355Q_BF16) ((uint16_t*)a.y)[o] = f32_to_bf16_rne(v);
                    else ((uint16_t*)a.y)[o] = f32_to_f16_rne(v);
                }
            }
        }
}

// Sum of the split-K partials in split order (deterministic), one rounding to the output type.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial, void* __restrict__ y,
                                                            uint32_t m, uint32_t n, uint32_t ys, uint32_t splits,
                                                            uint32_t y_dtype) {
    const size_t total = (size_t)m * n;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        float v = 0.f;
        for (uint32_t s = 0; s < splits; s++) v += partial[(size_t)s * total + i];
        const size_t row = i / n, col = i - row * n;
        const size_t o = row * ys + col;
        if (y_dtype == MI355Q_F32) ((float*)y)[o] = v;
        else if (y_dtype == MI355Q_BF16) ((uint16_t*)y)[o] = f32_to_bf16_rne(v);
        else ((uint16_t*)y)[o] = f32_to_f16_rne(v);
    }
}

// Tile choice.  Problems with at least one 256 x 256 tile per CU take those (eight wavefronts,
// double-buffered LDS, in-wave software pipeline); smaller ones take 128 x 128 tiles (same
// pipeline, four wavefronts, two or three workgroups per CU).
GemmLaunchShape gemm_mfma_shape(const mi355q_context* ctx, uint32_t m, uint32_t n, uint32_t k) {
    const uint32_t cus = (uint32_t)ctx->props.multiProcessorCount;
    auto tiles = [&](uint32_t bm, uint32_t bn) { return ((m + bm - 1) / bm) * ((n + bn - 1) / bn); };
    GemmLaunchShape g{};
    const uint32_t kt = k / kTileK;
    // 256 x 256 tiles on eight wavefronts when they fill the chip, alone or with K split so that tiles x splits comes
    // to about one workgroup per CU and a split keeps sixteen K-tiles (M = 2048, 14336 -> 4096: 128 tiles, 333 us
    // as 512 tiles of 128 x 128, 236 us as 128 x 2; M = 1024: 204 -> 131 us as 64 x 4; 4096 -> 14336 at M = 1024:
    // 171 -> 126 us as 224 x 1); else 128 x 128 tiles, split over K when they leave half the CUs idle.
    uint32_t wide_splits = 0;
    bool wide = false;
    const uint32_t t256 = tiles(256, 256);
    if (m > 128 && 10 * t256 >= 9 * cus) {
        wide = true;
    } else if (m >= 256) {
        uint32_t sp = cus / t256;
        while (sp > 1 && kt / sp < 16) sp--;
        if (sp >= 1 && t256 * sp * 4 >= cus * 3) { wide = true; wide_splits = sp; }
    }
    if (wide) { g.bm = 256; g.bn = 256; g.stages = 2; g.block = 512; }
    else { g.bm = 128; g.bn = 128; g.stages = 2; g.block = 256; }
    g.grid = (tiles(g.bm, g.bn) + 7) / 8 * 8;
    // K is split over workgroups when the tiles alone leave most CUs idle (short M): each split writes
    // an fp32 partial, a second launch adds them.  At least 8 K-tiles per split.
    g.splits = wide_splits ? wide_splits : 1;
    if (g.bm == 128 && tiles(128, 128) * 2 <= cus) {
        uint32_t want = (2 * cus) / tiles(128, 128);
        if (want > 16) want = 16;
        while (want > 1 && kt / want < 8) want--;
        g.splits = want ? want : 1;
    }
    g.kt_per_split = (kt + g.splits - 1) / g.splits;
    g.splits = (kt + g.kt_per_split - 1) / g.kt_per_split;
    g.lds_bytes = g.stages * (g.bm + g.bn) * (uint32_t)kRowBytes;
    return g;
}

namespace {

template <int BITS, int GROUP, int BM, int BN, bool QUANT, int STAGES, bool SB_BF16, int WAVES, bool T16>
mi355q_status launch_tile_sb(hipStream_t s, GemmArgs a) {
    a.tiles_m = (a.m + BM - 1) / BM;
    a.tiles_n = (a.n + BN - 1) / BN;
    const uint32_t total = a.tiles_m * a.tiles_n;
    const uint32_t grid = (total + 7) / 8 * 8;
    constexpr size_t lds = (size_t)STAGES * (BM + BN) * kRowBytes;
    auto kern = qgemm_mfma_kernel<BITS, GROUP, BM, BN, QUANT, STAGES, SB_BF16, WAVES, T16>;
    // The attribute belongs to the function on one device: one bit per device and instantiation.
    static std::atomic<uint64_t> lds_limit_raised{0};
    int device = 0;
    MI355Q_HIP(hipGetDevice(&device));
    const uint64_t bit = 1ull << (device & 63);
    if (!(lds_limit_raised.load(std::memory_order_relaxed) & bit)) {
        MI355Q_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        lds_limit_raised.fetch_or(bit, std::memory_order_relaxed);
    }
    const uint32_t kt = a.k / kTileK;
    const uint32_t splits = a.partial ? (kt + a.kt_per_split - 1) / a.kt_per_split : 1;
    if (!a.partial) a.kt_per_split = kt;
    kern<<<dim3(grid, splits), dim3(WAVES * 64), lds, s>>>(a);
    MI355Q_HIP(hipGetLastError());
    if (a.partial) {
        const size_t total = (size_t)a.m * a.n;
        size_t blocks = (total + 255) / 256;
        if (blocks > 8192) blocks = 8192;
        splitk_reduce_kernel<<<dim3((unsigned)blocks), dim3(256), 0, s>>>(a.partial, a.y, a.m, a.n, a.ys, splits, a.y_dtype);
        MI355Q_HIP(hipGetLastError());
    }
    return MI355Q_OK;
}

template <int BITS, int GROUP, int BM, int BN, bool QUANT, int STAGES, int WAVES = 4>
mi355q_status launch_tile(hipStream_t s, const GemmArgs& a) {
    if constexpr (QUANT && BITS == 4 && GROUP == 64 && STAGES == 2 && WAVES * 64 == 2 * BN) {
        if (a.tiles) {
            if (a.sb_dtype == MI355Q_BF16) return launch_tile_sb<BITS, GROUP, BM, BN, QUANT, STAGES, true, WAVES, true>(s, a);
            return launch_tile_sb<BITS, GROUP, BM, BN, QUANT, STAGES, false, WAVES, true>(s, a);
        }
    }
    if (a.tiles) return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "this tile shape does not read TILE16 records");
    if constexpr (QUANT) {
        if (a.sb_dtype == MI355Q_BF16) return launch_tile_sb<BITS, GROUP, BM, BN, QUANT, STAGES, true, WAVES, false>(s, a);
    }
    return launch_tile_sb<BITS, GROUP, BM, BN, QUANT, STAGES, false, WAVES, false>(s, a);
}

template <int BITS, int GROUP, bool QUANT>
mi355q_status launch_shape(hipStream_t s, mi355q_context* ctx, GemmArgs a) {
    const GemmLaunchShape g = gemm_mfma_shape(ctx, a.m, a.n, a.k);
    if (g.splits > 1) {
        const size_t need = (size_t)g.splits * a.m * a.n * sizeof(float);
        if (mi355q_status st = ensure_workspace(ctx, need)) return st;
        a.partial = (float*)ctx->workspace;
        a.kt_per_split = g.kt_per_split;
    }
    if (g.bm == 256 && g.bn == 256 && g.block == 512) return launch_tile<BITS, GROUP, 256, 256, QUANT, 2, 8>(s, a);
    return launch_tile<BITS, GROUP, 128, 128, QUANT, 2>(s, a);
}

}  // namespace

bool gemm_mfma_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride) {
    if (x_dtype != MI355Q_BF16 || m < 1) return false;
    if (w.layout == MI355Q_LAYOUT_TILE16)        // q4 g64 records, K % 128 == 0 by construction
        return w.tiles && w.bits == 4 && w.group == 64 && w.k % 128 == 0 && x_stride % 8 == 0;
    if (w.layout != MI355Q_LAYOUT_PLANES || !w.sz) return false;
    if (w.k % kTileK) return false;
    if (x_stride % 8) return false;                       // 128-bit activation loads
    if ((uintptr_t)w.codes % 16 || w.code_stride % 4) return false;
    const bool fmt_ok = (w.bits == 4 && (w.group == 64 || w.group == 128)) ||
                        (w.bits == 8 && (w.group == 32 || w.group == 64)) ||
                        (w.bits == 6 && w.group == 64) || (w.bits == 3 && w.group == 64) ||
                        (w.bits == 2 && w.group == 64);
    return fmt_ok;
}

mi355q_status launch_qgemm_mfma(hipStream_t s, mi355q_context* ctx, const WView& w, const void* x, int x_dtype,
                                void* y, int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride,
                                unsigned long long* probe, uint32_t flags) {
    // long prompts on 4-bit planes and blocks: the wide-tile kernel with the weights dequantised in registers
    if (gemm_wide_taken(w, x_dtype, m, x_stride, flags) && (uintptr_t)x % 16 == 0)
        return launch_qgemm_wide(s, ctx, w, x, x_dtype, y, y_dtype, m, x_stride, y_stride, probe);
    if (x_dtype != MI355Q_BF16) return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the tiled MFMA GEMM takes bf16 activations");
    if ((uintptr_t)x % 16) return fail(MI355Q_ERR_INVALID_ARGUMENT, "activation pointer must be 16-byte aligned");
    GemmArgs a{};
    a.codes = w.codes; a.sz = w.sz; a.bdense = nullptr;
    if (w.layout == MI355Q_LAYOUT_TILE16) { a.tiles = w.tiles; a.kblocks = w.k / 128; }
    a.x = (const uint16_t*)x; a.y = y;
    a.m = m; a.n = w.n; a.k = w.k; a.xs = x_stride; a.ys = y_stride;
    a.code_stride = w.code_stride; a.sz_stride = w.sz_stride;
    a.y_dtype = (uint32_t)y_dtype; a.sb_dtype = w.sb_dtype;
    a.probe = probe;
    switch (w.bits * 1000 + w.group) {
    case 4064: return launch_shape<4, 64, true>(s, ctx, a);
    case 4128: return launch_shape<4, 128, true>(s, ctx, a);
    case 8032: return launch_shape<8, 32, true>(s, ctx, a);
    case 8064: return launch_shape<8, 64, true>(s, ctx, a);
    case 6064: return launch_shape<6, 64, true>(s, ctx, a);
    case 3064: return launch_shape<3, 64, true>(s, ctx, a);
    case 2064: return launch_shape<2, 64, true>(s, ctx, a);
    default: break;
    }
    return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no MFMA GEMM for q%u g%u", w.bits, w.group);
}

mi355q_status launch_gemm_bf16_mfma(hipStream_t s, mi355q_context* ctx, const void* a_ptr, int a_dtype,
                                    const uint16_t* b, void* c, int c_dtype, uint32_t m, uint32_t n, uint32_t k,
                                    uint32_t a_stride, uint32_t c_stride) {
    if (a_dtype != MI355Q_BF16) return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the MFMA GEMM takes bf16 activations");
    if (k % kTileK) return fail(MI355Q_ERR_SHAPE, "K=%u must be a multiple of %d", k, kTileK);
    if (a_stride % 8 || (uintptr_t)a_ptr % 16 || (uintptr_t)b % 16)
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "operands must be 16-byte aligned with row strides multiple of 8");
    GemmArgs a{};
    a.bdense = b;
    a.x = (const uint16_t*)a_ptr; a.y = c;
    a.m = m; a.n = n; a.k = k; a.xs = a_stride; a.ys = c_stride;
    a.y_dtype = (uint32_t)c_dtype;
    return launch_shape<4, 64, false>(s, ctx, a);
}

}  // namespace mi355q
