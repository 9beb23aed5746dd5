// Prefill GEMM on the matrix cores for long prompts, 4-bit planes:  Y[M,N] = X[M,K] * W[N,K]^T  with the weights
// dequantised to bf16 IN REGISTERS, so that nothing but the activations goes through LDS.
//
// Stands in for the reference's dequant_q4_g{64,128}_bf16 + gemm_bf16_f32s pair and for its direct gemm_q4_g*_f32s
// (Sources/MetalCompiler/Generator/MetalSourceGenerator+Quantized.swift:22-156,361-416 and
//  MetalSourceGenerator+Linear.swift:18-81; selection Compiler/MetalPrefillStepBuilder.swift:533-560): the weights a
// product sees are bf16(scale * q + bias), as on the reference's two-dispatch route, without its N x K x 2 byte scratch.
//
// Shape of the kernel (what each choice answers is measured on an MI355X with all CUs busy):
//   * workgroup tile BM x 256 x 64, four wavefronts, one per SIMD; wavefront w owns columns 64 w .. 64 w + 63 of the
//     tile and ALL BM rows (BM / 32 x 2 accumulators of v_mfma_f32_32x32x16_bf16).  The weights are the instruction's
//     A operand: a lane (n, h) holds codes 32 h .. 32 h + 31 of row n's K-tile as one 16-byte load and turns word j
//     into the operand of k-step j.  No other wavefront needs those weights, so they never touch LDS, nothing is
//     dequantised twice inside a workgroup, and the 128-bit LDS fills of a dequantised tile (with their bank
//     conflicts) do not exist;
//   * the activations are the B operand, read from LDS; a K-tile of them (BM rows x 128 bytes, 16-byte chunks rotated
//     by (row / 2) % 8 so that fragment reads are free of bank conflicts) is copied global -> LDS directly
//     (global_load_lds_dwordx4), four stages deep.  A vector-memory instruction costs the issuing wavefront about 30
//     cycles of matrix-core time whatever it moves, so the copies are spread evenly, one per eight MFMAs, and never
//     issued back to back (eight together cost 100 cycles each: every wavefront then waits at the next barrier for
//     the one that was served last);
//   * weight words come four K-tiles at a time (so that a row's 128-byte line is fetched once), with the (scale, bias)
//     words of those four K-tiles as one more 16-byte load, and wait in registers; vmcnt is counted by hand, because
//     the copies into LDS are invisible to the compiler's own bookkeeping;
//   * one k-step is BM / 32 groups of two MFMAs; group q also reads activation fragment q of the NEXT k-step from LDS
//     and dequantises a share of the next k-step's weight fragments (byte-lane convert, fp32 fma, one rounding to
//     bf16 -- bit for bit the weights of dequant_q4_g*_bf16), so the matrix cores never wait for an operand;
//   * one barrier per K-tile, in the middle of it: K-tile kt + 1 has landed for everyone, and the stage of K-tile
//     kt - 1 is free for kt + 3;
//   * BM = 256 where that fills the chip (one workgroup per CU, 256 accumulator registers per lane), BM = 128 elsewhere
//     (two workgroups per CU).
#include "device_utils.h"
#include <atomic>

namespace mi355q {

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 wd_bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float wd_floatx16_t;
typedef __bf16 wd_bf16x2_v __attribute__((ext_vector_type(2)));
typedef float wd_float2_v __attribute__((ext_vector_type(2)));
typedef float wd_float4_v __attribute__((ext_vector_type(4)));

struct WideArgs {
    const uint32_t* codes;       // [N, K / 8] words, rows code_stride words apart
    const uint32_t* sz;          // (scale | bias << 16) per group, rows sz_stride words apart
    const uint16_t* x;           // bf16 [M, xs]
    void* y;
    uint32_t m, n, k, xs, ys;
    uint32_t code_stride, sz_stride;
    uint32_t tiles_m, tiles_n;
    uint32_t y_dtype;
    uint32_t wide_stores;        // rows of y are 16-byte aligned for every column that is a multiple of four
    float* partial;              // K split over workgroups: fp32 [splits][M][N] partial results (null otherwise)
    uint32_t splits, kt_per_split;   // K-tiles per split: a multiple of four
    unsigned long long* probe;   // optional: [0] shader cycles, [1] 100 MHz ticks that workgroup 0 spent in the kernel
};

constexpr int kWideStages = 4;   // LDS stages of activations
constexpr int kWideBN = 256;

__device__ __forceinline__ uint32_t wd_pack_bf16(float lo, float hi) {
    wd_float2_v v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, wd_bf16x2_v));
}

// A wave-uniform address as the scalar operand of hand-written memory instructions, wherever the compiler computed it
__device__ __forceinline__ const char* wd_scalar(const char* p) {
    const uint64_t v = (uint64_t)(uintptr_t)p;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return (const char*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

template <int BM, bool SB_BF16, int GROUP>
__global__ __launch_bounds__(256, (BM == 128 ? 2 : 1)) void qgemm_wide_kernel(WideArgs a) {
    constexpr int TM = BM / 32;                     // activation fragments = groups per k-step
    constexpr int A_STAGE = BM * 128;
    constexpr int AQ = BM / 32;                     // activation copies per wavefront and K-tile (8 rows each)
    constexpr int CPK = AQ / 4;                     // ... and per k-step
    constexpr int SZW = 4 * 64 / GROUP;             // (scale, bias) words of four K-tiles
    constexpr int WL = 8 + 2;                       // weight + (scale, bias) loads per wavefront and four K-tiles
    extern __shared__ u32x4 smem_wide[];
    char* const lds = (char*)smem_wide;
    const uint32_t lds_base = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);

    // tile of this workgroup: the workgroups of one XCD (id % 8) take consecutive tiles, row tiles of one column tile
    // first, so that they share that column tile's weights and a few row tiles' activations in the XCD's L2
    // (with K split over workgroups: all tiles of the first part of K, then those of the second ...)
    const uint32_t tiles = a.tiles_m * a.tiles_n;
    const uint32_t total = tiles * a.splits;
    const uint32_t per_xcd = (total + 7) / 8;
    const uint32_t t_id = (blockIdx.x % 8u) * per_xcd + blockIdx.x / 8u;
    if (t_id >= total) return;
    const uint32_t split = (uint32_t)__builtin_amdgcn_readfirstlane((int)(t_id / tiles)), tile = t_id - split * tiles;
    const uint32_t tn = tile / a.tiles_m, tm = tile % a.tiles_m;
    const uint32_t m0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tm * BM)), n0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tn * kWideBN));
    const uint32_t kt_begin = (uint32_t)__builtin_amdgcn_readfirstlane((int)(split * a.kt_per_split));

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t ln = lane & 31, lh = lane >> 5;
    const uint32_t kt_left = a.k / 64 - kt_begin;
    const uint32_t KT = (uint32_t)__builtin_amdgcn_readfirstlane((int)(kt_left < a.kt_per_split ? kt_left : a.kt_per_split));   // K-tiles of this workgroup: a multiple of four

    // ---- activations: global -> LDS ---------------------------------------------------------------
    // copy q of wavefront w covers tile rows 8 (AQ w + q) .. + 7; lane L lands at row L / 8, position L % 8, and
    // fetches the chunk that belongs there after the rotation.  Rows past M re-read the last one.
    const uint32_t m_last = a.m - 1 - m0;           // last valid row of the tile
    uint32_t x_off[AQ];
#pragma unroll
    for (int q = 0; q < AQ; q++) {
        const uint32_t row = 8 * (AQ * wave + q) + (lane >> 3);
        const uint32_t chunk = (lane & 7u) ^ ((row >> 1) & 7u);
        x_off[q] = (row < m_last ? row : m_last) * a.xs * 2 + chunk * 16;
    }
    const char* const xg = (const char*)(a.x + (size_t)m0 * a.xs + (size_t)kt_begin * 64);
    auto copy_x = [&](uint32_t kt, auto Q0, auto CNT) __attribute__((always_inline)) {
        const uint32_t t = kt < KT ? kt : KT - 1;   // past the end: a copy nobody reads, so that the counts stay the same
        const char* const g = wd_scalar(xg + (size_t)t * 128);
        const uint32_t as = lds_base + (kt % kWideStages) * A_STAGE + wave * (AQ * 1024);
#pragma unroll
        for (int q = decltype(Q0)::value; q < decltype(Q0)::value + decltype(CNT)::value; q++) {
            const uint32_t l = as + q * 1024;
            const uint32_t xo = x_off[q];
            asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(xo), "s"(g), "s"(l) : "memory");
        }
    };
    // ---- weights: global -> registers, four K-tiles at a time -------------------------------------------
    // lane (n, h) of fragment f holds codes 32 h .. 32 h + 31 of each K-tile of row 64 w + 32 f + n
    const uint32_t n_last = a.n - 1 - n0;
    uint32_t w_off[2], sz_off[2];
#pragma unroll
    for (int f = 0; f < 2; f++) {
        const uint32_t r = 64 * wave + 32 * f + ln;
        const uint32_t gr = r < n_last ? r : n_last;
        w_off[f] = gr * a.code_stride * 4 + lh * 16;
        sz_off[f] = gr * a.sz_stride * 4;
    }
    const char* const cg = (const char*)(a.codes + (size_t)n0 * a.code_stride) + (size_t)(kt_begin / 4) * 128;
    const char* const sg = (const char*)(a.sz + (size_t)n0 * a.sz_stride) + (size_t)(kt_begin / 4) * (SZW * 4);
    using sz_vec = std::conditional_t<SZW == 4, u32x4, u32x2>;      // kept whole: the loads write them behind the compiler's back
    u32x4 wnext[2][4], wcur[2][4];
    sz_vec sznext[2], szcur[2];
    auto load_w = [&](uint32_t four) __attribute__((always_inline)) {
        const uint32_t p = four * 4 < KT ? four : KT / 4 - 1;
        const char* const g = wd_scalar(cg + (size_t)p * 128);
        const char* const gs = wd_scalar(sg + (size_t)p * (SZW * 4));
#pragma unroll
        for (int f = 0; f < 2; f++) {
#pragma unroll
            for (int t = 0; t < 4; t++)
                asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(wnext[f][t]) : "v"(w_off[f]), "s"(g), "n"(t * 32) : "memory");
        }
#pragma unroll
        for (int f = 0; f < 2; f++) {
            if constexpr (SZW == 4) asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(sznext[f]) : "v"(sz_off[f]), "s"(gs) : "memory");
            else asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(sznext[f]) : "v"(sz_off[f]), "s"(gs) : "memory");
        }
    };
    // waits until at most `younger` vector-memory operations issued after the weight loads are outstanding, then
    // takes the loaded words over
    auto take_w = [&](auto YOUNGER) __attribute__((always_inline)) {
        constexpr int younger = decltype(YOUNGER)::value;
        asm volatile("s_waitcnt vmcnt(%10)"
                     : "+v"(wnext[0][0]), "+v"(wnext[0][1]), "+v"(wnext[0][2]), "+v"(wnext[0][3]), "+v"(wnext[1][0]),
                       "+v"(wnext[1][1]), "+v"(wnext[1][2]), "+v"(wnext[1][3]), "+v"(sznext[0]), "+v"(sznext[1])
                     : "n"(younger)
                     : "memory");
#pragma unroll
        for (int f = 0; f < 2; f++) {
#pragma unroll
            for (int t = 0; t < 4; t++) wcur[f][t] = wnext[f][t];
            szcur[f] = sznext[f];
        }
    };

    // ---- operands ----------------------------------------------------------------------------------
    // activation fragment (i, j): rows 32 i + ln, chunk 4 lh + j -- the K positions lane (., h) holds of word j
    uint32_t a_rd[4];
#pragma unroll
    for (int j = 0; j < 4; j++) a_rd[j] = ln * 128 + (((4 * lh + j) ^ ((ln >> 1) & 7u)) << 4);

    wd_bf16x8_t xf[2][TM], wf[2][2];
    wd_floatx16_t acc[2][TM];
#pragma unroll
    for (int f = 0; f < 2; f++)
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[f][i][r] = 0.0f;

    // scale and bias of K-tile t (0 .. 3) of the current four
    float sc[2], sc16[2], zr[2];
    auto scales = [&](auto T) __attribute__((always_inline)) {
        constexpr int t = decltype(T)::value;
#pragma unroll
        for (int f = 0; f < 2; f++) {
            const uint32_t szw = szcur[f][t * 64 / GROUP];
            if constexpr (SB_BF16) {
                sc[f] = __uint_as_float(szw << 16); zr[f] = __uint_as_float(szw & 0xFFFF0000u);
            } else {
                sc[f] = f16_to_f32((uint16_t)(szw & 0xFFFFu)); zr[f] = f16_to_f32((uint16_t)(szw >> 16));
            }
            sc16[f] = sc[f] * 0.0625f;              // exact: the scales are those of f16 range (>= 2^-24)
        }
    };
    // a quarter of the dequantisation of word w of fragment f: codes 2 b and 2 b + 1 (byte b of the even and of the odd
    // nibbles) as one packed bf16 pair.  The odd nibbles stay where they are, sixteen times too large, and take
    // scale / 16: fma(scale / 16, 16 q, bias) is fma(scale, q, bias) bit for bit.
    uint32_t dq_lo[2], dq_hi[2];
    auto dq_piece = [&](auto F, auto B, uint32_t w) __attribute__((always_inline)) -> uint32_t {
        constexpr int f = decltype(F)::value, b = decltype(B)::value;
        if constexpr (b == 0) { dq_lo[f] = w & 0x0F0F0F0Fu; dq_hi[f] = w & 0xF0F0F0F0u; }
        float q0, q1;
        if constexpr (b == 0) { asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(q0) : "v"(dq_lo[f])); asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(q1) : "v"(dq_hi[f])); }
        if constexpr (b == 1) { asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(q0) : "v"(dq_lo[f])); asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(q1) : "v"(dq_hi[f])); }
        if constexpr (b == 2) { asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(q0) : "v"(dq_lo[f])); asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(q1) : "v"(dq_hi[f])); }
        if constexpr (b == 3) { asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(q0) : "v"(dq_lo[f])); asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(q1) : "v"(dq_hi[f])); }
        return wd_pack_bf16(__builtin_fmaf(sc[f], q0, zr[f]), __builtin_fmaf(sc16[f], q1, zr[f]));
    };
    // One k-step = TM groups.  Group q: (every TM / CPK groups: one activation copy of K-tile kt_copy,) the read of
    // activation fragment q of the NEXT k-step (K-tile kt_next, word JN of K-tile TN of the current four), the two
    // MFMAs on fragment q of this one, and its share of the next k-step's weight fragments.
    u32x4 dq_o[2];
    auto kstep = [&](auto BUF, auto TN, auto JN, uint32_t kt_next, uint32_t kt_copy, auto SLOT) __attribute__((always_inline)) {
        constexpr int buf = decltype(BUF)::value, tn_ = decltype(TN)::value, jn = decltype(JN)::value;
        constexpr int slot = decltype(SLOT)::value;
        const char* const xs_next = lds + (kt_next % kWideStages) * A_STAGE + a_rd[jn];
        const uint32_t tc = kt_copy < KT ? kt_copy : KT - 1;
        const char* const gx = wd_scalar(xg + (size_t)tc * 128);
        const uint32_t lx = lds_base + (kt_copy % kWideStages) * A_STAGE + wave * (AQ * 1024);
        static_for<TM>([&](auto Q) __attribute__((always_inline)) {
            constexpr int q = decltype(Q)::value;
            if constexpr (q % (TM / CPK) == 0) {
                constexpr int cq = slot * CPK + q / (TM / CPK);
                const uint32_t l = lx + cq * 1024;
                const uint32_t xo = x_off[cq];
                asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(xo), "s"(gx), "s"(l) : "memory");
            }
            xf[buf ^ 1][q] = *(const wd_bf16x8_t*)(xs_next + q * 4096);
            acc[0][q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[buf][0], xf[buf][q], acc[0][q], 0, 0, 0);
            acc[1][q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[buf][1], xf[buf][q], acc[1][q], 0, 0, 0);
            // eight pieces (two fragments of four) over the TM groups
            static_for<8 / TM>([&](auto P) __attribute__((always_inline)) {
                constexpr int piece = q * (8 / TM) + decltype(P)::value;
                constexpr int f = piece / 4, b = piece % 4;
                dq_o[f][b] = dq_piece(std::integral_constant<int, f>{}, std::integral_constant<int, b>{}, wcur[f][tn_][jn]);
                if constexpr (b == 3) wf[buf ^ 1][f] = __builtin_bit_cast(wd_bf16x8_t, dq_o[f]);
            });
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>; using I3 = std::integral_constant<int, 3>;

    // clock probe: the first wavefront of workgroup 0 times itself with the shader-clock counter and the constant
    // 100 MHz counter; their ratio is the clock the matrix cores actually ran at
    const bool probing = a.probe != nullptr && blockIdx.x == 0 && wave == 0;
    unsigned long long probe_c0 = 0, probe_r0 = 0;
    if (probing) { probe_c0 = __builtin_readcyclecounter(); probe_r0 = __builtin_amdgcn_s_memrealtime(); }

    // ---- prologue -----------------------------------------------------------------------------------
    // The copies of K-tile kt + 3 go out between the barriers of iterations kt and kt + 1: half of them in k-steps 2
    // and 3 of iteration kt, half in k-steps 0 and 1 of iteration kt + 1.
    load_w(0);
    copy_x(0, I0{}, std::integral_constant<int, AQ>{});
    copy_x(1, I0{}, std::integral_constant<int, AQ>{});
    copy_x(2, I0{}, std::integral_constant<int, AQ / 2>{});
    take_w(std::integral_constant<int, 2 * AQ + AQ / 2>{});
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(AQ + AQ / 2) : "memory");
    __syncthreads();
    scales(I0{});
#pragma unroll
    for (int i = 0; i < TM; i++) xf[0][i] = *(const wd_bf16x8_t*)(lds + a_rd[0] + i * 4096);
    static_for<2>([&](auto F) __attribute__((always_inline)) {
        constexpr int f = decltype(F)::value;
        u32x4 o;
        o.x = dq_piece(F, I0{}, wcur[f][0][0]);
        o.y = dq_piece(F, I1{}, wcur[f][0][0]);
        o.z = dq_piece(F, I2{}, wcur[f][0][0]);
        o.w = dq_piece(F, I3{}, wcur[f][0][0]);
        wf[0][f] = __builtin_bit_cast(wd_bf16x8_t, o);
    });
    __builtin_amdgcn_sched_barrier(0);

    for (uint32_t kt0 = 0; kt0 < KT; kt0 += 4) {
        static_for<4>([&](auto U) __attribute__((always_inline)) {
            constexpr int u = decltype(U)::value;
            const uint32_t kt = kt0 + u;
            kstep(I0{}, U, I1{}, kt, kt + 2, I2{});
            kstep(I1{}, U, I2{}, kt, kt + 2, I3{});
            // K-tile kt + 1 has landed for everyone, K-tile kt - 1 is no longer read: its stage takes K-tile kt + 3.
            // Younger than this wavefront's copies of K-tile kt + 1 are its copies of kt + 2 and, in iteration 1, the
            // weight loads of iteration 0.
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(u == 1 ? AQ + WL : AQ) : "memory");
            __builtin_amdgcn_s_barrier();
            if constexpr (u == 0) load_w(kt0 / 4 + 1);
            __builtin_amdgcn_sched_barrier(0);
            kstep(I0{}, U, I3{}, kt, kt + 3, I0{});
            if constexpr (u == 3) {
                // the words of the next four K-tiles: younger are the copies of three K-tiles and those of k-step 2
                take_w(std::integral_constant<int, 3 * AQ + CPK>{});
                scales(I0{});
                kstep(I1{}, I0{}, I0{}, kt + 1, kt + 3, I1{});
            } else {
                scales(std::integral_constant<int, u + 1>{});
                kstep(I1{}, std::integral_constant<int, (u + 1) % 4>{}, I0{}, kt + 1, kt + 3, I1{});
            }
        });
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (probing) {
        const unsigned long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
        if (lane == 0) { a.probe[0] = c1 - probe_c0; a.probe[1] = r1 - probe_r0; }
    }

    // ---- epilogue: one rounding, to the output type -----------------------------------------------------
    // lane (m, h) of accumulator (f, i) holds row m0 + 32 i + m, columns 32 f + 8 g + 4 h + (0 .. 3) for g = 0 .. 3.
    // One accumulator at a time (the fences keep the compiler from fetching all 256 registers first).
    auto store_tiles = [&](auto DT, void* const y, const size_t ys, const bool wide) __attribute__((always_inline)) {
        constexpr int dt = decltype(DT)::value;
        static_for<2>([&](auto F) __attribute__((always_inline)) {
            static_for<TM>([&](auto I) __attribute__((always_inline)) {
                constexpr int f = decltype(F)::value, i = decltype(I)::value;
                const uint32_t row = m0 + i * 32 + ln;
                // an opaque touch per output type: identical register fetches in the three copies of this loop would
                // otherwise be merged in front of the branch, all 256 at once
                asm volatile("" : "+v"(acc[f][i]));
                if (row < a.m) {
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const uint32_t col = n0 + 64 * wave + 32 * f + 8 * g + 4 * lh;
                        const float v[4] = {acc[f][i][4 * g + 0], acc[f][i][4 * g + 1], acc[f][i][4 * g + 2], acc[f][i][4 * g + 3]};
                        const size_t o = (size_t)row * ys + col;
                        if (wide && col + 3 < a.n) {
                            if constexpr (dt == MI355Q_F32) {
                                const float4 t = {v[0], v[1], v[2], v[3]};
                                *(float4*)((float*)y + o) = t;
                            } else if constexpr (dt == MI355Q_BF16) {
                                uint2 t;
                                t.x = wd_pack_bf16(v[0], v[1]); t.y = wd_pack_bf16(v[2], v[3]);
                                *(uint2*)((uint16_t*)y + o) = t;
                            } else {
                                uint2 t;
                                t.x = (uint32_t)f32_to_f16_rne(v[0]) | ((uint32_t)f32_to_f16_rne(v[1]) << 16);
                                t.y = (uint32_t)f32_to_f16_rne(v[2]) | ((uint32_t)f32_to_f16_rne(v[3]) << 16);
                                *(uint2*)((uint16_t*)y + o) = t;
                            }
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                if (col + e < a.n) store_out<dt>(y, o + e, v[e]);
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        });
    };
    if (a.partial)         // this part of K as fp32 (N is a multiple of four: 16-byte stores); wide_reduce_kernel adds the parts
        store_tiles(std::integral_constant<int, MI355Q_F32>{}, a.partial + (size_t)split * a.m * a.n, a.n, true);
    else if (a.y_dtype == MI355Q_BF16) store_tiles(std::integral_constant<int, MI355Q_BF16>{}, a.y, a.ys, a.wide_stores != 0);
    else if (a.y_dtype == MI355Q_F32) store_tiles(std::integral_constant<int, MI355Q_F32>{}, a.y, a.ys, a.wide_stores != 0);
    else store_tiles(std::integral_constant<int, MI355Q_F16>{}, a.y, a.ys, a.wide_stores != 0);
}

// Sum of the parts of a K-split launch in part order (deterministic), one rounding to the output type.  N is a
// multiple of four; four columns per thread.
__global__ __launch_bounds__(256) void wide_reduce_kernel(const wd_float4_v* __restrict__ partial, void* __restrict__ y, uint32_t m,
                                                          uint32_t n, uint32_t ys, uint32_t splits, uint32_t y_dtype,
                                                          uint32_t wide_stores) {
    const size_t total = (size_t)m * n / 4;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        wd_float4_v v = __builtin_nontemporal_load(partial + i);
        for (uint32_t s = 1; s < splits; s++) v += __builtin_nontemporal_load(partial + (size_t)s * total + i);
        const size_t e = i * 4, row = e / n, col = e - row * n;
        const size_t o = row * ys + col;
        if (wide_stores) {
            if (y_dtype == MI355Q_F32) *(wd_float4_v*)((float*)y + o) = v;
            else if (y_dtype == MI355Q_BF16) {
                uint2 t;
                t.x = wd_pack_bf16(v.x, v.y); t.y = wd_pack_bf16(v.z, v.w);
                *(uint2*)((uint16_t*)y + o) = t;
            } else {
                uint2 t;
                t.x = (uint32_t)f32_to_f16_rne(v.x) | ((uint32_t)f32_to_f16_rne(v.y) << 16);
                t.y = (uint32_t)f32_to_f16_rne(v.z) | ((uint32_t)f32_to_f16_rne(v.w) << 16);
                *(uint2*)((uint16_t*)y + o) = t;
            }
        } else {
            const float f[4] = {v.x, v.y, v.z, v.w};
            for (int c = 0; c < 4; c++) {
                if (y_dtype == MI355Q_F32) ((float*)y)[o + c] = f[c];
                else if (y_dtype == MI355Q_BF16) ((uint16_t*)y)[o + c] = f32_to_bf16_rne(f[c]);
                else ((uint16_t*)y)[o + c] = f32_to_f16_rne(f[c]);
            }
        }
    }
}

template <int BM, bool SB_BF16, int GROUP>
mi355q_status launch_wide_tile(hipStream_t s, WideArgs a) {
    a.tiles_m = (a.m + BM - 1) / BM;
    a.tiles_n = (a.n + kWideBN - 1) / kWideBN;
    const uint32_t grid = (a.tiles_m * a.tiles_n * a.splits + 7) / 8 * 8;
    constexpr size_t lds = (size_t)kWideStages * BM * 128;
    auto kern = qgemm_wide_kernel<BM, SB_BF16, GROUP>;
    // the attribute belongs to the function on one device: one bit per device and instantiation
    static std::atomic<uint64_t> lds_limit_raised{0};
    int device = 0;
    MI355Q_HIP(hipGetDevice(&device));
    const uint64_t bit = 1ull << (device & 63);
    if (!(lds_limit_raised.load(std::memory_order_relaxed) & bit)) {
        MI355Q_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        lds_limit_raised.fetch_or(bit, std::memory_order_relaxed);
    }
    kern<<<dim3(grid), dim3(256), lds, s>>>(a);
    MI355Q_HIP(hipGetLastError());
    if (a.partial) {
        size_t blocks = ((size_t)a.m * a.n / 4 + 255) / 256;
        if (blocks > 16384) blocks = 16384;
        wide_reduce_kernel<<<dim3((unsigned)blocks), dim3(256), 0, s>>>((const wd_float4_v*)a.partial, a.y, a.m, a.n, a.ys, a.splits,
                                                                        a.y_dtype, a.wide_stores);
        MI355Q_HIP(hipGetLastError());
    }
    return MI355Q_OK;
}

template <int BM>
mi355q_status launch_wide_bm(hipStream_t s, const WideArgs& a, uint32_t group, bool sb_bf16) {
    if (group == 64) return sb_bf16 ? launch_wide_tile<BM, true, 64>(s, a) : launch_wide_tile<BM, false, 64>(s, a);
    return sb_bf16 ? launch_wide_tile<BM, true, 128>(s, a) : launch_wide_tile<BM, false, 128>(s, a);
}

}  // namespace

// 4-bit planes in groups of 64 or 128, bf16 activations, K a multiple of four K-tiles, 16-byte aligned rows of codes
// and of (scale, bias) words (a row's words of four K-tiles are one 16- or 8-byte load).
bool gemm_wide_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride) {
    if (x_dtype != MI355Q_BF16 || m < 1) return false;
    if (w.layout != MI355Q_LAYOUT_PLANES || !w.sz || !w.codes) return false;
    if (w.bits != 4 || (w.group != 64 && w.group != 128)) return false;
    if (w.k % 256 || x_stride % 8) return false;
    if ((uintptr_t)w.codes % 16 || w.code_stride % 4) return false;
    if ((uintptr_t)w.sz % 16 || w.sz_stride % 4) return false;
    // offsets inside a tile are 32-bit
    if ((uint64_t)x_stride * 2 * 256 >= (1ull << 32) || (uint64_t)w.code_stride * 4 * 256 >= (1ull << 32)) return false;
    return true;
}

// CUs of the current device (256 on an MI355X; fewer in a partitioned mode), asked once
uint32_t chip_cus() {
    static std::atomic<uint32_t> cached{0};
    uint32_t c = cached.load(std::memory_order_relaxed);
    if (c) return c;
    int device = 0, count = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return 256;                                   // no device: the planner still answers, for a whole MI355X
    }
    cached.store((uint32_t)count, std::memory_order_relaxed);
    return (uint32_t)count;
}

// A/B runs: tile height and K parts forced from outside (0: chosen here)
static std::atomic<uint32_t> g_wide_forced_bm{0}, g_wide_forced_splits{0};
void gemm_wide_force_shape(uint32_t bm, uint32_t splits) {
    g_wide_forced_bm.store(bm == 128 || bm == 256 ? bm : 0, std::memory_order_relaxed);
    g_wide_forced_splits.store(splits <= 8 ? splits : 0, std::memory_order_relaxed);
}

// Tile height and K parts.  What a wavefront spends on a K-tile depends on the tile height alone (the weights of its 64
// columns are dequantised once per K-tile whatever the rows: about 2500 cycles at 256 rows, 1600 at 128, measured
// under load), so 256-row tiles are the efficient ones and K is split into parts where they leave CUs idle: each part
// writes fp32, a second launch adds the parts (about 3 us and the traffic of splits + 1 result matrices).
GemmLaunchShape gemm_wide_shape(uint32_t m, uint32_t n, uint32_t k) {
    const uint32_t cus = chip_cus();
    const uint32_t tiles_n = (n + kWideBN - 1) / kWideBN;
    const uint32_t kt = k / 64;
    GemmLaunchShape g{};
    double best = 0;
    const uint32_t forced_bm = g_wide_forced_bm.load(std::memory_order_relaxed);
    const uint32_t forced_splits = g_wide_forced_splits.load(std::memory_order_relaxed);
    for (uint32_t bm : {256u, 128u}) {
        if (forced_bm && bm != forced_bm) continue;
        if (bm == 256 && m <= 128 && !forced_bm) continue;
        for (uint32_t splits : {1u, 2u, 3u, 4u}) {
            if (forced_splits && splits != forced_splits) continue;
            if (splits > 1 && (n % 4 || kt / splits < 16)) continue;
            const uint32_t per = (kt / 4 + splits - 1) / splits * 4;          // K-tiles a part, a multiple of four
            const uint32_t parts = (kt + per - 1) / per;
            if (parts != splits) continue;
            const uint32_t wgs = ((m + bm - 1) / bm) * tiles_n * parts;
            // cycles of a workgroup per K-tile, measured under load: 2500 at 256 rows (one workgroup a CU, whole rounds);
            // 1600 at 128 rows alone on its CU, 2950 for the two that share one (a last round of at most one per CU
            // runs alone)
            double cycles;
            if (bm == 256) {
                cycles = (double)((wgs + cus - 1) / cus) * per * 2500.0;
            } else {
                const uint32_t full = wgs / (2 * cus), rest = wgs % (2 * cus);
                cycles = (double)full * per * 2950.0 + (rest > cus ? per * 2950.0 : rest ? per * 1600.0 : 0.0);
            }
            const double rounds = bm == 256 ? (double)((wgs + cus - 1) / cus) : (double)((wgs + 2 * cus - 1) / (2 * cus));
            double cost = cycles / 1750.0 + 8.0 * rounds;                       // us at the clock the part holds
            if (parts > 1) cost += 3.0 + (double)(parts + 1) * m * n * 4.0 / 3.5e6;
            if (best == 0 || cost < best) {
                best = cost;
                g.bm = bm; g.splits = parts; g.kt_per_split = per;
            }
        }
    }
    if (best == 0) { g.bm = 128; g.splits = 1; g.kt_per_split = kt; }       // forced values that do not fit
    g.bn = kWideBN;
    g.stages = kWideStages;
    g.block = 256;
    g.grid = (((m + g.bm - 1) / g.bm) * tiles_n * g.splits + 7) / 8 * 8;
    g.lds_bytes = kWideStages * g.bm * 128;
    return g;
}

// Rows from which this kernel is taken instead of the tiled one (which splits K over workgroups for short M) and of
// the two-dispatch route: enough tiles to occupy three quarters of the CUs.
bool gemm_wide_chosen(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride) {
    if (!gemm_wide_eligible(w, x_dtype, m, x_stride) || m < kWideMinRows) return false;
    const GemmLaunchShape g = gemm_wide_shape(m, w.n, w.k);
    const uint32_t wgs = ((m + g.bm - 1) / g.bm) * ((w.n + kWideBN - 1) / kWideBN) * g.splits;
    return 4 * wgs >= 3 * chip_cus();
}

mi355q_status launch_qgemm_wide(hipStream_t s, mi355q_context* ctx, const WView& w, const void* x, int x_dtype, void* y,
                                int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride, unsigned long long* probe) {
    if (!gemm_wide_eligible(w, x_dtype, m, x_stride))
        return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the wide-tile MFMA GEMM does not accept this format, layout or stride");
    if ((uintptr_t)x % 16) return fail(MI355Q_ERR_INVALID_ARGUMENT, "activation pointer must be 16-byte aligned");
    WideArgs a{};
    a.codes = w.codes; a.sz = w.sz;
    a.x = (const uint16_t*)x; a.y = y;
    a.m = m; a.n = w.n; a.k = w.k; a.xs = x_stride; a.ys = y_stride;
    a.code_stride = w.code_stride; a.sz_stride = w.sz_stride;
    a.y_dtype = (uint32_t)y_dtype;
    a.wide_stores = (y_stride % 4 == 0 && (uintptr_t)y % 16 == 0) ? 1u : 0u;
    a.probe = probe;
    const GemmLaunchShape g = gemm_wide_shape(m, w.n, w.k);
    a.splits = g.splits; a.kt_per_split = g.kt_per_split;
    if (g.splits > 1) {
        if (mi355q_status st = ensure_workspace(ctx, (size_t)g.splits * m * w.n * sizeof(float))) return st;
        a.partial = (float*)ctx->workspace;
    }
    const bool sb_bf16 = w.sb_dtype == MI355Q_BF16;
    if (g.bm == 256) return launch_wide_bm<256>(s, a, w.group, sb_bf16);
    return launch_wide_bm<128>(s, a, w.group, sb_bf16);
}

}  // namespace mi355q
