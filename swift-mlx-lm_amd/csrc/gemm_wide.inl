// Kernel text of the wide-tile prefill GEMM; included by gemm_wide_bf16.hip and gemm_wide_f16.hip, which set
// WIDE_XF16 (the activation type) so that the two halves of the instantiations compile side by side.
#include "gemm_wide.h"
#include "device_utils.h"
#include <atomic>

namespace mi355q {

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 wd_bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 wd_f16x8_t;
typedef _Float16 wd_f16x2_v __attribute__((ext_vector_type(2)));
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float wd_floatx16_t;
typedef __bf16 wd_bf16x2_v __attribute__((ext_vector_type(2)));
typedef float wd_float2_v __attribute__((ext_vector_type(2)));
typedef float wd_float4_v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t wd_pack_bf16(float lo, float hi) {
    wd_float2_v v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, wd_bf16x2_v));
}
__device__ __forceinline__ uint32_t wd_pack_f16(float lo, float hi) {       // round to nearest even, as the bf16 pair
    wd_float2_v v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, wd_f16x2_v));
}

// A wave-uniform address as the scalar operand of hand-written memory instructions, wherever the compiler computed it
__device__ __forceinline__ const char* wd_scalar(const char* p) {
    const uint64_t v = (uint64_t)(uintptr_t)p;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return (const char*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

// BLOCKS: the weights are the reference's interleaved blocks read in place (f16 scale, f16 zero, then the group's codes:
// 36 bytes per 64 codes, 68 per 128); a lane's sixteen code bytes then sit at a 4-byte aligned address and the
// (scale, zero) pair of a K-tile is one more 4-byte load.  XF16: f16 activations, weights rounded to f16, f16 MFMA.
template <int BM, bool SB_BF16, int GROUP, bool BLOCKS, bool XF16>
__global__ __launch_bounds__(256, (BM == 128 ? 2 : 1)) void qgemm_wide_kernel(WideArgs a) {
    constexpr int TM = BM / 32;                     // activation fragments = groups per k-step
    constexpr int A_STAGE = BM * 128;
    constexpr int AQ = BM / 32;                     // activation copies per wavefront and K-tile (8 rows each)
    constexpr int CPK = AQ / 4;                     // ... and per k-step
    constexpr int SZW = 4 * 64 / GROUP;             // (scale, bias) words of four K-tiles
    constexpr int WL = 8 + (BLOCKS ? 2 * SZW : 2);  // weight + (scale, bias) loads per wavefront and four K-tiles
    constexpr int BLOCK_BYTES = 4 + GROUP / 2;      // blocks in place: one group
    constexpr int FOUR_BYTES = BLOCKS ? BLOCK_BYTES * 256 / GROUP : 128;   // a row's codes of four K-tiles (with their headers)
    using frag_t = std::conditional_t<XF16, wd_f16x8_t, wd_bf16x8_t>;
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
    const uint32_t tn_all = tile / a.tiles_m, tm = tile % a.tiles_m;
    // the matrix of this column tile (one of up to three that share the activations): its weights here, its result in
    // the epilogue, which asks again -- nothing of the choice is kept in registers over the K loop but the tile's number
    uint32_t tn = tn_all;
    const uint32_t* seg_codes = a.codes;
    const uint32_t* seg_sz = a.sz;
    const uint8_t* seg_blocks = a.blocks;
    uint32_t w_n = a.n;
    if (a.segments > 1 && tn_all >= a.seg_tile0[0]) {
        const uint32_t sg_ = tn_all >= a.seg_tile0[1] ? 1u : 0u;
        seg_codes = a.seg_codes[sg_]; seg_sz = a.seg_sz[sg_]; seg_blocks = a.seg_blocks[sg_];
        w_n = a.seg_n[sg_];
        tn -= a.seg_tile0[sg_];
    }
    // Gated (a.gated != 0): the two 32-column fragments of a wavefront are the same 32 output columns of gate_proj and of
    // up_proj, so a tile is 128 output columns wide and activation(gate) * up is formed in the registers of the epilogue.
    const uint32_t tile_cols = a.gated ? kWideBN / 2 : kWideBN;
    const uint32_t m0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tm * BM)), n0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tn * tile_cols));
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
    const uint32_t n_last = w_n - 1 - n0;
    uint32_t w_off[2], sz_off[2];
#pragma unroll
    for (int f = 0; f < 2; f++) {
        const uint32_t r = a.gated ? 32 * wave + ln : 64 * wave + 32 * f + ln;
        const uint32_t gr = r < n_last ? r : n_last;
        if constexpr (BLOCKS) {
            sz_off[f] = gr * a.row_bytes;                 // the header of the row's first block
            w_off[f] = sz_off[f] + 4 + lh * 16;
        } else {
            w_off[f] = gr * a.code_stride * 4 + lh * 16;
            sz_off[f] = gr * a.sz_stride * 4;
        }
    }
    const char* const cg = BLOCKS ? (const char*)seg_blocks + (size_t)n0 * a.row_bytes : (const char*)(seg_codes + (size_t)n0 * a.code_stride);
    const char* const sg = BLOCKS ? cg : (const char*)(seg_sz + (size_t)n0 * a.sz_stride);
    // the second fragment's matrix: up_proj where gated, else the same one
    const char* const cg1 = !a.gated ? cg : BLOCKS ? (const char*)a.blocks_up + (size_t)n0 * a.row_bytes
                                                   : (const char*)(a.codes_up + (size_t)n0 * a.code_stride);
    const char* const sg1 = !a.gated ? sg : BLOCKS ? cg1 : (const char*)(a.sz_up + (size_t)n0 * a.sz_stride);
    const uint32_t four_begin = kt_begin / 4;
    using sz_vec = std::conditional_t<SZW == 4, u32x4, u32x2>;      // kept whole: the loads write them behind the compiler's back
    u32x4 wnext[2][4], wcur[2][4];
    sz_vec sznext[2];
    uint32_t szone[2][SZW];                                         // blocks in place: one word per K-tile (g64) or per two
    uint32_t szcur[2][SZW];
    auto load_w = [&](uint32_t four) __attribute__((always_inline)) {
        uint32_t p = four_begin + (four * 4 < KT ? four : KT / 4 - 1);
        p = p >= a.w_fours ? p - a.w_fours : p;      // the second half of [hi | lo] activations meets the same weights again
        const char* const gb[2] = {wd_scalar(cg + (size_t)p * FOUR_BYTES), wd_scalar(cg1 + (size_t)p * FOUR_BYTES)};
        const char* const gsb[2] = {BLOCKS ? gb[0] : wd_scalar(sg + (size_t)p * (SZW * 4)),
                                    BLOCKS ? gb[1] : wd_scalar(sg1 + (size_t)p * (SZW * 4))};
#pragma unroll
        for (int f = 0; f < 2; f++) {
            const char* const g = gb[f];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                // K-tile t of the four: 32 bytes on in the planes; in blocks, behind the header of its group
                asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3"
                             : "=v"(wnext[f][t])
                             : "v"(w_off[f]), "s"(g), "n"(!BLOCKS ? t * 32 : GROUP == 64 ? t * BLOCK_BYTES : (t / 2) * BLOCK_BYTES + (t % 2) * 32)
                             : "memory");
            }
        }
#pragma unroll
        for (int f = 0; f < 2; f++) {
            const char* const gs = gsb[f];
            if constexpr (BLOCKS) {
#pragma unroll
                for (int i = 0; i < SZW; i++)
                    asm volatile("global_load_dword %0, %1, %2 offset:%3" : "=v"(szone[f][i]) : "v"(sz_off[f]), "s"(gs), "n"(i * BLOCK_BYTES) : "memory");
            } else if constexpr (SZW == 4) {
                asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(sznext[f]) : "v"(sz_off[f]), "s"(gs) : "memory");
            } else {
                asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(sznext[f]) : "v"(sz_off[f]), "s"(gs) : "memory");
            }
        }
    };
    // waits until at most `younger` vector-memory operations issued after the weight loads are outstanding, then
    // takes the loaded words over
    auto take_w = [&](auto YOUNGER) __attribute__((always_inline)) {
        constexpr int younger = decltype(YOUNGER)::value;
        if constexpr (!BLOCKS) {
            asm volatile("s_waitcnt vmcnt(%10)"
                         : "+v"(wnext[0][0]), "+v"(wnext[0][1]), "+v"(wnext[0][2]), "+v"(wnext[0][3]), "+v"(wnext[1][0]),
                           "+v"(wnext[1][1]), "+v"(wnext[1][2]), "+v"(wnext[1][3]), "+v"(sznext[0]), "+v"(sznext[1])
                         : "n"(younger)
                         : "memory");
        } else if constexpr (SZW == 4) {
            asm volatile("s_waitcnt vmcnt(%16)"
                         : "+v"(wnext[0][0]), "+v"(wnext[0][1]), "+v"(wnext[0][2]), "+v"(wnext[0][3]), "+v"(wnext[1][0]),
                           "+v"(wnext[1][1]), "+v"(wnext[1][2]), "+v"(wnext[1][3]), "+v"(szone[0][0]), "+v"(szone[0][1]),
                           "+v"(szone[0][2]), "+v"(szone[0][3]), "+v"(szone[1][0]), "+v"(szone[1][1]), "+v"(szone[1][2]),
                           "+v"(szone[1][3])
                         : "n"(younger)
                         : "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(%12)"
                         : "+v"(wnext[0][0]), "+v"(wnext[0][1]), "+v"(wnext[0][2]), "+v"(wnext[0][3]), "+v"(wnext[1][0]),
                           "+v"(wnext[1][1]), "+v"(wnext[1][2]), "+v"(wnext[1][3]), "+v"(szone[0][0]), "+v"(szone[0][1]),
                           "+v"(szone[1][0]), "+v"(szone[1][1])
                         : "n"(younger)
                         : "memory");
        }
#pragma unroll
        for (int f = 0; f < 2; f++) {
#pragma unroll
            for (int t = 0; t < 4; t++) wcur[f][t] = wnext[f][t];
#pragma unroll
            for (int i = 0; i < SZW; i++) szcur[f][i] = BLOCKS ? szone[f][i] : sznext[f][i];
        }
    };

    // ---- operands ----------------------------------------------------------------------------------
    // activation fragment (i, j): rows 32 i + ln, chunk 4 lh + j -- the K positions lane (., h) holds of word j
    uint32_t a_rd[4];
#pragma unroll
    for (int j = 0; j < 4; j++) a_rd[j] = ln * 128 + (((4 * lh + j) ^ ((ln >> 1) & 7u)) << 4);

    frag_t xf[2][TM], wf[2][2];
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
        const float w0 = __builtin_fmaf(sc[f], q0, zr[f]), w1 = __builtin_fmaf(sc16[f], q1, zr[f]);
        return XF16 ? wd_pack_f16(w0, w1) : wd_pack_bf16(w0, w1);
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
            xf[buf ^ 1][q] = *(const frag_t*)(xs_next + q * 4096);
            if constexpr (XF16) {
                acc[0][q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[buf][0], xf[buf][q], acc[0][q], 0, 0, 0);
                acc[1][q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[buf][1], xf[buf][q], acc[1][q], 0, 0, 0);
            } else {
                acc[0][q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[buf][0], xf[buf][q], acc[0][q], 0, 0, 0);
                acc[1][q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[buf][1], xf[buf][q], acc[1][q], 0, 0, 0);
            }
            // eight pieces (two fragments of four) over the TM groups
            static_for<8 / TM>([&](auto P) __attribute__((always_inline)) {
                constexpr int piece = q * (8 / TM) + decltype(P)::value;
                constexpr int f = piece / 4, b = piece % 4;
                dq_o[f][b] = dq_piece(std::integral_constant<int, f>{}, std::integral_constant<int, b>{}, wcur[f][tn_][jn]);
                if constexpr (b == 3) wf[buf ^ 1][f] = __builtin_bit_cast(frag_t, dq_o[f]);
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
    for (int i = 0; i < TM; i++) xf[0][i] = *(const frag_t*)(lds + a_rd[0] + i * 4096);
    static_for<2>([&](auto F) __attribute__((always_inline)) {
        constexpr int f = decltype(F)::value;
        u32x4 o;
        o.x = dq_piece(F, I0{}, wcur[f][0][0]);
        o.y = dq_piece(F, I1{}, wcur[f][0][0]);
        o.z = dq_piece(F, I2{}, wcur[f][0][0]);
        o.w = dq_piece(F, I3{}, wcur[f][0][0]);
        wf[0][f] = __builtin_bit_cast(frag_t, o);
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
    // the result of this tile's matrix (asked again, from a copy of the tile's number the compiler takes for another)
    uint32_t tn_again = tn_all;
    asm volatile("" : "+s"(tn_again));
    void* seg_y = a.y;
    uint32_t seg_n = a.n, seg_ys = a.ys, part_col0 = 0, part_pitch = a.n;
    if (a.segments > 1) {
        part_pitch = a.n_total;
        if (tn_again >= a.seg_tile0[0]) {
            const uint32_t sg_ = tn_again >= a.seg_tile0[1] ? 1u : 0u;
            seg_y = a.seg_y[sg_]; seg_n = a.seg_n[sg_]; seg_ys = a.seg_ys[sg_]; part_col0 = a.seg_col0[sg_];
        }
    }
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
                        if (wide && col + 3 < seg_n) {
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
                                if (col + e < seg_n) store_out<dt>(y, o + e, v[e]);
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        });
    };
    // Whole cache lines instead: a wavefront's 32 rows x 64 columns of one accumulator row pass through LDS (the
    // activation stages are free now), are read back eight (fp32: four) rows at a time with sixteen bytes per lane, and
    // go out as full 128-byte lines.  (Stores of eight bytes per lane, 32 rows apart, as the loop above makes them,
    // took 11 us per tile when every workgroup of a round stored at once; these take about 3.)  Taken when the tile's
    // 256 columns lie inside the matrix and the rows of y are 16-byte aligned.
    auto store_lines = [&](auto DT, void* const y, const size_t ys) __attribute__((always_inline)) {
        constexpr int dt = decltype(DT)::value;
        constexpr int ESZ = dt == MI355Q_F32 ? 4 : 2;
        constexpr int PITCH = 64 * ESZ + 16;                       // a row of the staging block: 16 bytes of padding
        constexpr int RPI = ESZ == 4 ? 4 : 8;                      // rows per read-back instruction
        constexpr int LPR = 64 / RPI;                              // lanes per row
        char* const stage = lds + wave * (32 * PITCH);
        __builtin_amdgcn_s_barrier();                              // every wavefront is done with the activation stages
        static_for<TM>([&](auto I) __attribute__((always_inline)) {
            constexpr int i = decltype(I)::value;
            asm volatile("" : "+v"(acc[0][i]), "+v"(acc[1][i]));
#pragma unroll
            for (int f = 0; f < 2; f++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const float v0 = acc[f][i][4 * g + 0], v1 = acc[f][i][4 * g + 1], v2 = acc[f][i][4 * g + 2], v3 = acc[f][i][4 * g + 3];
                    char* const at = stage + ln * PITCH + (32 * f + 8 * g + 4 * lh) * ESZ;
                    if constexpr (dt == MI355Q_F32) {
                        const wd_float4_v t = {v0, v1, v2, v3};
                        *(wd_float4_v*)at = t;
                    } else {
                        u32x2 t;
                        t.x = dt == MI355Q_BF16 ? wd_pack_bf16(v0, v1) : wd_pack_f16(v0, v1);
                        t.y = dt == MI355Q_BF16 ? wd_pack_bf16(v2, v3) : wd_pack_f16(v2, v3);
                        *(u32x2*)at = t;
                    }
                }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int t = 0; t < 32 / RPI; t++) {
                const uint32_t r = t * RPI + lane / LPR, piece = lane % LPR;
                const u32x4 d = *(const u32x4*)(stage + r * PITCH + piece * 16);
                const uint32_t row = m0 + i * 32 + r;
                if (row < a.m)
                    *(u32x4*)((char*)y + ((size_t)row * ys + n0 + 64 * wave) * ESZ + piece * 16) = d;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        });
    };
    // Gated: activation(gate) * up where the two accumulators of a row block meet (gate and up values rounded to the
    // output type first, as the reference's elementwise kernel reads them from buffers of that type), the 32 x 32
    // results of a wavefront through LDS and out in 16-byte pieces; tiles at the edge of the matrix element by element.
    auto store_gated = [&](auto DT) __attribute__((always_inline)) {
        constexpr int dt = decltype(DT)::value;
        constexpr int ESZ = dt == MI355Q_F32 ? 4 : 2;
        constexpr int PITCH = 32 * ESZ + 16;
        constexpr int LPR = 32 * ESZ / 16;                         // lanes per row of the read-back
        constexpr int RPI = 64 / LPR;                              // rows per read-back instruction
        char* const stage = lds + wave * (32 * PITCH);
        const bool whole = n0 + kWideBN / 2 <= seg_n && a.line_stores;
        const uint32_t act = a.gated - 1;
        __builtin_amdgcn_s_barrier();                              // every wavefront is done with the activation stages
        static_for<TM>([&](auto I) __attribute__((always_inline)) {
            constexpr int i = decltype(I)::value;
            asm volatile("" : "+v"(acc[0][i]), "+v"(acc[1][i]));
            float v[16];
#pragma unroll
            for (int r = 0; r < 16; r++) v[r] = gated_value(acc[0][i][r], acc[1][i][r], act, (uint32_t)dt);
            if (whole) {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    char* const at = stage + ln * PITCH + (8 * g + 4 * lh) * ESZ;
                    if constexpr (dt == MI355Q_F32) {
                        const wd_float4_v t = {v[4 * g], v[4 * g + 1], v[4 * g + 2], v[4 * g + 3]};
                        *(wd_float4_v*)at = t;
                    } else {
                        u32x2 t;
                        t.x = dt == MI355Q_BF16 ? wd_pack_bf16(v[4 * g], v[4 * g + 1]) : wd_pack_f16(v[4 * g], v[4 * g + 1]);
                        t.y = dt == MI355Q_BF16 ? wd_pack_bf16(v[4 * g + 2], v[4 * g + 3]) : wd_pack_f16(v[4 * g + 2], v[4 * g + 3]);
                        *(u32x2*)at = t;
                    }
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
                for (int t = 0; t < 32 / RPI; t++) {
                    const uint32_t r = t * RPI + lane / LPR, piece = lane % LPR;
                    const u32x4 d = *(const u32x4*)(stage + r * PITCH + piece * 16);
                    const uint32_t row = m0 + i * 32 + r;
                    if (row < a.m)
                        *(u32x4*)((char*)seg_y + ((size_t)row * seg_ys + n0 + 32 * wave) * ESZ + piece * 16) = d;
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            } else {
                const uint32_t row = m0 + i * 32 + ln;
                if (row < a.m) {
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const uint32_t col = n0 + 32 * wave + 8 * (r / 4) + 4 * lh + r % 4;
                        if (col < seg_n) store_out<dt>(seg_y, (size_t)row * seg_ys + col, v[r]);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    if (a.gated) {
        if (a.y_dtype == MI355Q_BF16) store_gated(std::integral_constant<int, MI355Q_BF16>{});
        else if (a.y_dtype == MI355Q_F32) store_gated(std::integral_constant<int, MI355Q_F32>{});
        else store_gated(std::integral_constant<int, MI355Q_F16>{});
        return;
    }
    const bool inner = n0 + kWideBN <= seg_n;                        // (uniform over the workgroup)
    if (a.partial) {       // this part of K as fp32 (N is a multiple of four: 16-byte stores); wide_reduce_kernel adds the parts
        float* const part = a.partial + (size_t)split * a.m * part_pitch + part_col0;
        if (inner) store_lines(std::integral_constant<int, MI355Q_F32>{}, part, part_pitch);
        else store_tiles(std::integral_constant<int, MI355Q_F32>{}, part, part_pitch, true);
        return;
    }
    const bool lines = inner && a.line_stores;
    if (a.y_dtype == MI355Q_BF16) {
        if (lines) store_lines(std::integral_constant<int, MI355Q_BF16>{}, seg_y, seg_ys);
        else store_tiles(std::integral_constant<int, MI355Q_BF16>{}, seg_y, seg_ys, a.wide_stores != 0);
    } else if (a.y_dtype == MI355Q_F32) {
        if (lines) store_lines(std::integral_constant<int, MI355Q_F32>{}, seg_y, seg_ys);
        else store_tiles(std::integral_constant<int, MI355Q_F32>{}, seg_y, seg_ys, a.wide_stores != 0);
    } else {
        if (lines) store_lines(std::integral_constant<int, MI355Q_F16>{}, seg_y, seg_ys);
        else store_tiles(std::integral_constant<int, MI355Q_F16>{}, seg_y, seg_ys, a.wide_stores != 0);
    }
}


template <int BM, bool SB_BF16, int GROUP, bool BLOCKS>
mi355q_status launch_wide_tile(hipStream_t s, WideArgs a) {
    a.tiles_m = (a.m + BM - 1) / BM;
    if (a.segments <= 1) a.tiles_n = a.gated ? (a.n + kWideBN / 2 - 1) / (kWideBN / 2) : (a.n + kWideBN - 1) / kWideBN;
    const uint32_t grid = (a.tiles_m * a.tiles_n * a.splits + 7) / 8 * 8;
    constexpr size_t lds = (size_t)kWideStages * BM * 128;
    auto kern = qgemm_wide_kernel<BM, SB_BF16, GROUP, BLOCKS, WIDE_XF16 != 0>;
    if (mi355q_status st = raise_lds_limit((const void*)kern, lds)) return st;
    kern<<<dim3(grid), dim3(256), lds, s>>>(a);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

template <int BM>
mi355q_status launch_wide_bm(hipStream_t s, const WideArgs& a, uint32_t group, bool sb_bf16, bool blocks) {
    if (blocks) return group == 64 ? launch_wide_tile<BM, false, 64, true>(s, a) : launch_wide_tile<BM, false, 128, true>(s, a);
    if (group == 64) return sb_bf16 ? launch_wide_tile<BM, true, 64, false>(s, a) : launch_wide_tile<BM, false, 64, false>(s, a);
    return sb_bf16 ? launch_wide_tile<BM, true, 128, false>(s, a) : launch_wide_tile<BM, false, 128, false>(s, a);
}

}  // namespace

#if WIDE_XF16
mi355q_status launch_wide_kernel_f16(hipStream_t s, WideArgs a, uint32_t bm, uint32_t group, bool sb_bf16, bool blocks) {
#else
mi355q_status launch_wide_kernel_bf16(hipStream_t s, WideArgs a, uint32_t bm, uint32_t group, bool sb_bf16, bool blocks) {
#endif
    return bm == 256 ? launch_wide_bm<256>(s, a, group, sb_bf16, blocks) : launch_wide_bm<128>(s, a, group, sb_bf16, blocks);
}

}  // namespace mi355q
