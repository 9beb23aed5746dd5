// Projection of 17 to 96 activation rows on the matrix cores with the weights streamed through registers:
//   Y[M,N] = X[M,K] * W[N,K]^T,  W = 4- or 8-bit group-affine codes on the split planes, bf16 or f16 activations.
//
// Stands in, at these sequence lengths, for the reference's direct quantized GEMM gemm_q4_g64 / gemm_q4_g128 /
// gemm_q8_g32 / gemm_q8_g64 (Sources/MetalCompiler/Generator/MetalSourceGenerator+Quantized.swift:22-156) and for its dequant + matmul2d pair
// (MetalSourceGenerator+Linear.swift:18-81).  The tiled prefill kernel dequantises a weight K-tile into LDS once per
// workgroup and spends a barrier round trip on it whatever M is; with at most three 32-row blocks of activations the
// whole M extent fits one wavefront's accumulators, so here nothing but the activations goes through LDS:
//   * eight wavefronts of a workgroup own 64 weight rows: two blocks of 32 rows, each walked by four wavefronts
//     that take every fourth 64-code K-tile (K slice s takes tiles 4 i + s), so the four touch one 128-byte line of
//     a row together;
//   * lane (n, h) of a wavefront loads 16 bytes = words 4h .. 4h+3 of row n's K-tile and uses word j in k-step j:
//     the eight codes of a word become the B operand of v_mfma_f32_32x32x16_bf16 in registers (byte-lane convert,
//     fp32 fma with the group's scale and bias, one rounding to bf16: the weights of the tiled kernel, bit for bit;
//     with f16 activations one rounding to f16 and the f16 instruction; 8-bit codes: eight words a lane, two a k-step);
//     the A operand is the activations' chunk 4h + j of that K-tile, read from LDS;
//   * per iteration four more wavefronts of the workgroup stage [32 MB rows][256 columns] of activations
//     (XOR-swizzled 128-byte rows per K slice) two iterations ahead into the third of three LDS stages, copied
//     global -> LDS directly; the multiplying wavefronts fetch weight words three or six iterations ahead and wait for nothing
//     else; one barrier per iteration;
//   * up to 32 rows (groups of whole K-tiles) the operand holds the codes themselves and scale and bias are applied to
//     each K-tile's fp32 sums: unrounded weights, the decode kernels' arithmetic;
//   * weights left in the reference's interleaved blocks are read in place: a lane's 32 codes lie in one block behind
//     its (scale, zero) header (STAF payload, Sources/MetalCompiler/STAF/QuantizationFormat.swift:1121-1235);
//   * two or three matrices that share the activations (q+k+v, gate+up) run as one launch, each owning whole
//     workgroups; the gated MLP projection (Sources/MetalCompiler/Compilable/MLPFragment.swift:7-27) gives a workgroup's
//     first row block to gate_proj and its second to the same rows of up_proj and stores activation(gate) * up;
//   * the four K slices of a row block add their accumulators through LDS at the end, all twelve wavefronts sharing the
//     outputs; with K split over workgroups (few rows, long K) fp32 partial results go to scratch and a second launch
//     adds them.
#include "device_utils.h"
#include "gemm_stream.h"
#include <atomic>

#ifndef QBITS
#error "define QBITS (the code width this translation unit instantiates) before including gemm_stream.inl"
#endif

namespace mi355q {


typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 st_bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float st_floatx16_t;
typedef __bf16 st_bf16x2_v __attribute__((ext_vector_type(2)));
typedef float st_float2_v __attribute__((ext_vector_type(2)));
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 st_f16x8_t;
typedef _Float16 st_f16x2_v __attribute__((ext_vector_type(2)));

// iterations the weight words are fetched ahead (and the loop's unroll; a multiple of the three LDS stages): measured,
// 4096 -> 14336 at 32 rows 16.6 us with three against 17.1 with six and 19.7 with twelve, at 64 rows 22.0 / 21.1 / 26.2
constexpr int stream_ahead(int m_blocks) { return m_blocks == 1 ? 3 : 6; }
constexpr int kStreamThreads = 768;    // eight multiplying wavefronts and four that stage the activations

// two fp32 values rounded (to nearest even) to the activations' 16-bit type, the first in the low half
template <bool XF16>
__device__ __forceinline__ uint32_t st_pack(float lo, float hi) {
    st_float2_v v = {lo, hi};
    if constexpr (XF16) return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, st_f16x2_v));
    else return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, st_bf16x2_v));
}

// Byte offset of 16-byte chunk `chunk` of row `row` in a [rows][128 bytes] array: the chunk position is rotated by
// (row / 2) % 8, so sixteen consecutive rows reading or writing one logical chunk touch sixteen different bank groups.
__device__ __forceinline__ uint32_t st_lds_off(uint32_t row, uint32_t chunk) {
    return row * 128u + ((chunk ^ ((row >> 1) & 7u)) << 4);
}

// 16 bytes at an address that is a multiple of four
typedef uint32_t st_u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

// BLOCKS: the weights lie in the reference's interleaved blocks (one (scale f16, zero f16) header and the codes of a group
// each) instead of the planes; SB_BF16 is false then.
// EXACT (one block of activation rows, groups of 64 or 128): the operand holds the codes themselves, which bf16 and f16
// represent exactly, and scale and bias are applied to a K-tile's sums in fp32 -- acc += s * sum(q x) + z * sum(x), the
// decode kernels' arithmetic with unrounded weights; sum(x) comes from one more matrix instruction per k-step against
// an operand of ones.
template <int BITS, int GROUP, int MB, bool SB_BF16, bool XF16, bool BLOCKS, bool EXACT>
__global__ __launch_bounds__(kStreamThreads) void qgemm_stream_kernel(StreamArgs a) {
    static_assert(!EXACT || (MB == 1 && GROUP % 64 == 0), "scale and bias per K-tile: one row block, whole K-tiles per group");
    constexpr int LW = BITS;                              // words a lane loads per K-tile: 32 codes
    constexpr int TW = 2 * LW;                            // words of a row's K-tile
    constexpr bool WIDE_LOADS = BITS == 4 || BITS == 8;   // 16-byte loads; the other widths (2, 3, 5, 6 bits) word by word
    constexpr int RV = WIDE_LOADS ? LW / 4 : 1;
    constexpr int MPAD = 32 * MB;                         // staged activation rows
    constexpr int SLICE_BYTES = MPAD * 128;               // one K slice of a stage: [MPAD][64] bf16
    constexpr int STAGE = 4 * SLICE_BYTES;
    constexpr int XP = 4 * MB;                            // copy instructions (eight rows of a K slice each) per stage
    constexpr int U = stream_ahead(MB);
    extern __shared__ u32x4 smem_st[];
    char* const lds = (char*)smem_st;

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const bool stager = wave >= 8;                        // wavefronts 8..11 move the activations, 0..7 multiply
    const uint32_t rb = (wave >> 2) & 1u, slice = wave & 3u;     // row block, K slice
    const uint32_t ln = lane & 31, lh = lane >> 5;
    // the matrix of this workgroup; gated projection: of this row block (gate_proj, up_proj: rows n0 .. n0 + 31 of both)
    const bool gated = a.gated != 0;
    const bool in1 = gated ? rb == 1 : blockIdx.x >= a.wg_end[0], in2 = !gated && blockIdx.x >= a.wg_end[1];
    const uint32_t seg_n = in2 ? a.n[2] : in1 ? a.n[1] : a.n[0];
    const uint32_t n0 = gated ? blockIdx.x * 32 : (blockIdx.x - (in2 ? a.wg_end[1] : in1 ? a.wg_end[0] : 0u)) * kStreamRows + rb * 32;

    const uint32_t KT = a.k / 64;                         // K-tiles
    const uint32_t it_all = (a.k + kStreamIterK - 1) / kStreamIterK;
    const uint32_t it_begin = blockIdx.y * a.iters_per_part;
    const uint32_t it_end = it_begin + a.iters_per_part < it_all ? it_begin + a.iters_per_part : it_all;

    st_floatx16_t acc[MB];
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0.0f;

    if (stager) {
        // Activations, global -> LDS without a register in between (global_load_lds_dwordx4: lane L's 16 bytes land at
        // the base in M0 + 16 L), two iterations ahead into the third stage.  Staging wavefront w moves K slice w: one
        // instruction covers eight rows of the slice, and lane L fetches the chunk that belongs at its position after
        // the rotation of st_lds_off.  These wavefronts wait on nothing but their own copies (which hit the L2): were
        // the multiplying wavefronts to stage the activations themselves, every wait for a staged chunk would also
        // wait for the older weight loads, and the distance the weights are fetched ahead would shrink to that of the
        // activations.
        const uint32_t xs_slice = wave - 8;
        const uint32_t lds_base = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds) + xs_slice * SLICE_BYTES;
        const uint32_t xrow = lane >> 3;
        auto issue = [&](uint32_t stage, uint32_t it) __attribute__((always_inline)) {
            uint32_t col0 = it * kStreamIterK + xs_slice * 64;
            col0 = col0 + 64 <= a.k ? col0 : a.k - 64;    // a K slice past K has no tile there: what it stages is not read
#pragma unroll
            for (int q = 0; q < XP; q++) {
                const uint32_t row = 8 * q + xrow;
                const uint32_t chunk = (lane & 7u) ^ ((row >> 1) & 7u);
                const uint32_t r = row < a.m ? row : a.m - 1;
                const uint16_t* const g = a.x + (size_t)r * a.xs + col0 + chunk * 8;
                const uint32_t l = lds_base + stage * STAGE + q * 1024;
                asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(l) : "memory");
            }
        };
        issue(0, it_begin);
        if (it_begin + 1 < it_end) {
            issue(1, it_begin + 1);
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(XP) : "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        __syncthreads();
        for (uint32_t it0 = it_begin; it0 < it_end; it0 += 3) {
            static_for<3>([&](auto I) __attribute__((always_inline)) {
                constexpr int i = decltype(I)::value;
                const uint32_t it = it0 + i;
                if (it < it_end) {
                    // the stage iteration it - 1 was read from is free since the last barrier; iteration it + 1 must
                    // have landed before the next one
                    if (it + 2 < it_end) {
                        issue((i + 2) % 3, it + 2);
                        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(XP) : "memory");
                    } else {
                        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    }
                    __syncthreads();
                }
            });
        }
    } else {
        uint32_t wrow = n0 + ln;
        wrow = wrow < seg_n ? wrow : seg_n - 1;           // rows past the end re-read the last one
        const uint32_t* crow = nullptr;
        const uint32_t* szrow = nullptr;
        const uint8_t* brow = nullptr;
        if constexpr (BLOCKS) {
            brow = (in2 ? a.blocks[2] : in1 ? a.blocks[1] : a.blocks[0]) + (size_t)wrow * a.row_bytes;
        } else {
            crow = (in2 ? a.codes[2] : in1 ? a.codes[1] : a.codes[0]) +
                   (size_t)wrow * (in2 ? a.code_stride[2] : in1 ? a.code_stride[1] : a.code_stride[0]) + LW * lh;
            szrow = (in2 ? a.sz[2] : in1 ? a.sz[1] : a.sz[0]) +
                    (size_t)wrow * (in2 ? a.sz_stride[2] : in1 ? a.sz_stride[1] : a.sz_stride[0]);
        }
        // weight words and (scale, bias) word of this wavefront's K-tile of iteration `it`
        u32x4 ring[U][RV];
        uint32_t gring[U][WIDE_LOADS ? 1 : LW];            // the other widths: the lane's words one by one
        uint32_t szring[U];
        auto load_w = [&](auto I, uint32_t it) __attribute__((always_inline)) {
            constexpr int i = decltype(I)::value;
            uint32_t t = it * 4 + slice;
            t = t < KT ? t : KT - 1;
            if constexpr (BLOCKS) {
                // the lane's 32 codes start at code c0 of the row: block c0 / GROUP, behind its 4-byte header
                constexpr uint32_t BLOCK_BYTES = 4 + GROUP * BITS / 8;
                const uint32_t c0 = t * 64 + 32 * lh;
                const uint8_t* const blk = brow + (size_t)(c0 / GROUP) * BLOCK_BYTES;
                szring[i] = *(const uint32_t*)blk;
                if constexpr (WIDE_LOADS) {
#pragma unroll
                    for (int v = 0; v < RV; v++)
                        ring[i][v] = *(const st_u32x4_a4*)(blk + 4 + (c0 % GROUP) * BITS / 8 + 16 * v);
                } else {
                    const uint32_t* const p = (const uint32_t*)(blk + 4 + (c0 % GROUP) * BITS / 8);
#pragma unroll
                    for (int v = 0; v < LW; v++) gring[i][v] = p[v];
                }
            } else {
                if constexpr (WIDE_LOADS) {
#pragma unroll
                    for (int v = 0; v < RV; v++) ring[i][v] = *(const u32x4*)(crow + (size_t)t * TW + 4 * v);
                } else {
                    const uint32_t* const p = crow + (size_t)t * TW;
#pragma unroll
                    for (int v = 0; v < LW; v++) gring[i][v] = p[v];
                }
                szring[i] = szrow[(t * 64 + 32 * lh) / GROUP];     // the group of this lane's 32 codes
            }
        };
        static_for<U>([&](auto I) __attribute__((always_inline)) { load_w(I, it_begin + decltype(I)::value); });
        __syncthreads();
        for (uint32_t it0 = it_begin; it0 < it_end; it0 += U) {
            static_for<U>([&](auto I) __attribute__((always_inline)) {
                constexpr int i = decltype(I)::value;
                constexpr int stage = i % 3;
                const uint32_t it = it0 + i;
                if (it < it_end) {                        // the same for every wavefront of the workgroup
                    u32x4 w[RV];
                    uint32_t gw[WIDE_LOADS ? 1 : LW];
                    if constexpr (WIDE_LOADS) {
#pragma unroll
                        for (int v = 0; v < RV; v++) w[v] = ring[i][v];
                    } else {
#pragma unroll
                        for (int v = 0; v < LW; v++) gw[v] = gring[i][v];
                    }
                    const uint32_t szw = szring[i];
                    load_w(I, it + U);
                    if (it * 4 + slice < KT) {
                        float s, z;
                        if constexpr (SB_BF16) {
                            s = __uint_as_float(szw << 16); z = __uint_as_float(szw & 0xFFFF0000u);
                        } else {
                            s = f16_to_f32((uint16_t)(szw & 0xFFFFu)); z = f16_to_f32((uint16_t)(szw >> 16));
                        }
                        const char* const xs_lds = lds + stage * STAGE + slice * SLICE_BYTES;
                        st_floatx16_t dq, dx;                    // EXACT: this K-tile's sum(q x) and sum(x)
                        static_for<4>([&](auto J) __attribute__((always_inline)) {
                            constexpr int j = decltype(J)::value;
                            // the eight codes of k-step j as bytes: (c0,c2,c4,c6) and (c1,c3,c5,c7) of a 4-bit word,
                            // (c0..c3) and (c4..c7) of two 8-bit words
                            uint32_t lo = 0, hi = 0;
                            if constexpr (BITS == 4) {
                                const uint32_t word = w[0][j];
                                lo = word & 0x0F0F0F0Fu; hi = (word >> 4) & 0x0F0F0F0Fu;
                            } else if constexpr (BITS == 8) {
                                lo = w[j / 2][2 * (j % 2)]; hi = w[j / 2][2 * (j % 2) + 1];
                            } else {
                                // the other widths: codes 8 j .. 8 j + 7 of the lane's 32 as bytes, field by field
                                // (a field may straddle two words)
                                static_for<4>([&](auto E) __attribute__((always_inline)) {
                                    constexpr int e = decltype(E)::value;
                                    lo |= extract_code<(8 * j + e) * BITS, BITS, LW>(gw) << (8 * e);
                                    hi |= extract_code<(8 * j + 4 + e) * BITS, BITS, LW>(gw) << (8 * e);
                                });
                            }
                            float q[8];
                            constexpr int at0 = 0, at1 = BITS == 4 ? 2 : 1, at2 = BITS == 4 ? 4 : 2, at3 = BITS == 4 ? 6 : 3;
                            asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(q[at0]) : "v"(lo));
                            asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(q[at1]) : "v"(lo));
                            asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(q[at2]) : "v"(lo));
                            asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(q[at3]) : "v"(lo));
                            constexpr int bt0 = BITS == 4 ? 1 : 4, bt1 = BITS == 4 ? 3 : 5, bt2 = BITS == 4 ? 5 : 6, bt3 = 7;
                            asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(q[bt0]) : "v"(hi));
                            asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(q[bt1]) : "v"(hi));
                            asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(q[bt2]) : "v"(hi));
                            asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(q[bt3]) : "v"(hi));
                            u32x4 o;
                            if constexpr (EXACT) {
                                o.x = st_pack<XF16>(q[0], q[1]); o.y = st_pack<XF16>(q[2], q[3]);
                                o.z = st_pack<XF16>(q[4], q[5]); o.w = st_pack<XF16>(q[6], q[7]);
                                const u32x4 ax = *(const u32x4*)(xs_lds + st_lds_off(ln, 4 * lh + j));
                                constexpr uint32_t one2 = XF16 ? 0x3C003C00u : 0x3F803F80u;
                                const u32x4 ones = {one2, one2, one2, one2};
                                const st_floatx16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                                if constexpr (XF16) {
                                    dq = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(st_f16x8_t, ax), __builtin_bit_cast(st_f16x8_t, o), j == 0 ? zero : dq, 0, 0, 0);
                                    dx = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(st_f16x8_t, ax), __builtin_bit_cast(st_f16x8_t, ones), j == 0 ? zero : dx, 0, 0, 0);
                                } else {
                                    dq = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(st_bf16x8_t, ax), __builtin_bit_cast(st_bf16x8_t, o), j == 0 ? zero : dq, 0, 0, 0);
                                    dx = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(st_bf16x8_t, ax), __builtin_bit_cast(st_bf16x8_t, ones), j == 0 ? zero : dx, 0, 0, 0);
                                }
                                if constexpr (j == 3) {
#pragma unroll
                                    for (int r = 0; r < 16; r++) acc[0][r] = __builtin_fmaf(s, dq[r], __builtin_fmaf(z, dx[r], acc[0][r]));
                                }
                                return;
                            }
                            o.x = st_pack<XF16>(__builtin_fmaf(s, q[0], z), __builtin_fmaf(s, q[1], z));
                            o.y = st_pack<XF16>(__builtin_fmaf(s, q[2], z), __builtin_fmaf(s, q[3], z));
                            o.z = st_pack<XF16>(__builtin_fmaf(s, q[4], z), __builtin_fmaf(s, q[5], z));
                            o.w = st_pack<XF16>(__builtin_fmaf(s, q[6], z), __builtin_fmaf(s, q[7], z));
#pragma unroll
                            for (int b = 0; b < MB; b++) {
                                const u32x4 ax = *(const u32x4*)(xs_lds + st_lds_off(b * 32 + ln, 4 * lh + j));
                                if constexpr (XF16)
                                    acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(st_f16x8_t, ax),
                                                                                    __builtin_bit_cast(st_f16x8_t, o), acc[b], 0, 0, 0);
                                else
                                    acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(st_bf16x8_t, ax),
                                                                                     __builtin_bit_cast(st_bf16x8_t, o), acc[b], 0, 0, 0);
                            }
                            if constexpr (MB >= 3) __builtin_amdgcn_sched_barrier(0);   // one word at a time: registers
                        });
                    }
                    __syncthreads();
                }
            });
        }
    }

    // ---- the four K slices of a row block add up through LDS (the staged activations are done with) ----------------
    // Every multiplying wavefront parks its accumulators; then all twelve wavefronts, the staging ones too, share the
    // outputs register by register (a lane's position in the 32 x 32 tile is the same in every wavefront): slice 0 + 1 +
    // 2 + 3 in that order, then the store -- or, gated, activation(gate sums) * (up sums) of the two row blocks.  One
    // wavefront a row block doing all of it costs 4 us a workgroup with the activation, 1 us without.
    constexpr uint32_t T = 16 * MB * 64;                  // floats of one wavefront's accumulators
    float* const red = (float*)lds;
    if (!stager) {
        float* const mine = red + (size_t)(rb * 4 + slice) * T;
#pragma unroll
        for (int b = 0; b < MB; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) mine[(b * 16 + r) * 64 + lane] = acc[b][r];
    }
    __syncthreads();
    const uint32_t wg_n0 = gated ? n0 : n0 - rb * 32;     // the workgroup's first weight row
    void* const seg_y = in2 ? a.y[2] : (!gated && in1) ? a.y[1] : a.y[0];
    const uint32_t seg_ys = in2 ? a.ys[2] : (!gated && in1) ? a.ys[1] : a.ys[0];
    const uint32_t pcol0 = in2 ? a.col0[2] : (!gated && in1) ? a.col0[1] : a.col0[0];
#pragma nounroll
    for (uint32_t i = wave; i < (gated ? 1u : 2u) * 16u * MB; i += kStreamThreads / 64) {
        const uint32_t rbx = i / (16u * MB), j = i - rbx * (16u * MB), r = j & 15u;
        const uint32_t row = (j >> 4) * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
        const uint32_t col = wg_n0 + rbx * 32 + ln;
        if (row >= a.m || col >= seg_n) continue;
        const float* const p = red + (size_t)(rbx * 4) * T + j * 64 + lane;
        float v = ((p[0] + p[T]) + p[2 * T]) + p[3 * T];
        if (gated) {
            const float* const q = p + 4 * T;
            v = gated_value(v, ((q[0] + q[T]) + q[2 * T]) + q[3 * T], a.gated - 1, a.y_dtype);
        } else if (a.partial) {
            a.partial[((size_t)blockIdx.y * a.m + row) * a.n_total + pcol0 + col] = v;
            continue;
        }
        const size_t o = (size_t)row * seg_ys + col;
        if (a.y_dtype == MI355Q_F32) ((float*)seg_y)[o] = v;
        else if (a.y_dtype == MI355Q_BF16) ((uint16_t*)seg_y)[o] = f32_to_bf16_rne(v);
        else ((uint16_t*)seg_y)[o] = f32_to_f16_rne(v);
    }
}

namespace {

template <int BITS, int GROUP, int MB, bool SB_BF16, bool XF16, bool BLOCKS, bool EXACT = false>
mi355q_status launch_stream_mb(hipStream_t s, const StreamArgs& a, const StreamLaunchShape& g) {
    auto kern = qgemm_stream_kernel<BITS, GROUP, MB, SB_BF16, XF16, BLOCKS, EXACT>;
    if (g.lds_bytes > 64u * 1024u) {
        // the attribute belongs to the function on one device: one bit per device and instantiation
        static std::atomic<uint64_t> lds_limit_raised{0};
        int device = 0;
        MI355Q_HIP(hipGetDevice(&device));
        const uint64_t bit = 1ull << (device & 63);
        if (!(lds_limit_raised.load(std::memory_order_relaxed) & bit)) {
            MI355Q_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)g.lds_bytes));
            lds_limit_raised.fetch_or(bit, std::memory_order_relaxed);
        }
    }
    kern<<<dim3(g.row_blocks, g.parts), dim3(kStreamThreads), g.lds_bytes, s>>>(a);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

template <int BITS, int GROUP, bool SB_BF16, bool XF16, bool BLOCKS>
mi355q_status launch_stream_blocks(hipStream_t s, const StreamArgs& a, const StreamLaunchShape& g) {
    switch (g.m_blocks) {
    case 1:
        if constexpr (GROUP % 64 == 0) {
            if (a.exact) return launch_stream_mb<BITS, GROUP, 1, SB_BF16, XF16, BLOCKS, true>(s, a, g);
        }
        return launch_stream_mb<BITS, GROUP, 1, SB_BF16, XF16, BLOCKS>(s, a, g);
    case 2: return launch_stream_mb<BITS, GROUP, 2, SB_BF16, XF16, BLOCKS>(s, a, g);
    case 3: return launch_stream_mb<BITS, GROUP, 3, SB_BF16, XF16, BLOCKS>(s, a, g);
    default: break;
    }
    return fail(MI355Q_ERR_SHAPE, "the streamed-weight kernel takes at most %u rows", kStreamMaxRows);
}

template <int BITS, int GROUP>
mi355q_status launch_stream_group(hipStream_t s, const StreamArgs& a, const StreamLaunchShape& g, bool sb_bf16, bool x_f16,
                                  bool blocks) {
    if (blocks)     // block headers are f16
        return x_f16 ? launch_stream_blocks<BITS, GROUP, false, true, true>(s, a, g) : launch_stream_blocks<BITS, GROUP, false, false, true>(s, a, g);
    if (sb_bf16) return x_f16 ? launch_stream_blocks<BITS, GROUP, true, true, false>(s, a, g) : launch_stream_blocks<BITS, GROUP, true, false, false>(s, a, g);
    return x_f16 ? launch_stream_blocks<BITS, GROUP, false, true, false>(s, a, g) : launch_stream_blocks<BITS, GROUP, false, false, false>(s, a, g);
}

}  // namespace

#define MI355Q_STREAM_CAT2(a, b) a##b
#define MI355Q_STREAM_CAT(a, b) MI355Q_STREAM_CAT2(a, b)

mi355q_status MI355Q_STREAM_CAT(launch_stream_q, QBITS)(hipStream_t s, const StreamArgs& a, const StreamLaunchShape& g,
                                                       uint32_t group, bool sb_bf16, bool x_f16, bool blocks) {
#if QBITS == 4
    if (group == 64) return launch_stream_group<4, 64>(s, a, g, sb_bf16, x_f16, blocks);
    if (group == 128) return launch_stream_group<4, 128>(s, a, g, sb_bf16, x_f16, blocks);
#elif QBITS == 8
    if (group == 32) return launch_stream_group<8, 32>(s, a, g, sb_bf16, x_f16, blocks);
    if (group == 64) return launch_stream_group<8, 64>(s, a, g, sb_bf16, x_f16, blocks);
    if (group == 128) return launch_stream_group<8, 128>(s, a, g, sb_bf16, x_f16, blocks);
#else
    if (group == 64) return launch_stream_group<QBITS, 64>(s, a, g, sb_bf16, x_f16, blocks);
#endif
    return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no streamed-weight kernel for q%d g%u", QBITS, group);
}

}  // namespace mi355q
