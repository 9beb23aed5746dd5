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
//     (two workgroups per CU); where 256-row tiles would leave CUs idle, K goes over workgroups in parts.
// The kernel text is gemm_wide.inl; this file chooses the shape, launches, and adds the parts of K.
#include "gemm_wide.h"
#include "device_utils.h"
#include <atomic>

namespace mi355q {

namespace {

typedef __bf16 wd_bf16x2_v __attribute__((ext_vector_type(2)));
typedef float wd_float2_v __attribute__((ext_vector_type(2)));
typedef float wd_float4_v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t wd_pack_bf16(float lo, float hi) {
    wd_float2_v v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, wd_bf16x2_v));
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

}  // namespace

// 4 bits in groups of 64 or 128, bf16 or f16 activations, K a multiple of four K-tiles.  Planes: 16-byte aligned rows
// of codes and of (scale, bias) words (a row's words of four K-tiles are one 16- or 8-byte load).  Blocks in place:
// whole blocks of 4 + group / 2 bytes at a 4-byte aligned address.
bool gemm_wide_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride) {
    if ((x_dtype != MI355Q_BF16 && x_dtype != MI355Q_F16 && x_dtype != MI355Q_F32) || m < 1) return false;
    if (x_dtype == MI355Q_F32 && x_stride % 4) return false;        // 16-byte loads of the rows that are split
    if (w.bits != 4 || (w.group != 64 && w.group != 128)) return false;
    if (w.k % 256 || x_stride % 8) return false;
    if ((uint64_t)x_stride * 2 * 256 >= (1ull << 32)) return false;               // offsets inside a tile are 32-bit
    if (w.layout == MI355Q_LAYOUT_STAF_BLOCKS) {
        if (!w.blocks || (uintptr_t)w.blocks % 4 || w.bytes_per_block != 4 + w.group / 2) return false;
        return (uint64_t)w.blocks_per_row * w.bytes_per_block * 256 < (1ull << 32);
    }
    if (w.layout != MI355Q_LAYOUT_PLANES || !w.sz || !w.codes) return false;
    if ((uintptr_t)w.codes % 16 || w.code_stride % 4) return false;
    if ((uintptr_t)w.sz % 16 || w.sz_stride % 4) return false;
    return (uint64_t)w.code_stride * 4 * 256 < (1ull << 32);
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
GemmLaunchShape gemm_wide_shape(uint32_t m, uint32_t n, uint32_t k, bool one_part) {
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
            if (one_part ? splits != 1 : forced_splits && splits != forced_splits) continue;
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
// the two-dispatch route: enough workgroups (tiles x K parts) to occupy five eighths of the CUs.  4096 -> 14336: 34 us
// at 128 rows (128-row tiles, K in four parts) against 41 us on the tiled kernel, 47 against 56-59 at 192 and 256, 57
// against 78 at 320; 14336 -> 4096 has too few column tiles below 320 rows (59-62 us against 40-55) and changes over
// there (63 against 78).
bool gemm_wide_chosen(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride) {
    if (!gemm_wide_eligible(w, x_dtype, m, x_stride) || m < kWideMinRows) return false;
    const GemmLaunchShape g = gemm_wide_shape(m, w.n, gemm_wide_k(w.k, x_dtype));
    const uint32_t wgs = ((m + g.bm - 1) / g.bm) * ((w.n + kWideBN - 1) / kWideBN) * g.splits;
    // where the tiled kernel does not read the weight or the activation type (blocks in place, f16 and fp32 rows) the
    // other route is the two-dispatch one, and half of the CUs are enough: 8192 -> 8192 on blocks with f16 rows 46-48 us at
    // 100-128 rows against 66-72 us, 14336 -> 4096 70 against 82 at 256 rows, 4096 -> 4096 33-35 against 38 at 192-256
    // (with a quarter of the CUs 14336 -> 4096 loses a tenth at 100-128 rows and 8192 -> 2048 a fifth throughout)
    return 8 * wgs >= (gemm_mfma_eligible(w, x_dtype, m, x_stride) ? 5 : 4) * chip_cus();
}

mi355q_status launch_qgemm_wide(hipStream_t s, mi355q_context* ctx, const WView& w, const void* x, int x_dtype, void* y,
                                int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride, unsigned long long* probe) {
    if (!gemm_wide_eligible(w, x_dtype, m, x_stride))
        return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the wide-tile MFMA GEMM does not accept this format, layout or stride");
    if ((uintptr_t)x % 16) return fail(MI355Q_ERR_INVALID_ARGUMENT, "activation pointer must be 16-byte aligned");
    const uint32_t k_walk = gemm_wide_k(w.k, x_dtype);
    const GemmLaunchShape g = gemm_wide_shape(m, w.n, k_walk);
    // fp32 activations (the reference's prefill type, gemm_q4_g*_f32s): every row becomes [hi | lo], hi = bf16(x) and
    // lo = bf16(x - hi), sixteen bits of each activation, in scratch of the context; the kernel walks 2 K against the
    // weights twice, so the two halves meet in the fp32 accumulators
    const size_t split_bytes = x_dtype == MI355Q_F32 ? (((size_t)m * k_walk * 2 + 255) & ~(size_t)255) : 0;
    const size_t part_bytes = g.splits > 1 ? (size_t)g.splits * m * w.n * sizeof(float) : 0;
    const void* xk = x;
    uint32_t xk_stride = x_stride;
    if (split_bytes) {
        if (mi355q_status st = ensure_split_buffer(ctx, split_bytes)) return st;
        uint16_t* const hi = (uint16_t*)ctx->split_buffer;
        if (mi355q_status st = launch_split_f32_bf16x2(s, (const float*)x, m, w.k, x_stride, hi, hi + w.k, k_walk)) return st;
        xk = hi;
        xk_stride = k_walk;
    }
    WideArgs a{};
    const bool blocks = w.layout == MI355Q_LAYOUT_STAF_BLOCKS;
    a.codes = w.codes; a.sz = w.sz; a.blocks = w.blocks;
    a.row_bytes = w.blocks_per_row * w.bytes_per_block;
    a.x = (const uint16_t*)xk; a.y = y;
    a.m = m; a.n = w.n; a.k = k_walk; a.xs = xk_stride; a.ys = y_stride;
    a.w_fours = w.k / 256;
    a.code_stride = w.code_stride; a.sz_stride = w.sz_stride;
    a.y_dtype = (uint32_t)y_dtype;
    a.wide_stores = (y_stride % 4 == 0 && (uintptr_t)y % 16 == 0) ? 1u : 0u;
    a.line_stores = ((size_t)y_stride * (y_dtype == MI355Q_F32 ? 4 : 2) % 16 == 0 && (uintptr_t)y % 16 == 0) ? 1u : 0u;
    a.probe = probe;
    a.splits = g.splits; a.kt_per_split = g.kt_per_split;
    if (part_bytes) {
        if (mi355q_status st = ensure_workspace(ctx, part_bytes)) return st;
        a.partial = (float*)ctx->workspace;
    }
    const bool sb_bf16 = w.sb_dtype == MI355Q_BF16;
    if (mi355q_status st = x_dtype == MI355Q_F16 ? launch_wide_kernel_f16(s, a, g.bm, w.group, sb_bf16, blocks)
                                                 : launch_wide_kernel_bf16(s, a, g.bm, w.group, sb_bf16, blocks))
        return st;
    if (a.partial) {
        size_t wgs = ((size_t)a.m * a.n / 4 + 255) / 256;
        if (wgs > 16384) wgs = 16384;
        wide_reduce_kernel<<<dim3((unsigned)wgs), dim3(256), 0, s>>>((const wd_float4_v*)a.partial, a.y, a.m, a.n, a.ys, a.splits,
                                                                     a.y_dtype, a.wide_stores);
        MI355Q_HIP(hipGetLastError());
    }
    return MI355Q_OK;
}

// ---- two or three matrices that share the activations ----------------------------------------------------------------
namespace {
struct WideSumArgs {
    const float* partial;      // [splits][m][n_total]
    void* y[3];
    uint32_t ys[3], col_end[3];
    uint32_t m, n_total, splits, y_dtype;
};
// Sum of the K parts in part order, four columns a thread (every matrix is a multiple of four columns wide), each
// matrix's columns to its own result.
__global__ __launch_bounds__(256) void wide_reduce_multi_kernel(WideSumArgs a) {
    const size_t total = (size_t)a.m * a.n_total / 4;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const wd_float4_v* const p = (const wd_float4_v*)a.partial + i;
        wd_float4_v v = __builtin_nontemporal_load(p);
        for (uint32_t s = 1; s < a.splits; s++) v += __builtin_nontemporal_load(p + (size_t)s * total);
        const size_t e = i * 4, row = e / a.n_total;
        const uint32_t pcol = (uint32_t)(e - row * a.n_total);
        const uint32_t sg = pcol >= a.col_end[1] ? 2u : pcol >= a.col_end[0] ? 1u : 0u;
        const uint32_t col = pcol - (sg == 2 ? a.col_end[1] : sg == 1 ? a.col_end[0] : 0u);
        void* const y = sg == 2 ? a.y[2] : sg == 1 ? a.y[1] : a.y[0];
        const size_t o = row * (sg == 2 ? a.ys[2] : sg == 1 ? a.ys[1] : a.ys[0]) + col;
        const float f[4] = {v.x, v.y, v.z, v.w};
        for (int c = 0; c < 4; c++) {
            if (a.y_dtype == MI355Q_F32) ((float*)y)[o + c] = f[c];
            else if (a.y_dtype == MI355Q_BF16) ((uint16_t*)y)[o + c] = f32_to_bf16_rne(f[c]);
            else ((uint16_t*)y)[o + c] = f32_to_f16_rne(f[c]);
        }
    }
}
}  // namespace

bool gemm_wide_multi_eligible(uint32_t count, const WView* w, int x_dtype, uint32_t m, uint32_t x_stride) {
    if (count < 2 || count > 3) return false;
    uint64_t total = 0;
    for (uint32_t i = 0; i < count; i++) {
        if (!gemm_wide_eligible(w[i], x_dtype, m, x_stride)) return false;
        if (w[i].k != w[0].k || w[i].layout != w[0].layout || w[i].group != w[0].group || w[i].bits != w[0].bits ||
            w[i].sb_dtype != w[0].sb_dtype || w[i].code_stride != w[0].code_stride || w[i].sz_stride != w[0].sz_stride ||
            w[i].blocks_per_row != w[0].blocks_per_row || w[i].bytes_per_block != w[0].bytes_per_block)
            return false;
        if (w[i].n % 4 || (i + 1 < count && w[i].n % kWideBN)) return false;     // whole tiles; K parts in 16-byte pieces
        total += w[i].n;
    }
    return total < (1ull << 31);
}

GemmLaunchShape gemm_wide_multi_shape(uint32_t count, const WView* w, uint32_t m, int x_dtype) {
    uint32_t total = 0;
    for (uint32_t i = 0; i < count; i++) total += w[i].n;
    return gemm_wide_shape(m, total, gemm_wide_k(w[0].k, x_dtype));
}

// From the rows where the streamed-weight kernel ends, whatever the size: against a launch per projection (each with
// its own K parts and sum) the one launch took half the time wherever it was measured -- q+k+v 4096 -> 4096 + 1024 +
// 1024 at 97 / 128 / 512 / 2048 rows 26 / 28 / 49 / 94 us against 57 / 58 / 88 / 135, 2048 + 512 + 512 at 97 to 384
// rows 25-32 against 50-64, 1024 + 256 + 256 23-32 against 51-68, two of 256 columns 23-27 against 35-43, gate+up
// 2 x 8192 at 97 to 384 rows 34-63 against 57-111, 2 x 14336 at 128 / 512 rows 50 / 107 against 65 / 131.
bool gemm_wide_multi_chosen(uint32_t count, const WView* w, int x_dtype, uint32_t m, uint32_t x_stride) {
    return gemm_wide_multi_eligible(count, w, x_dtype, m, x_stride) && m >= kWideMinRows;
}

mi355q_status launch_qgemm_wide_multi(hipStream_t s, mi355q_context* ctx, uint32_t count, const WView* w, const void* x,
                                      int x_dtype, void* const* y, const uint32_t* y_strides, int y_dtype, uint32_t m,
                                      uint32_t x_stride) {
    if (!gemm_wide_multi_eligible(count, w, x_dtype, m, x_stride))
        return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the wide-tile MFMA GEMM does not take these weights as one launch");
    if ((uintptr_t)x % 16) return fail(MI355Q_ERR_INVALID_ARGUMENT, "activation pointer must be 16-byte aligned");
    const GemmLaunchShape g = gemm_wide_multi_shape(count, w, m, x_dtype);
    // fp32 activations: every row once as [hi | lo] bf16 halves for all the matrices (as launch_qgemm_wide does for one)
    const uint32_t k_walk = gemm_wide_k(w[0].k, x_dtype);
    const void* xk = x;
    uint32_t xk_stride = x_stride;
    if (x_dtype == MI355Q_F32) {
        if (mi355q_status st = ensure_split_buffer(ctx, ((size_t)m * k_walk * 2 + 255) & ~(size_t)255)) return st;
        uint16_t* const hi = (uint16_t*)ctx->split_buffer;
        if (mi355q_status st = launch_split_f32_bf16x2(s, (const float*)x, m, w[0].k, x_stride, hi, hi + w[0].k, k_walk)) return st;
        xk = hi;
        xk_stride = k_walk;
    }
    WideArgs a{};
    const bool blocks = w[0].layout == MI355Q_LAYOUT_STAF_BLOCKS;
    const size_t esz = y_dtype == MI355Q_F32 ? 4 : 2;
    a.codes = w[0].codes; a.sz = w[0].sz; a.blocks = w[0].blocks;
    a.y = y[0]; a.n = w[0].n; a.ys = y_strides[0];
    a.segments = count;
    a.wide_stores = 1; a.line_stores = 1;
    uint32_t tiles = 0, cols = 0;
    WideSumArgs sum{};
    for (uint32_t i = 0; i < count; i++) {
        if (i) {
            a.seg_tile0[i - 1] = tiles; a.seg_col0[i - 1] = cols;
            a.seg_codes[i - 1] = w[i].codes; a.seg_sz[i - 1] = w[i].sz; a.seg_blocks[i - 1] = w[i].blocks;
            a.seg_y[i - 1] = y[i]; a.seg_n[i - 1] = w[i].n; a.seg_ys[i - 1] = y_strides[i];
        }
        tiles += (w[i].n + kWideBN - 1) / kWideBN;
        cols += w[i].n;
        sum.y[i] = y[i]; sum.ys[i] = y_strides[i]; sum.col_end[i] = cols;
        if (y_strides[i] % 4 || (uintptr_t)y[i] % 16) a.wide_stores = 0;
        if ((size_t)y_strides[i] * esz % 16 || (uintptr_t)y[i] % 16) a.line_stores = 0;
    }
    if (count == 2) {                                  // no third matrix: nothing reaches it
        a.seg_tile0[1] = 0xFFFFFFFFu;
        sum.y[2] = y[1]; sum.ys[2] = y_strides[1]; sum.col_end[1] = 0xFFFFFFFFu; sum.col_end[2] = 0xFFFFFFFFu;
    }
    a.tiles_n = tiles;
    a.n_total = cols;
    a.row_bytes = w[0].blocks_per_row * w[0].bytes_per_block;
    a.x = (const uint16_t*)xk;
    a.m = m; a.k = k_walk; a.xs = xk_stride;
    a.w_fours = w[0].k / 256;
    a.code_stride = w[0].code_stride; a.sz_stride = w[0].sz_stride;
    a.y_dtype = (uint32_t)y_dtype;
    a.splits = g.splits; a.kt_per_split = g.kt_per_split;
    if (g.splits > 1) {
        if (mi355q_status st = ensure_workspace(ctx, (size_t)g.splits * m * cols * sizeof(float))) return st;
        a.partial = (float*)ctx->workspace;
    }
    const bool sb_bf16 = w[0].sb_dtype == MI355Q_BF16;
    if (mi355q_status st = x_dtype == MI355Q_F16 ? launch_wide_kernel_f16(s, a, g.bm, w[0].group, sb_bf16, blocks)
                                                 : launch_wide_kernel_bf16(s, a, g.bm, w[0].group, sb_bf16, blocks))
        return st;
    if (a.partial) {
        sum.partial = a.partial; sum.m = m; sum.n_total = cols; sum.splits = g.splits; sum.y_dtype = (uint32_t)y_dtype;
        size_t wgs = ((size_t)m * cols / 4 + 255) / 256;
        if (wgs > 16384) wgs = 16384;
        wide_reduce_multi_kernel<<<dim3((unsigned)wgs), dim3(256), 0, s>>>(sum);
        MI355Q_HIP(hipGetLastError());
    }
    return MI355Q_OK;
}

// ---- gated MLP projection ------------------------------------------------------------------------------------------
bool gemm_wide_gated_eligible(const WView& gate, const WView& up, int x_dtype, uint32_t m, uint32_t x_stride) {
    if (x_dtype != MI355Q_BF16 && x_dtype != MI355Q_F16) return false;
    if (!gemm_wide_eligible(gate, x_dtype, m, x_stride) || !gemm_wide_eligible(up, x_dtype, m, x_stride)) return false;
    return gate.n == up.n && gate.k == up.k && gate.layout == up.layout && gate.group == up.group && gate.bits == up.bits &&
           gate.sb_dtype == up.sb_dtype && gate.code_stride == up.code_stride && gate.sz_stride == up.sz_stride &&
           gate.blocks_per_row == up.blocks_per_row && gate.bytes_per_block == up.bytes_per_block;
}

bool gemm_wide_gated_chosen(const WView& gate, const WView& up, int x_dtype, uint32_t m, uint32_t x_stride) {
    if (!gemm_wide_gated_eligible(gate, up, x_dtype, m, x_stride) || m < kWideMinRows) return false;
    const GemmLaunchShape g = gemm_wide_shape(m, 2 * gate.n, gate.k, true);
    const uint32_t wgs = ((m + g.bm - 1) / g.bm) * ((gate.n + kWideBN / 2 - 1) / (kWideBN / 2));
    // K stays in one part (a partial sum cannot be gated), so the tiles alone must fill the chip.  The activation costs
    // the matrix-core wavefronts about 5 us a round of tiles (two roundings, a 2^x and a reciprocal per output), the
    // elementwise launch it replaces 65 us at 2048 rows of 14336: 4096 -> 2 x 14336 at 256 rows 66 us against 100 for
    // the two projections and the elementwise launch, at 512 rows 108 against 144, at 1024 rows 209 against 236, at
    // 2048 rows 422 against 463.  (With exp and an IEEE division in the activation, 10 us a round, the one launch won
    // only up to two rounds of tiles: 484 against 475 at 2048 rows.)
    // One row of 128-row tiles (97 to 128 rows): from a quarter of the CUs, where the projections apart split K and
    // add their parts (128 rows of 4096 -> 2 x N: N = 6144, 48 workgroups, 59 us either way; 8192 59 against 62;
    // 11008 60 against 63; 14336 60 against 69).
    const uint32_t eighths = g.bm == 128 && m <= 128 ? 2 : 5;
    return 8 * wgs >= eighths * chip_cus();
}

bool gemm_wide_gated_taken(const mi355q_context* ctx, const WView& gate, const WView& up, int x_dtype, uint32_t m, uint32_t x_stride,
                           uint32_t flags) {
    if (flags & MI355Q_FLAG_PROBE_WIDE) return gemm_wide_gated_eligible(gate, up, x_dtype, m, x_stride);
    if (flags & (MI355Q_FLAG_FORCE_GENERIC | MI355Q_FLAG_FORCE_SMALL_M | MI355Q_FLAG_FORCE_MFMA | MI355Q_FLAG_FORCE_TWO_STEP |
                 MI355Q_FLAG_FORCE_STREAM))
        return false;
    return gemm_wide_gated_chosen(gate, up, x_dtype, m, x_stride) && (m < kWideRowsBesideLibrary || library_ruled_out(ctx));
}

mi355q_status launch_qgemm_wide_gated(hipStream_t s, mi355q_context* ctx, const WView& gate, const WView& up, const void* x,
                                      int x_dtype, void* y, int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride,
                                      int activation) {
    (void)ctx;
    if (!gemm_wide_gated_eligible(gate, up, x_dtype, m, x_stride))
        return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the wide-tile MFMA GEMM does not take this pair of weights as a gated projection");
    if ((uintptr_t)x % 16) return fail(MI355Q_ERR_INVALID_ARGUMENT, "activation pointer must be 16-byte aligned");
    const GemmLaunchShape g = gemm_wide_shape(m, 2 * gate.n, gate.k, true);
    WideArgs a{};
    const bool blocks = gate.layout == MI355Q_LAYOUT_STAF_BLOCKS;
    a.codes = gate.codes; a.sz = gate.sz; a.blocks = gate.blocks;
    a.codes_up = up.codes; a.sz_up = up.sz; a.blocks_up = up.blocks;
    a.gated = 1u + (uint32_t)activation;
    a.row_bytes = gate.blocks_per_row * gate.bytes_per_block;
    a.x = (const uint16_t*)x; a.y = y;
    a.m = m; a.n = gate.n; a.k = gate.k; a.xs = x_stride; a.ys = y_stride;
    a.w_fours = gate.k / 256;
    a.code_stride = gate.code_stride; a.sz_stride = gate.sz_stride;
    a.y_dtype = (uint32_t)y_dtype;
    a.line_stores = ((size_t)y_stride * (y_dtype == MI355Q_F32 ? 4 : 2) % 16 == 0 && (uintptr_t)y % 16 == 0) ? 1u : 0u;
    a.splits = 1; a.kt_per_split = gate.k / 64;
    const bool sb_bf16 = gate.sb_dtype == MI355Q_BF16;
    return x_dtype == MI355Q_F16 ? launch_wide_kernel_f16(s, a, g.bm, gate.group, sb_bf16, blocks)
                                 : launch_wide_kernel_bf16(s, a, g.bm, gate.group, sb_bf16, blocks);
}

}  // namespace mi355q
