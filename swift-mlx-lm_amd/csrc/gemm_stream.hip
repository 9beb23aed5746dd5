// Host side of the streamed-weight matrix-core kernel (gemm_stream.inl): eligibility, launch shape, the shared launch of two
// or three matrices, the sum of the K parts.
#include "device_utils.h"
#include "gemm_stream.h"

namespace mi355q {

// y_i = the sum of the K parts' fp32 partial results over matrix i's columns, part 0 first, rounded once to the output type
__global__ __launch_bounds__(256) void stream_sum_parts_kernel(StreamArgs a, uint32_t parts) {
    const size_t total = (size_t)a.m * a.n_total;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        float v = 0.f;
        for (uint32_t p = 0; p < parts; p++) v += a.partial[(size_t)p * total + i];
        const size_t row = i / a.n_total;
        const uint32_t pcol = (uint32_t)(i - row * a.n_total);
        const bool in1 = pcol >= a.col0[1], in2 = pcol >= a.col0[2];
        void* const y = in2 ? a.y[2] : in1 ? a.y[1] : a.y[0];
        const size_t o = row * (in2 ? a.ys[2] : in1 ? a.ys[1] : a.ys[0]) + (pcol - (in2 ? a.col0[2] : in1 ? a.col0[1] : 0u));
        if (a.y_dtype == MI355Q_F32) ((float*)y)[o] = v;
        else if (a.y_dtype == MI355Q_BF16) ((uint16_t*)y)[o] = f32_to_bf16_rne(v);
        else ((uint16_t*)y)[o] = f32_to_f16_rne(v);
    }
}

bool gemm_stream_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride) {
    if ((x_dtype != MI355Q_BF16 && x_dtype != MI355Q_F16) || m < 1 || m > kStreamMaxRows) return false;
    if (w.layout == MI355Q_LAYOUT_STAF_BLOCKS) {
        if (!w.blocks || (uintptr_t)w.blocks % 4 || w.bytes_per_block != 4 + w.group * w.bits / 8) return false;
    } else if (w.layout != MI355Q_LAYOUT_PLANES || !w.sz || !w.codes) {
        return false;
    }
    if (!((w.bits == 4 && (w.group == 64 || w.group == 128)) ||
          (w.bits == 8 && (w.group == 32 || w.group == 64 || w.group == 128)) ||
          ((w.bits == 2 || w.bits == 3 || w.bits == 5 || w.bits == 6) && w.group == 64)))
        return false;
    if (w.k % 64 || w.k < 64 || x_stride % 8) return false;
    // 4- and 8-bit planes are read with 16-byte loads; the other widths word by word
    if (w.layout == MI355Q_LAYOUT_PLANES && (w.bits == 4 || w.bits == 8) && ((uintptr_t)w.codes % 16 || w.code_stride % 4)) return false;
    return true;
}

bool gemm_stream_unrounded(const WView& w, uint32_t m) { return m <= 32 && w.group % 64 == 0; }

StreamLaunchShape gemm_stream_shape(const mi355q_context* ctx, uint32_t m, uint32_t n, uint32_t k) {
    return gemm_stream_shape_blocks(ctx, m, (n + kStreamRows - 1) / kStreamRows, k);
}

StreamLaunchShape gemm_stream_shape_blocks(const mi355q_context* ctx, uint32_t m, uint32_t row_blocks, uint32_t k) {
    StreamLaunchShape g{};
    const uint32_t cus = (uint32_t)ctx->props.multiProcessorCount;
    g.row_blocks = row_blocks;
    const uint32_t it_all = (k + kStreamIterK - 1) / kStreamIterK;
    // K parts while the row blocks alone leave half the CUs idle and a part keeps four iterations
    uint32_t parts = 1;
    while (g.row_blocks * parts * 2 <= cus && it_all / (parts * 2) >= 4) parts *= 2;
    g.iters_per_part = (it_all + parts - 1) / parts;
    g.parts = (it_all + g.iters_per_part - 1) / g.iters_per_part;
    g.m_blocks = (m + 31) / 32;
    g.lds_bytes = 3u * 4u * g.m_blocks * 32u * 128u;       // three stages of [32 m_blocks][256] bf16
    return g;
}


namespace {
// the instantiation unit of the code width
mi355q_status launch_stream_width(hipStream_t s, const StreamArgs& a, const StreamLaunchShape& g, const WView& w, int x_dtype) {
    const bool bf = w.sb_dtype == MI355Q_BF16, xf = x_dtype == MI355Q_F16, bl = w.layout == MI355Q_LAYOUT_STAF_BLOCKS;
    switch (w.bits) {
    case 2: return launch_stream_q2(s, a, g, w.group, bf, xf, bl);
    case 3: return launch_stream_q3(s, a, g, w.group, bf, xf, bl);
    case 4: return launch_stream_q4(s, a, g, w.group, bf, xf, bl);
    case 5: return launch_stream_q5(s, a, g, w.group, bf, xf, bl);
    case 6: return launch_stream_q6(s, a, g, w.group, bf, xf, bl);
    case 8: return launch_stream_q8(s, a, g, w.group, bf, xf, bl);
    default: break;
    }
    return MI355Q_ERR_KERNEL_NOT_FOUND;
}
}  // namespace

mi355q_status launch_qgemm_stream(hipStream_t s, mi355q_context* ctx, const WView& w, const void* x, int x_dtype, void* y,
                                  int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride) {
    void* ys[1] = {y};
    const uint32_t strides[1] = {y_stride};
    return launch_qgemm_stream_multi(s, ctx, 1, &w, x, x_dtype, ys, strides, y_dtype, m, x_stride);
}

bool gemm_stream_multi_eligible(uint32_t count, const WView* w, int x_dtype, uint32_t m, uint32_t x_stride) {
    if (count < 1 || count > (uint32_t)kStreamMaxSegments) return false;
    for (uint32_t i = 0; i < count; i++)
        if (!gemm_stream_eligible(w[i], x_dtype, m, x_stride) || w[i].k != w[0].k || w[i].group != w[0].group ||
            w[i].bits != w[0].bits || w[i].sb_dtype != w[0].sb_dtype || w[i].layout != w[0].layout)
            return false;
    return true;
}

mi355q_status launch_qgemm_stream_multi(hipStream_t s, mi355q_context* ctx, uint32_t count, const WView* w, const void* x,
                                        int x_dtype, void* const* y, const uint32_t* y_strides, int y_dtype, uint32_t m,
                                        uint32_t x_stride) {
    if (!gemm_stream_multi_eligible(count, w, x_dtype, m, x_stride))
        return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the streamed-weight kernel does not take these weights or activations");
    if ((uintptr_t)x % 16) return fail(MI355Q_ERR_INVALID_ARGUMENT, "activation pointer must be 16-byte aligned");
    StreamArgs a{};
    uint32_t blocks = 0, cols = 0;
    for (uint32_t i = 0; i < (uint32_t)kStreamMaxSegments; i++) {
        const uint32_t j = i < count ? i : count - 1;          // unused entries repeat the last matrix and own nothing
        a.codes[i] = w[j].codes; a.sz[i] = w[j].sz; a.blocks[i] = w[j].blocks; a.y[i] = y[j];
        a.n[i] = w[j].n; a.ys[i] = y_strides[j];
        a.code_stride[i] = w[j].code_stride; a.sz_stride[i] = w[j].sz_stride;
        if (i < count) {
            a.col0[i] = cols;
            blocks += (w[i].n + kStreamRows - 1) / kStreamRows;
            cols += w[i].n;
            a.wg_end[i] = blocks;
        } else {
            a.col0[i] = 0xFFFFFFFFu;                           // no column and no workgroup reaches an unused entry
            a.wg_end[i] = 0xFFFFFFFFu;
        }
    }
    a.row_bytes = (uint64_t)w[0].blocks_per_row * w[0].bytes_per_block;
    a.x = (const uint16_t*)x;
    a.m = m; a.k = w[0].k; a.xs = x_stride; a.n_total = cols;
    a.y_dtype = (uint32_t)y_dtype;
    const StreamLaunchShape g = gemm_stream_shape_blocks(ctx, m, blocks, w[0].k);
    a.iters_per_part = g.iters_per_part;
    // unrounded weights wherever the variant exists: 0.3 to 1 us of a 15 to 23 us launch (4096 -> 14336 q4 g64 at 32
    // rows 16.9 against 16.5 us), rel-L2 1.3e-7 instead of 1.7e-3 (bf16 weights) or 1.9e-4 (f16 weights)
    a.exact = gemm_stream_unrounded(w[0], m);
    if (g.parts > 1) {
        if (mi355q_status st = ensure_workspace(ctx, (size_t)g.parts * m * cols * sizeof(float))) return st;
        a.partial = (float*)ctx->workspace;
    }
    const mi355q_status st = launch_stream_width(s, a, g, w[0], x_dtype);
    if (st != MI355Q_OK || g.parts == 1) return st;
    const size_t total = (size_t)m * cols;
    size_t sum_blocks = (total + 255) / 256;
    if (sum_blocks > 4096) sum_blocks = 4096;
    stream_sum_parts_kernel<<<dim3((unsigned)sum_blocks), dim3(256), 0, s>>>(a, g.parts);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

// ---- gated MLP projection ------------------------------------------------------------------------------------------
StreamLaunchShape gemm_stream_gated_shape(const mi355q_context* ctx, uint32_t m, uint32_t n, uint32_t k) {
    return gemm_stream_shape_blocks(ctx, m, (n + 31) / 32, k);
}

bool gemm_stream_gated_taken(const mi355q_context* ctx, const WView& gate, const WView& up, int x_dtype, uint32_t m,
                             uint32_t x_stride, uint32_t flags) {
    if (gate.n != up.n) return false;
    const WView both[2] = {gate, up};
    if (shared_route(ctx, 2, both, x_dtype, m, x_stride, flags, true) != SharedRoute::kStream) return false;
    if (flags & MI355Q_FLAG_FORCE_STREAM) return true;
    return gemm_stream_gated_shape(ctx, m, gate.n, gate.k).parts == 1;      // a partial sum cannot be gated
}

mi355q_status launch_qgemm_stream_gated(hipStream_t s, mi355q_context* ctx, const WView& gate, const WView& up, const void* x,
                                        int x_dtype, void* y, int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride,
                                        int activation) {
    const WView w[2] = {gate, up};
    if (gate.n != up.n || !gemm_stream_multi_eligible(2, w, x_dtype, m, x_stride))
        return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the streamed-weight kernel does not take this pair of weights as a gated projection");
    if ((uintptr_t)x % 16) return fail(MI355Q_ERR_INVALID_ARGUMENT, "activation pointer must be 16-byte aligned");
    StreamArgs a{};
    for (uint32_t i = 0; i < (uint32_t)kStreamMaxSegments; i++) {
        const uint32_t j = i < 2 ? i : 1;
        a.codes[i] = w[j].codes; a.sz[i] = w[j].sz; a.blocks[i] = w[j].blocks; a.y[i] = y;
        a.n[i] = w[j].n; a.ys[i] = y_stride;
        a.code_stride[i] = w[j].code_stride; a.sz_stride[i] = w[j].sz_stride;
        a.col0[i] = 0xFFFFFFFFu; a.wg_end[i] = 0xFFFFFFFFu;     // (not read: a workgroup's row blocks name the matrices)
    }
    a.row_bytes = (uint64_t)gate.blocks_per_row * gate.bytes_per_block;
    a.x = (const uint16_t*)x;
    a.m = m; a.k = gate.k; a.xs = x_stride; a.n_total = gate.n;
    a.y_dtype = (uint32_t)y_dtype;
    a.gated = 1u + (uint32_t)activation;
    StreamLaunchShape g = gemm_stream_gated_shape(ctx, m, gate.n, gate.k);
    g.parts = 1;
    g.iters_per_part = (gate.k + kStreamIterK - 1) / kStreamIterK;
    a.iters_per_part = g.iters_per_part;
    a.exact = gemm_stream_unrounded(gate, m);
    return launch_stream_width(s, a, g, gate, x_dtype);
}

}  // namespace mi355q
