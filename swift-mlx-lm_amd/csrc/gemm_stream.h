// Arguments and launch entry points of the streamed-weight matrix-core kernel (gemm_stream.inl), shared by the per-width
// translation units and the host side (gemm_stream.hip).
#pragma once

#include "common.h"

namespace mi355q {

constexpr int kStreamMaxSegments = 3;

struct StreamArgs {
    // up to three matrices that share the activations, K, the group size and the scale type (q+k+v, gate+up): matrix i
    // owns the workgroups [wg_end[i-1], wg_end[i]) and the columns [col0[i], col0[i] + n[i]) of the fp32 partial results
    const uint32_t* codes[kStreamMaxSegments];     // [N][code_stride] words, eight codes a word
    const uint32_t* sz[kStreamMaxSegments];        // [N][sz_stride] words: scale | bias << 16 per group
    void* y[kStreamMaxSegments];
    uint32_t n[kStreamMaxSegments], ys[kStreamMaxSegments];
    uint32_t code_stride[kStreamMaxSegments], sz_stride[kStreamMaxSegments];
    const uint8_t* blocks[kStreamMaxSegments];     // block layout: [N][row_bytes], a block = (scale f16, zero f16, codes)
    uint64_t row_bytes;                            // block layout: bytes from one row to the next
    uint32_t wg_end[kStreamMaxSegments], col0[kStreamMaxSegments];
    const uint16_t* x;         // bf16 [M][xs]
    float* partial;            // K split over workgroups: fp32 [parts][M][n_total]; else null
    uint32_t m, k, xs, n_total;
    uint32_t y_dtype;
    uint32_t iters_per_part;   // iterations (256 columns each) per K part; blockIdx.y is the part
    uint32_t exact;            // host side: the variant with unrounded weights (at most 32 rows, groups of 64 or 128)
    // gated MLP projection (0: none; else 1 + mi355q_gated_activation): matrix 0 is gate_proj, matrix 1 up_proj, a
    // workgroup owns rows 32 blockIdx.x .. + 31 of both (its two row blocks) and y[0] receives activation(gate) * up;
    // K in one part
    uint32_t gated;
};

constexpr int kStreamIterK = 256;      // columns of K per iteration: one 64-code K-tile per K slice
constexpr int kStreamRows = 64;        // weight rows per workgroup

// One translation unit per bit width instantiates the kernel (gemm_stream_q{2,3,4,5,6,8}.hip).
#define MI355Q_STREAM_LAUNCH(BITS)                                                                                          \
    mi355q_status launch_stream_q##BITS(hipStream_t s, const StreamArgs& a, const StreamLaunchShape& g, uint32_t group, \
                                        bool sb_bf16, bool x_f16, bool blocks)
MI355Q_STREAM_LAUNCH(2);
MI355Q_STREAM_LAUNCH(3);
MI355Q_STREAM_LAUNCH(4);
MI355Q_STREAM_LAUNCH(5);
MI355Q_STREAM_LAUNCH(6);
MI355Q_STREAM_LAUNCH(8);

}  // namespace mi355q
