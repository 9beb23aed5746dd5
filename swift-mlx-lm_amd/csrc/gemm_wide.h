// Shared by gemm_wide.hip (choice of shape, launch, sum of K parts) and the two instantiation units of the kernel
// (gemm_wide_bf16.hip, gemm_wide_f16.hip; kernel text in gemm_wide.inl).
#pragma once
#include "common.h"

namespace mi355q {

struct WideArgs {
    const uint32_t* codes;       // planes: [N, K / 8] words, rows code_stride words apart
    const uint32_t* sz;          // planes: (scale | bias << 16) per group, rows sz_stride words apart
    const uint8_t* blocks;       // blocks in place: [f16 scale][f16 zero][codes] per group, rows row_bytes apart
    const uint16_t* x;           // bf16 or f16 [M, xs]
    void* y;
    uint32_t m, n, k, xs, ys;
    uint32_t code_stride, sz_stride, row_bytes;
    uint32_t tiles_m, tiles_n;
    uint32_t y_dtype;
    uint32_t wide_stores;        // rows of y are 16-byte aligned for every column that is a multiple of four
    uint32_t line_stores;        // rows of y are 16-byte aligned at every tile's first column: whole lines through LDS
    float* partial;              // K split over workgroups: fp32 [splits][M][N] partial results (null otherwise)
    uint32_t splits, kt_per_split;   // K-tiles per split: a multiple of four
    uint32_t w_fours;                // groups of four K-tiles in a weight row: the walk over K wraps there (fp32 activations
                                     // come as [hi | lo] rows of 2 K bf16 values against the same weights twice)
    // gated MLP projection (0: none; else 1 + mi355q_gated_activation): the second fragment of every wavefront reads
    // up_proj where the first reads gate_proj (codes / sz / blocks above), a tile is 128 output columns wide, tiles_n
    // counts those, and y receives activation(gate) * up; no K parts
    uint32_t gated;
    const uint32_t* codes_up;
    const uint32_t* sz_up;
    const uint8_t* blocks_up;
    // two or three matrices that share the activations (q+k+v, gate+up) as one launch: `segments` > 1, the column tiles
    // [0, seg_tile0[0]) belong to the matrix above, [seg_tile0[0], seg_tile0[1]) to seg_*[0], the rest to seg_*[1] (two
    // matrices: seg_tile0[1] = tiles_n); every matrix but the last is a whole number of 256-column tiles; tiles_n is
    // given; K parts land at column seg_col0 of fp32 rows of n_total columns
    uint32_t segments;
    uint32_t seg_tile0[2], seg_n[2], seg_ys[2], seg_col0[2], n_total;
    const uint32_t* seg_codes[2];
    const uint32_t* seg_sz[2];
    const uint8_t* seg_blocks[2];
    void* seg_y[2];
    unsigned long long* probe;   // optional: [0] shader cycles, [1] 100 MHz ticks that workgroup 0 spent in the kernel
};

constexpr int kWideStages = 4;   // LDS stages of activations
constexpr int kWideBN = 256;

// the kernel launch alone (tiles_m, tiles_n filled in here); activations bf16 / f16
mi355q_status launch_wide_kernel_bf16(hipStream_t s, WideArgs a, uint32_t bm, uint32_t group, bool sb_bf16, bool blocks);
mi355q_status launch_wide_kernel_f16(hipStream_t s, WideArgs a, uint32_t bm, uint32_t group, bool sb_bf16, bool blocks);

}  // namespace mi355q
