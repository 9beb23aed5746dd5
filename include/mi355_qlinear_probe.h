/* Measurement aids of libmi355_qlinear: entry points without a counterpart in the reference, used by the
 * benchmark and the profiles to price the kernels against the part itself.  They are exported by the same
 * shared library but declared apart from mi355_qlinear.h on purpose: a host binding of the quantized
 * projection path (the Swift module map, a ctypes or cgo stub) includes only mi355_qlinear.h and never sees
 * them. */
#ifndef MI355_QLINEAR_PROBE_H
#define MI355_QLINEAR_PROBE_H

#include "mi355_qlinear.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Launch flag for mi355q_qgemm (its `flags` argument, beside the MI355Q_FLAG_* values of mi355_qlinear.h): on
 * the matrix-core kernel, the first wavefront of workgroup 0 records how long it was in the kernel. */
enum { MI355Q_FLAG_PROBE_CLOCK = 8 };
/* Launch flag for mi355q_qgemm and mi355q_plan_prefill_steps: where the fused matrix-core route would take the wide-tile
 * kernel (long prompts on 4-bit planes), keep the tiled kernel that dequantises into LDS (A/B runs). */
enum { MI355Q_FLAG_PROBE_TILED = 64 };
/* ... and the other way round: the wide-tile kernel wherever it reads the weight, whatever the size (tests of small shapes). */
enum { MI355Q_FLAG_PROBE_WIDE = 128 };

/* After an mi355q_qgemm call with MI355Q_FLAG_PROBE_CLOCK that ran on the matrix cores has completed, returns
 * what that wavefront counted: shader-clock cycles and ticks of the constant 100 MHz counter.
 * cycles / ticks / 10 is the clock in GHz the kernel ran at (it depends on the operand data: the part lowers
 * its clock under matrix-core load).  Synchronises with the device. */
MI355Q_API mi355q_status mi355q_clock_probe_read(mi355q_context* ctx, uint64_t* shader_cycles,
                                                 uint64_t* realtime_ticks);

/* One launch that only reads `bytes` of device memory with the load instructions the decode kernels use for
 * weights.  Its duration is what HBM delivers to a launch of that size on this part: the practical ceiling the
 * decode GEMV is compared with.  16-byte aligned pointer and size. */
MI355Q_API mi355q_status mi355q_buffer_read_probe(mi355q_context* ctx, void* stream, const void* src_dev,
                                                  size_t bytes);

/* Bytes of device scratch the context holds right now: [0] fp32 partial results / dense copies, [1] split activation
 * rows, [2] gate and up sums of the gated projection.  A test of an entry point that must not allocate compares them
 * before and after the call. */
MI355Q_API mi355q_status mi355q_context_scratch_bytes(mi355q_context* ctx, uint64_t out_bytes[3]);

/* A/B runs of the wide-tile prefill kernel: tile height (128 or 256 rows) and the number of parts K is split into
 * (1 .. 4), for every later launch of the process; 0 leaves the choice to the library.  Values that do not fit a
 * problem (fewer than sixteen K-tiles a part, N not a multiple of four) are ignored for it. */
MI355Q_API void mi355q_probe_wide_shape(uint32_t tile_rows, uint32_t k_parts);

/* The route table on a synthetic weight (no device needed): what the launcher would run for the problem
 * ("route" or "route/kernel": split-rows, two-step, stream, small-batch/<kernel>, fused/wide, fused/tiled, error:...)
 * and the device kernels the plan records name for it, joined by '+'.  Launcher and planner read the same table; the
 * CPU test suite walks it.  layout: mi355q_layout; sb_dtype: scale type of planes; library_available: whether the
 * dense library counts as usable; decode_entry: mi355q_qgemv / plan_decode_step, else mi355q_qgemm / plan_prefill_steps. */
MI355Q_API mi355q_status mi355q_probe_route(uint8_t scheme_identifier, uint32_t layout, uint32_t sb_dtype, uint64_t n_rows,
                                            uint64_t k, mi355q_dtype x_dtype, uint32_t m, uint32_t x_row_stride,
                                            uint32_t flags, int decode_entry, int library_available, char* launcher_out,
                                            char* planner_out, size_t cap);

/* The same for two or three projections that share their activations (mi355q_batched_qgemm, the shared steps of a plan):
 * what the launcher would run ("shared/<kernel>" for one launch over the rows of all matrices, "split-rows", "steps",
 * "separate") and the device kernel the plan record of that step names. */
MI355Q_API mi355q_status mi355q_probe_shared_route(uint8_t scheme_identifier, uint32_t layout, uint32_t sb_dtype, uint32_t count,
                                                   const uint64_t* n_rows, uint64_t k, mi355q_dtype x_dtype, uint32_t m,
                                                   uint32_t x_row_stride, uint32_t flags, char* launcher_out,
                                                   char* planner_out, size_t cap);

#ifdef __cplusplus
}
#endif
#endif
