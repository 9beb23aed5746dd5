// Internal declarations shared by the translation units of libmi355_qlinear.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>

#include "../../include/mi355_qlinear.h"
#include "../../include/mi355_qlinear_probe.h"

namespace mi355q {

// ---- error plumbing ------------------------------------------------------------------------
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
mi355q_status fail(mi355q_status code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define MI355Q_HIP(call)                                                                       \
    do {                                                                                       \
        hipError_t _e = (call);                                                                \
        if (_e != hipSuccess)                                                                  \
            return ::mi355q::fail(_e == hipErrorOutOfMemory ? MI355Q_ERR_OUT_OF_MEMORY         \
                                                            : MI355Q_ERR_DEVICE,               \
                                  "%s failed: %s", #call, hipGetErrorString(_e));              \
    } while (0)

// ---- format registry (formats.cpp) ---------------------------------------------------------
const mi355q_format* find_format_mlx(int bits, int group);
const mi355q_format* find_format_scheme(uint8_t scheme);
int format_count();
const mi355q_format* format_at(int i);

// ---- device-side view of one packed weight -------------------------------------------------
struct WView {
    const uint8_t* blocks;    // STAF interleaved blocks (layout 0)
    const uint32_t* codes;    // planes (layout 1)
    const uint16_t* scales;
    const uint16_t* biases;
    const uint32_t* sz;       // planes: scale | bias << 16 per group (packed once at prepare time)
    const uint32_t* tiles;    // TILE16 records (layout 2)
    uint32_t n, k;
    uint32_t group, bits;
    uint32_t bytes_per_block, blocks_per_row, words_per_row;
    uint32_t code_stride;     // planes: 32-bit words from one row of codes to the next (>= words_per_row)
    uint32_t sz_stride;       // planes: 32-bit words from one row of sz to the next (>= blocks_per_row)
    uint32_t layout;          // mi355q_layout
    uint32_t sb_dtype;        // mi355q_dtype of scale/bias (F16 for STAF)
};

}  // namespace mi355q

namespace mi355q { struct DenseLibrary; }

struct mi355q_context {
    int device;
    hipDeviceProp_t props;
    // small cells: [16..17] clock probe of the prefill GEMM, [24] sink of the read-only probe launch
    unsigned long long* argmax_scratch;
    // fused output head: one packed (ordered value, ~row) key per workgroup of the projection launch
    // (kArgmaxPartialCapacity entries), then kArgmaxStandaloneKeys entries for the stand-alone argmax
    unsigned long long* argmax_partials;
    // fp32 partial results (split-K of the prefill GEMM, K parts of the tile kernel): grown on demand, never shrunk;
    // outgrown buffers are kept until the context goes, because captured graphs hold their addresses
    void* workspace;
    size_t workspace_bytes;
    void* retired[96];                 // shared by the three scratch buffers: each at most doubles ~30 times
    int retired_count;
    // fp32 activations split into bf16 rows, and the partial projections of those rows (the decode kernels that run on
    // them may use `workspace` themselves); grown and retired like `workspace`
    void* split_buffer;
    size_t split_bytes;
    // gate and up sums of the gated projection where they do not stay in registers (its own buffer: the projections
    // that fill it may use the other two)
    void* gated_buffer;
    size_t gated_bytes;
    // the platform's dense GEMM library (second half of the two-dispatch prefill route), opened on first use
    mi355q::DenseLibrary* dense_library;
    bool dense_library_failed;
    bool dense_library_forbidden;      // mi355q_context_set_library_use(ctx, 0): in-tree kernels only
    // One stream per context at a time: the stream whose launches last used the scratch above, an event that is
    // recorded behind them when another stream turns up (or when that stream is destroyed through this library:
    // scratch_marked), and whether the entry point now running has touched the scratch (see ScratchGuard)
    hipStream_t scratch_stream;
    hipEvent_t scratch_event;
    bool scratch_pending, scratch_touched, scratch_marked;
};
constexpr int kRetiredWorkspaces = 96;

struct mi355q_weight {
    mi355q_context* ctx;
    mi355q_format fmt;
    uint64_t n, k;
    uint8_t layout, sb_dtype, owns;
    void* blocks;
    void* codes;
    void* scales;
    void* biases;
    void* sz;                 // packed (scale, bias) words for the planes layout
    void* tiles;              // owned: TILE16 records (layout 2)
    size_t tiles_bytes;
    // Owned plane weights keep each row's code words and its sz words side by side in ONE buffer
    // ([codes of row r | sz of row r | pad to 16 bytes]): `codes` points at it, `sz` points
    // words_per_row further, and both advance by the same stride, so a row is one contiguous
    // stream in memory.  Borrowed planes (wrap) keep the caller's codes and an owned sz plane.
    uint32_t code_stride, sz_stride;   // in 32-bit words
    uint8_t sz_separate;               // sz is an allocation of its own (borrowed planes)
    size_t blocks_bytes, codes_bytes, sb_bytes;
    mi355q::WView view() const {
        mi355q::WView v;
        v.blocks = (const uint8_t*)blocks;
        v.codes = (const uint32_t*)codes;
        v.scales = (const uint16_t*)scales;
        v.biases = (const uint16_t*)biases;
        v.sz = (const uint32_t*)sz;
        v.tiles = (const uint32_t*)tiles;
        v.n = (uint32_t)n;
        v.k = (uint32_t)k;
        v.group = fmt.group_size;
        v.bits = fmt.bits;
        v.bytes_per_block = fmt.bytes_per_block;
        v.blocks_per_row = (uint32_t)(k / fmt.group_size);
        v.words_per_row = (uint32_t)(k * fmt.bits / 32);
        v.code_stride = code_stride;
        v.sz_stride = sz_stride;
        v.layout = layout;
        v.sb_dtype = sb_dtype;
        return v;
    }
};

namespace mi355q {

// ---- launchers implemented in the kernel translation units ---------------------------------
// Each returns MI355Q_OK or a launch-time failure; all shape checks happen in api.hip before.
mi355q_status launch_unpack_codes(hipStream_t s, const WView& w, uint8_t* out);
mi355q_status launch_dequant_bf16(hipStream_t s, const WView& w, uint16_t* out);
mi355q_status launch_dequant_f32(hipStream_t s, const WView& w, float* out);
mi355q_status launch_dequant_f16(hipStream_t s, const WView& w, uint16_t* out);
mi355q_status launch_split_rows_bf16(hipStream_t s, const void* x, int x_dtype, uint32_t m, uint32_t k, uint32_t x_stride,
                                     uint16_t* out, uint32_t out_stride);
mi355q_status launch_sum_parts_rows(hipStream_t s, const float* yp, uint32_t parts, uint32_t m, uint32_t n, void* y, int y_dtype,
                                    uint32_t y_stride);
// (`out_stride`: elements from one row of hi / lo to the next; 0 = k)
mi355q_status launch_split_f32_bf16x2(hipStream_t s, const float* x, uint32_t m, uint32_t k, uint32_t x_stride, uint16_t* hi,
                                      uint16_t* lo, uint32_t out_stride = 0);
mi355q_status launch_gemv_generic(hipStream_t s, const WView& w, const void* x, int x_dtype,
                                  void* y, int y_dtype, uint32_t m, uint32_t x_stride,
                                  uint32_t y_stride);
mi355q_status launch_embedding_lookup(hipStream_t s, const WView& w, const int32_t* token_ids, uint32_t sequence_length,
                                      void* out, int out_dtype, uint32_t out_stride, int has_scale,
                                      float embedding_scale);
// Partial keys of the fused output head: one per workgroup of the projection launch.
constexpr uint32_t kArgmaxPartialCapacity = 65536;
// Where a fused head leaves its partial keys, and how many fit (null: the launch has no arg-max tail).
struct HeadKeys {
    unsigned long long* ptr = nullptr;
    uint32_t capacity = 0;
};
// The entry point that allocates nothing keeps its keys in a device array of the library image: one pointer per device,
// resolved when a context is created on that device (runtime.hip); null before that.  kStaticHeadKeys keys for the fused
// head, then kArgmaxStandaloneKeys for the two-launch arg-max.
constexpr uint32_t kStaticHeadKeys = 32768;
unsigned long long* static_head_keys(int device);
mi355q_status launch_argmax_finish(hipStream_t s, const unsigned long long* partial, uint32_t count, int32_t* token_out);
// `partial`: 256 keys of scratch for the two-launch form taken by long vectors (null: always one workgroup).
constexpr uint32_t kArgmaxStandaloneKeys = 256;
mi355q_status launch_argmax(hipStream_t s, const void* logits, int dtype, uint32_t n,
                            int32_t* token_out, unsigned long long* partial);
mi355q_status launch_pack_sz(hipStream_t s, const uint16_t* scales, const uint16_t* biases, uint32_t* sz,
                             size_t groups, uint32_t blocks_per_row, uint32_t sz_stride);

// Fast split-plane GEMV (kernels_gemv.hip).  can_* say whether a shape is eligible.
bool gemv_fast_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride);
mi355q_status launch_gemv_fast(hipStream_t s, const mi355q_context* ctx, const WView& w,
                               const void* x, int x_dtype, void* y, int y_dtype, uint32_t m,
                               uint32_t x_stride, uint32_t y_stride, float* logits_f32,
                               int32_t* token_out, HeadKeys keys);
// Gate and up projection of one activation row with the gated activation as epilogue, one launch (rows kernel over row
// pairs); `gemv_gated_eligible` says whether the pair of weights and the shape have such a launch.
bool gemv_gated_eligible(const mi355q_context* ctx, const WView& gate, const WView& up, int x_dtype, uint32_t m, uint32_t x_stride);
mi355q_status launch_gemv_gated(hipStream_t s, const mi355q_context* ctx, const WView& gate, const WView& up, const void* x,
                                int x_dtype, void* y, int y_dtype, uint32_t x_stride, int activation);
mi355q_status launch_gated_activation(hipStream_t s, const void* gate, const void* up, void* out, int dtype, uint32_t dimension,
                                      uint32_t sequence_length, uint32_t gate_stride, uint32_t up_stride, uint32_t out_stride,
                                      int activation);
// Raises a kernel's dynamic-LDS limit above 64 KiB once per (kernel, device) instead of on every launch.
mi355q_status raise_lds_limit(const void* kernel, size_t lds_bytes);
// Block-layout GEMV (gemv_staf.hip): reads STAF interleaved blocks in place.
bool gemv_staf_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride);
mi355q_status launch_gemv_staf(hipStream_t s, const mi355q_context* ctx, const WView& w, const void* x, int x_dtype,
                               void* y, int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride);
mi355q_status launch_gemv_staf_multi(hipStream_t s, const mi355q_context* ctx, uint32_t count, const WView* w,
                                     const void* x, int x_dtype, void* const* y, const uint32_t* y_strides, int y_dtype,
                                     uint32_t m, uint32_t x_stride, float* logits_f32, int32_t* token_out,
                                     HeadKeys keys);
struct GemvLaunchShape {
    uint32_t grid, block, lds_bytes, rows_per_workgroup;
    const char* kernel;
};
GemvLaunchShape gemv_staf_shape(const mi355q_context* ctx, const WView& w, uint32_t m);
GemvLaunchShape gemv_fast_shape(const mi355q_context* ctx, const WView& w, uint32_t m, int x_dtype);

mi355q_status launch_gemv_fast_multi(hipStream_t s, const mi355q_context* ctx, uint32_t count, const WView* w,
                                     const void* x, int x_dtype, void* const* y, const uint32_t* y_strides, int y_dtype,
                                     uint32_t m, uint32_t x_stride, float* logits_f32, int32_t* token_out,
                                     HeadKeys keys);

// Matrix-core decode kernel over the TILE16 layout (gemv_tile16.hip)
constexpr int kTile16MaxSegments = 3;
struct Tile16LaunchShape {
    uint32_t ksplit, tiles_per_wg, waves, blocks_per_wave, grid, block, lds_bytes;
    uint32_t passes;     // row tiles a wavefront walks on one staged copy of the activations
    uint32_t parts;      // K parts (1: whole rows); each part has wgs_per_part workgroups and stages only its columns
    uint32_t wgs_per_part;
};
// Rows the matrix-core decode kernels stage for m activation rows: an f16 row is staged as two bf16 rows (gemv_tile16.hip)
inline uint32_t staged_rows(int x_dtype, uint32_t m) { return x_dtype == MI355Q_F16 ? 2 * m : m; }
bool gemv_tile16_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride);
// K parts a launch of M rows takes: 1 = whole rows (needed by fused q+k+v / gate+up launches and by the fused head)
// (m: staged rows, see staged_rows)
uint32_t gemv_tile16_k_parts(const mi355q_context* ctx, const WView& w, uint32_t m);
// the same for a shape: 0 when no power-of-two split of K leaves M staged rows inside LDS
// block_codes: codes in 64 bytes of a weight row (128 at 4 bits)
uint32_t gemv_tile16_parts_for(uint32_t k, uint32_t m, uint32_t n_row_tiles, uint32_t cus, uint32_t block_codes = 128);
Tile16LaunchShape gemv_tile16_shape(const mi355q_context* ctx, uint32_t n_row_tiles, uint32_t k, uint32_t m,
                                    uint32_t block_codes = 128);
mi355q_status launch_gemv_tile16_multi(hipStream_t s, mi355q_context* ctx, uint32_t count, const WView* w,
                                       const void* x, int x_dtype, void* const* y, const uint32_t* y_strides, int y_dtype,
                                       uint32_t m, uint32_t x_stride, float* logits_f32, int32_t* token_out,
                                       HeadKeys keys);
mi355q_status launch_tile16_pack(hipStream_t s, const WView& planes, uint32_t* tiles);

// Matrix-core small-batch kernel over the split planes (gemv_mfma_planes.hip): 2 <= M <= 16, q4 g64 / g128.  Its
// workgroups are shaped like those of the TILE16 kernel (16-row tiles, blocks of 128 codes).
// Rows from which it is taken; below, the split-plane dot-product kernels are as fast or faster (measured, Llama-3-8B
// layer step in four launches: M = 2 42 us against 48 us here, M = 4 59 against 56, M = 8 117 against 55).
// fewest activation rows for which the matrix-core kernel beats the dot-product kernels on the same planes (measured;
// 8 bits, 4096 -> 14336: two rows 16 us on the dot products, three 25 us, against 19 us on the matrix cores; 4 bits, a
// Llama-3-8B layer step: two rows 42 us on the dot products, three 58-61 us, against 52-55 us on the matrix cores)
inline uint32_t mfma_planes_min_rows(uint32_t bits) { (void)bits; return 3u; }
// f16 rows are staged as two bf16 rows each: three f16 rows (six staged) pay on the matrix cores, two stay on the f16
// dot-product kernels (a Llama-3-8B layer step at two f16 rows: 42.6 us there)
inline bool mfma_planes_pays(uint32_t bits, int x_dtype, uint32_t m) {
    return x_dtype == MI355Q_F16 ? m >= 3 : m >= mfma_planes_min_rows(bits);
}
// Three or four bf16 rows on small 4-bit matrices (rows of two K-steps of the dot-product rows kernel; below 24 MB of
// weights in the launch at three rows, below 12 MB at four) stay on that kernel, every row on each unpacked code
// pair: its launch starts and ends faster than the matrix-core kernel's, whose workgroups stage the batch and add
// partial tiles through LDS (Llama-3-8B: q+k+v 14 MB at three rows 7.5 us against 8.8 us, at four 9.4 against 9.0;
// o 9 MB 6.1 against 8.7 and 6.8 against 8.8; gate+up and down stay on the matrix cores).
inline bool gemv_rows_batch_pays(uint32_t count, const WView* v, int x_dtype, uint32_t m) {
    if (x_dtype != MI355Q_BF16 || m < 3 || m > 4) return false;
    uint64_t bytes = 0;
    for (uint32_t i = 0; i < count; i++) {
        if (v[i].layout != MI355Q_LAYOUT_PLANES || v[i].bits != 4 || (v[i].group != 64 && v[i].group != 128)) return false;
        if (v[i].k <= 2048 || v[i].k > 4096) return false;
        bytes += (uint64_t)v[i].n * (v[i].k / v[i].group) * (4 + v[i].group / 2);
    }
    return bytes < ((uint64_t)(m == 3 ? 24 : 12) << 20);
}
bool gemv_mfma_planes_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride);
// (m below: staged rows, see staged_rows)
uint32_t gemv_mfma_planes_k_parts(const mi355q_context* ctx, const WView& w, uint32_t m);
Tile16LaunchShape gemv_mfma_planes_shape(const mi355q_context* ctx, uint32_t n_row_tiles, uint32_t k, uint32_t bits, uint32_t m);
mi355q_status launch_gemv_mfma_planes_multi(hipStream_t s, mi355q_context* ctx, uint32_t count, const WView* w,
                                            const void* x, int x_dtype, void* const* y, const uint32_t* y_strides, int y_dtype,
                                            uint32_t m, uint32_t x_stride);
// Rows one launch of the small-batch kernels takes for this weight: 16 on TILE16 records and on planes the
// matrix-core kernel reads, else 8.
uint32_t small_batch_rows(const WView& w, int x_dtype, uint32_t x_stride);
// Rows up to which mi355q_qgemm stays on those kernels (launch after launch) before the fused prefill kernel takes over
uint32_t small_batch_limit(const WView& w, int x_dtype, uint32_t x_stride);

// Validated dispatch shared by the direct entry points and by plan replay (api.hip)
mi355q_status dispatch_batched(mi355q_context* ctx, hipStream_t s, uint32_t count, const mi355q_weight* const* weights,
                               const void* x, int x_dtype, void* const* ys, int y_dtype, uint32_t m, uint32_t xs,
                               uint32_t flags);
mi355q_status dispatch_linear(mi355q_context* ctx, hipStream_t s, const mi355q_weight* w, const void* x, int x_dtype,
                              void* y, int y_dtype, uint32_t m, uint32_t xs, uint32_t ys, uint32_t flags,
                              bool small_m_only);
mi355q_status dispatch_gated(mi355q_context* ctx, hipStream_t s, const mi355q_weight* w_gate, const mi355q_weight* w_up,
                             const void* x_dev, int x_dtype, void* y_dev, int y_dtype, uint32_t m, uint32_t xs, uint32_t ys,
                             int activation, uint32_t flags);
mi355q_status dispatch_output_head(mi355q_context* ctx, hipStream_t s, const mi355q_weight* w, const void* x,
                                   int x_dtype, float* logits, int32_t* token, uint32_t flags, HeadKeys keys,
                                   bool no_allocation = false);
void plan_shared_launch_shape(const mi355q_weight* const* ws, uint32_t count, uint32_t m, int x_dtype, uint32_t x_stride,
                              uint32_t flags, mi355q_step* s);

// MFMA GEMM (kernels_gemm.hip)
struct GemmLaunchShape {
    uint32_t bm, bn, stages, grid, block, lds_bytes, splits, kt_per_split;
};
GemmLaunchShape gemm_mfma_shape(const mi355q_context* ctx, uint32_t m, uint32_t n, uint32_t k);
// ---- the one table of routes (route.cpp) --------------------------------------------------------------------
// Which route a linear projection takes is decided in ONE place, from the weight's view, the activation type, the
// row count, the row stride and the caller's flags; dispatch_linear (api.hip) launches what it says and the planner
// (planner.cpp) describes what it says, so a plan record cannot name a kernel the launch would not run.
enum class LinearRoute : int {
    kErrorRows = 0,            // the decode entry point takes at most eight rows
    kErrorFlags,               // contradictory selection flags
    kErrorTwoStepUnavailable,  // FORCE_TWO_STEP on a problem the route does not take
    kErrorNoFusedKernel,       // FORCE_MFMA on a weight no fused matrix-core kernel reads
    kSplitRows,                // fp32 rows as three bf16 rows each on the bf16 decode kernels, partial results added
    kTwoStep,                  // dequantise once into scratch, then the platform's dense GEMM
    kStream,                   // weights streamed through registers into the matrix cores (a few to 96 rows)
    kSmallBatch,               // the decode kernels, eight or sixteen rows a launch (small_kernel() names the kernel)
    kFused                     // fused dequantise + matrix-core GEMM: the wide-tile kernel where gemm_wide_taken(), else the tiled one
};
struct RouteFacts {
    bool decode_entry;         // mi355q_qgemv / plan_decode_step (at most eight rows), else mi355q_qgemm / plan_prefill_steps
    bool library_ok;           // the dense library can serve this problem (launcher: asked; planner: not ruled out for the context)
    bool x_aligned;            // the activation pointer is 16-byte aligned (the planner assumes it)
};
LinearRoute linear_route(const WView& v, int x_dtype, uint32_t m, uint32_t x_stride, uint32_t flags, const RouteFacts& facts);
const char* linear_route_name(LinearRoute r);
// The decode kernel a small batch (or one slice of it) runs on.
enum class SmallKernel : int { kTile16 = 0, kMfmaPlanes, kDotPlanes, kStafInPlace, kGeneric };
SmallKernel small_kernel(const WView& v, int x_dtype, uint32_t rows, uint32_t x_stride, uint32_t flags, bool x_aligned);
const char* small_kernel_name(SmallKernel k);
uint32_t small_batch_step(const WView& v, int x_dtype, uint32_t m, uint32_t x_stride, uint32_t flags);
// What two or three projections that share their activations run as (q+k+v, gate+up): one launch over the rows of all
// matrices on one of five kernels, the rows split first, the shared launch in steps, or a launch per projection.  Asked
// by dispatch_batched (api.hip), which launches it, and by the planner, which describes it.
enum class SharedRoute : int {
    kStream = 0,       // the streamed-weight kernel over the matrices together
    kMfmaPlanes,       // the small-batch matrix-core kernel over the planes
    kDotPlanes,        // the dot-product decode kernels over the planes
    kTile16,           // the matrix-core kernel over TILE16 records
    kStafInPlace,      // the in-place kernel over the reference's blocks
    kWide,             // prompts: the wide-tile prefill kernel over the column tiles of all matrices
    kSplitRows,        // fp32 rows split into bf16 rows once for all projections, then one of the above on those
    kSteps,            // more rows than one shared launch takes: the shared launch in steps
    kSeparate,         // each projection on its own route (linear_route)
};
SharedRoute shared_route(const mi355q_context* ctx, uint32_t count, const WView* views, int x_dtype, uint32_t m, uint32_t xs,
                         uint32_t flags, bool x_aligned);
const char* shared_route_name(SharedRoute r);

// Every entry point that enqueues work opens one of these first.  The context's scratch (partial results, dense
// copies, split rows, gate / up sums, arg-max keys) is shared by its launches, so they must be ordered: when the scratch
// was last used on ANOTHER stream and an event recorded behind that work has not completed, the entry point fails
// with MI355Q_ERR_INVALID_ARGUMENT instead of racing (the null stream is ordered with every blocking stream and is let
// through).  On the way out, if the call touched the scratch, the event is recorded again (not while capturing).
struct ScratchGuard {
    mi355q_context* ctx;
    hipStream_t stream;
    mi355q_status status;
    ScratchGuard(mi355q_context* c, hipStream_t s);
    ~ScratchGuard();
    ScratchGuard(const ScratchGuard&) = delete;
    ScratchGuard& operator=(const ScratchGuard&) = delete;
};
// Grows the context's scratch buffer for fp32 partial results; nothing is released before the context goes.
mi355q_status ensure_workspace(mi355q_context* ctx, size_t bytes);
mi355q_status ensure_split_buffer(mi355q_context* ctx, size_t bytes);
mi355q_status ensure_gated_buffer(mi355q_context* ctx, size_t bytes);
// fp32 activations as three bf16 rows each on the bf16 decode kernels (api.hip): row pitch of the bf16 rows, bf16 rows
// per activation row (0: the type is not split), and whether a call takes that route
inline uint32_t split_rows_stride(uint32_t k) { return (k + 7u) & ~7u; }
inline uint32_t split_rows_parts(int x_dtype) { return x_dtype == MI355Q_F32 ? 3u : 0u; }
bool split_rows_chosen(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride, uint32_t flags);
bool split_rows_small_batch(const WView& w, uint32_t parts, uint32_t m);
bool split_rows_take_stream(const WView& w, int x_dtype, uint32_t m);
bool gemm_mfma_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride);
// `flags`: MI355Q_FLAG_PROBE_TILED keeps the tiled kernel where the wide-tile one (gemm_wide.hip) would be taken,
// MI355Q_FLAG_PROBE_WIDE takes the wide-tile kernel wherever it reads the weight (A/B runs and tests)
mi355q_status launch_qgemm_mfma(hipStream_t s, mi355q_context* ctx, const WView& w,
                                const void* x, int x_dtype, void* y, int y_dtype, uint32_t m,
                                uint32_t x_stride, uint32_t y_stride, unsigned long long* probe = nullptr,
                                uint32_t flags = 0);

// Wide-tile MFMA GEMM for long prompts (gemm_wide.hip): 4-bit planes in groups of 64 / 128, bf16 activations; the weights
// are dequantised in registers, only the activations pass through LDS.  Taken from kWideMinRows rows (beyond what the
// streamed-weight kernel takes) where its workgroups occupy five eighths of the CUs (measured against the tiled kernel and
// the two-dispatch route: see gemm_wide_chosen).
// the dense library is forbidden for the context or could not be opened: the two-dispatch route serves nothing
inline bool library_ruled_out(const mi355q_context* ctx) { return ctx->dense_library_failed || ctx->dense_library_forbidden; }
constexpr uint32_t kWideMinRows = 97;
constexpr uint32_t kWideRowsBesideLibrary = 2560;   // from here the two-dispatch route is taken where the dense library is there
bool gemm_wide_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride);
bool gemm_wide_chosen(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride);
// `k`: the K the kernel walks (twice the weight's K for fp32 activations, see gemm_wide_k)
GemmLaunchShape gemm_wide_shape(uint32_t m, uint32_t n, uint32_t k, bool one_part = false);
// fp32 activations run as two bf16 halves side by side, hi = bf16(x) and lo = bf16(x - hi), against the weights twice
inline uint32_t gemm_wide_k(uint32_t k, int x_dtype) { return x_dtype == MI355Q_F32 ? 2 * k : k; }
uint32_t chip_cus();
void gemm_wide_force_shape(uint32_t bm, uint32_t splits);      // A/B runs (mi355q_probe_wide_shape)
// Two or three matrices that share the activations as one launch of the wide-tile kernel: every column tile belongs to
// one matrix (all but the last are whole numbers of 256-column tiles), K parts and their sum over the columns of all.
// `chosen`: from the rows where the streamed-weight kernel ends (measured against a launch per projection).
bool gemm_wide_multi_eligible(uint32_t count, const WView* w, int x_dtype, uint32_t m, uint32_t x_stride);
bool gemm_wide_multi_chosen(uint32_t count, const WView* w, int x_dtype, uint32_t m, uint32_t x_stride);
GemmLaunchShape gemm_wide_multi_shape(uint32_t count, const WView* w, uint32_t m, int x_dtype);
mi355q_status launch_qgemm_wide_multi(hipStream_t s, mi355q_context* ctx, uint32_t count, const WView* w, const void* x,
                                      int x_dtype, void* const* y, const uint32_t* y_strides, int y_dtype, uint32_t m,
                                      uint32_t x_stride);
// The gated MLP projection on the wide-tile kernel: gate_proj and up_proj as the two column fragments of every
// wavefront, activation(gate) * up in the epilogue, one launch and no intermediate matrices.  Chosen under the same
// rule as the plain kernel, over the 2 N columns of the two matrices, K in one part.
bool gemm_wide_gated_eligible(const WView& gate, const WView& up, int x_dtype, uint32_t m, uint32_t x_stride);
bool gemm_wide_gated_chosen(const WView& gate, const WView& up, int x_dtype, uint32_t m, uint32_t x_stride);
// what dispatch_gated (api.hip) runs and the planner describes: the probe flag takes the kernel wherever it reads the
// pair, other selection flags leave the gated projection to the separate launches they select; from the rows where the
// two-dispatch route is ahead the projections go there and the activation stays a launch of its own
bool gemm_wide_gated_taken(const mi355q_context* ctx, const WView& gate, const WView& up, int x_dtype, uint32_t m, uint32_t x_stride,
                           uint32_t flags);
mi355q_status launch_qgemm_wide_gated(hipStream_t s, mi355q_context* ctx, const WView& gate, const WView& up, const void* x,
                                      int x_dtype, void* y, int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride,
                                      int activation);
inline bool gemm_wide_taken(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride, uint32_t flags) {
    if (flags & MI355Q_FLAG_PROBE_TILED) return false;
    if (flags & MI355Q_FLAG_PROBE_WIDE) return gemm_wide_eligible(w, x_dtype, m, x_stride);
    return gemm_wide_chosen(w, x_dtype, m, x_stride);
}
mi355q_status launch_qgemm_wide(hipStream_t s, mi355q_context* ctx, const WView& w, const void* x, int x_dtype, void* y,
                                int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride, unsigned long long* probe = nullptr);
// Streamed-weight matrix-core kernel (gemm_stream.hip): 4- and 8-bit planes, bf16 or f16 activations, at most 96 rows.
constexpr uint32_t kStreamMaxRows = 96;
// blocks in place: codes (N x K) from which it replaces the in-place decode kernel at three rows / at five rows
constexpr uint64_t kStreamBlocksLargeCodes = (uint64_t)1 << 25, kStreamBlocksMediumCodes = (uint64_t)1 << 23;
struct StreamLaunchShape {
    uint32_t row_blocks;       // workgroups along N (64 weight rows each)
    uint32_t parts;            // K parts (workgroups along K; fp32 partial results added by a second launch)
    uint32_t iters_per_part;   // iterations of 256 columns per part
    uint32_t m_blocks;         // 32-row blocks of activations
    uint32_t lds_bytes;
};
bool gemm_stream_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride);
bool gemm_stream_chosen(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride);
bool gemm_stream_chosen_multi(uint32_t count, const WView* w, int x_dtype, uint32_t m, uint32_t x_stride);
// Whether the kernel keeps the weights unrounded at m rows (scale and bias applied to a K-tile's fp32 sums): one block
// of activation rows, groups of whole K-tiles.
bool gemm_stream_unrounded(const WView& w, uint32_t m);
StreamLaunchShape gemm_stream_shape(const mi355q_context* ctx, uint32_t m, uint32_t n, uint32_t k);
mi355q_status launch_qgemm_stream(hipStream_t s, mi355q_context* ctx, const WView& w, const void* x, int x_dtype, void* y,
                                  int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride);
// Up to three matrices that share the activations, K, the group size and the scale type, as one launch.
StreamLaunchShape gemm_stream_shape_blocks(const mi355q_context* ctx, uint32_t m, uint32_t row_blocks, uint32_t k);
bool gemm_stream_multi_eligible(uint32_t count, const WView* w, int x_dtype, uint32_t m, uint32_t x_stride);
mi355q_status launch_qgemm_stream_multi(hipStream_t s, mi355q_context* ctx, uint32_t count, const WView* w, const void* x,
                                        int x_dtype, void* const* y, const uint32_t* y_strides, int y_dtype, uint32_t m,
                                        uint32_t x_stride);
// The gated MLP projection on the streamed-weight kernel: a workgroup's two row blocks read the same 32 rows of gate_proj
// and up_proj, activation(gate) * up stored from its epilogue, one launch.  Taken where gate+up would share a launch of
// this kernel (shared_route) and the workgroups of the gated form (32 output columns each) need no K parts; the flag
// that forces the kernel takes it with K in one part whatever the shape.
bool gemm_stream_gated_taken(const mi355q_context* ctx, const WView& gate, const WView& up, int x_dtype, uint32_t m,
                             uint32_t x_stride, uint32_t flags);
StreamLaunchShape gemm_stream_gated_shape(const mi355q_context* ctx, uint32_t m, uint32_t n, uint32_t k);
mi355q_status launch_qgemm_stream_gated(hipStream_t s, mi355q_context* ctx, const WView& gate, const WView& up, const void* x,
                                        int x_dtype, void* y, int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride,
                                        int activation);
// Two-dispatch prefill route: dequantise the whole matrix to bf16 in the context's scratch, then the platform's
// dense GEMM.  `dense_library_serves` answers whether the library can be opened and has an algorithm for the problem.
// The library's workspace is its own allocation per context (zeroed once, written by nothing else).
constexpr size_t kDenseLibraryWorkspace = (size_t)64 << 20;
// Both operands in `ab_dtype` (bf16, f16 or fp32), fp32 accumulation, output in y_dtype.
bool dense_library_serves(mi355q_context* ctx, int ab_dtype, uint32_t m, uint32_t n, uint32_t k, uint32_t x_stride,
                          uint32_t y_stride, int y_dtype);
// `accumulate`: Y += X W^T instead of Y = X W^T (the second half of a split-activation product).  The first eager call
// of a problem checks sampled result elements against plain dot products (and synchronises the stream); a wrong
// matrix makes the problem unusable and returns MI355Q_ERR_KERNEL_NOT_FOUND, on which callers take another route.
mi355q_status dense_library_gemm(hipStream_t s, mi355q_context* ctx, int ab_dtype, const void* x, const void* w_dense,
                                 void* y, int y_dtype, uint32_t m, uint32_t n, uint32_t k, uint32_t x_stride,
                                 uint32_t y_stride, bool accumulate = false);
void dense_library_release(mi355q_context* ctx);
// Rows from which the two-dispatch route is taken.  Beside the fused matrix-core kernel (measured at sustained load,
// q4 g64, N(0,1) activations, fused against two-dispatch with the library's candidates timed): 4096 -> 14336 at M = 512
// 83 against 86 us, M = 768 136 against 101, M = 1024 126 against 115, M = 2048 242 against 199; 4096 -> 4096 at
// M = 256 32 against 33 us, M = 512 46 against 41, M = 1024 61 against 53, M = 2048 92 against 67; 14336 -> 4096 at
// M = 1024 133 against 153 us, M = 2048 234 against 236, M = 3072 349 against 289.  So: rows longer than the matrix
// is tall (K > N) from 2048, wide matrices (N >= 8192) from 768, the others from 512.
// Where only the decode kernels would serve (formats and layouts the fused kernel does not read; block layout,
// 4096 -> 14336: M = 32 in four launches of eight rows 147 us, two-dispatch 47 us) it starts at sixteen rows.
// f16 rows that the matrix-core decode kernels take eight a launch: from 32 rows.
constexpr uint32_t kTwoStepMinRowsLongK = 2048, kTwoStepMinRowsWide = 768, kTwoStepMinRowsBesideFused = 512;
constexpr uint32_t kTwoStepWideColumns = 8192, kTwoStepMinRowsOtherwise = 16;
constexpr uint32_t kTwoStepMinRowsF16Batches = 32;
// Rows from which mi355q_gemm_bf16 hands a plain dense product to the library.
constexpr uint32_t kDenseLibraryMinRows = 128;
bool decode_kernel_reads(const WView& w, int x_dtype, uint32_t x_stride);
// whether the library has an algorithm for the product(s) the route would run for these types and rows
bool gemm_two_step_serves(mi355q_context* ctx, const WView& w, int x_dtype, int y_dtype, uint32_t m, uint32_t x_stride,
                          uint32_t y_stride);
// rows of `cols` elements from one floating-point type to another (bf16, f16, fp32), strides in elements
mi355q_status launch_convert_rows(hipStream_t s, const void* src, int src_dtype, uint32_t src_stride, void* dst, int dst_dtype,
                                  uint32_t dst_stride, uint32_t rows, uint32_t cols);
bool gemm_two_step_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride);
bool gemm_two_step_chosen(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride, uint32_t flags);
mi355q_status launch_qgemm_two_step(hipStream_t s, mi355q_context* ctx, const WView& w, const void* x, int x_dtype,
                                    void* y, int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride);
mi355q_status launch_gemm_bf16_mfma(hipStream_t s, mi355q_context* ctx, const void* a,
                                    int a_dtype, const uint16_t* b, void* c, int c_dtype,
                                    uint32_t m, uint32_t n, uint32_t k, uint32_t a_stride,
                                    uint32_t c_stride);

}  // namespace mi355q
