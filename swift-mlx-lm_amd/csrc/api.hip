// Launch entry points of the C ABI: argument validation on the host, then kernel selection.
// Nothing here computes on the CPU; a shape no kernel accepts is an error, never a fallback.
#include <cstdlib>

#include "common.h"

using namespace mi355q;

namespace {

bool dtype_ok(int d) { return d == MI355Q_F16 || d == MI355Q_BF16 || d == MI355Q_F32; }

mi355q_status check_launch(mi355q_context* ctx, const mi355q_weight* w) {
    if (!ctx) return fail(MI355Q_ERR_NULL_HANDLE, "context is null");
    if (!w) return fail(MI355Q_ERR_NULL_HANDLE, "weight handle is null");
    if (w->ctx != ctx) return fail(MI355Q_ERR_INVALID_ARGUMENT, "weight handle belongs to another context");
    hipError_t e = hipSetDevice(ctx->device);
    if (e != hipSuccess) return fail(MI355Q_ERR_DEVICE, "hipSetDevice failed: %s", hipGetErrorString(e));
    return MI355Q_OK;
}

mi355q_status check_io(const mi355q_weight* w, const void* x, int x_dtype, const void* y, int y_dtype, uint32_t m,
                       uint32_t& x_stride, uint32_t& y_stride) {
    if (!x || !y) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null activation or output pointer");
    if (!dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return fail(MI355Q_ERR_INVALID_ARGUMENT, "bad dtype tag");
    if (m == 0) return fail(MI355Q_ERR_INVALID_ARGUMENT, "sequence length M must be >= 1");
    if (x_stride == 0) x_stride = (uint32_t)w->k;
    if (y_stride == 0) y_stride = (uint32_t)w->n;
    if (x_stride < w->k)
        return fail(MI355Q_ERR_SHAPE, "inputRowStride %u < inputDimension %llu", x_stride, (unsigned long long)w->k);
    if (y_stride < w->n)
        return fail(MI355Q_ERR_SHAPE, "output row stride %u < outputDimension %llu", y_stride,
                    (unsigned long long)w->n);
    const size_t xa = x_dtype == MI355Q_F32 ? 4 : 2, ya = y_dtype == MI355Q_F32 ? 4 : 2;
    if ((uintptr_t)x % xa || (uintptr_t)y % ya) return fail(MI355Q_ERR_INVALID_ARGUMENT, "misaligned pointer");
    return MI355Q_OK;
}

// Small-M path: the split-plane kernel or the matrix-core tile kernel when the layout and shape
// allow it, else the per-code kernel.
mi355q_status run_small_m(mi355q_context* ctx, hipStream_t s, const mi355q_weight* w, const void* x, int x_dtype,
                          void* y, int y_dtype, uint32_t m, uint32_t xs, uint32_t ys, uint32_t flags) {
    const WView v = w->view();
    const size_t xsz = x_dtype == MI355Q_F32 ? 4 : 2, ysz = y_dtype == MI355Q_F32 ? 4 : 2;
    const uint32_t step = small_batch_step(v, x_dtype, m, xs, flags);
    for (uint32_t m0 = 0; m0 < m; m0 += step) {
        const uint32_t mm = m - m0 < step ? m - m0 : step;
        const void* xp = (const char*)x + (size_t)m0 * xs * xsz;
        void* yp = (char*)y + (size_t)m0 * ys * ysz;
        mi355q_status st;
        void* yv[1] = {yp};
        const uint32_t strides[1] = {ys};
        switch (small_kernel(v, x_dtype, mm, xs, flags, (uintptr_t)xp % 16 == 0)) {
        case SmallKernel::kTile16:
            st = launch_gemv_tile16_multi(s, ctx, 1, &v, xp, x_dtype, yv, strides, y_dtype, mm, xs, nullptr, nullptr, HeadKeys{});
            break;
        case SmallKernel::kMfmaPlanes:
            st = launch_gemv_mfma_planes_multi(s, ctx, 1, &v, xp, x_dtype, yv, strides, y_dtype, mm, xs);
            break;
        case SmallKernel::kDotPlanes:
            // the dot-product kernels take eight rows a launch
            st = MI355Q_OK;
            for (uint32_t r0 = 0; r0 < mm && st == MI355Q_OK; r0 += 8)
                st = launch_gemv_fast(s, ctx, v, (const char*)xp + (size_t)r0 * xs * xsz, x_dtype,
                                      (char*)yp + (size_t)r0 * ys * ysz, y_dtype, mm - r0 < 8 ? mm - r0 : 8, xs, ys, nullptr,
                                      nullptr, HeadKeys{});
            break;
        case SmallKernel::kStafInPlace:
            st = launch_gemv_staf(s, ctx, v, xp, x_dtype, yp, y_dtype, mm, xs, ys);
            break;
        default:
            st = launch_gemv_generic(s, v, xp, x_dtype, yp, y_dtype, mm, xs, ys);
            break;
        }
        if (st != MI355Q_OK) return st;
    }
    return MI355Q_OK;
}

// fp32 activations, a few rows, on a weight the bf16 decode kernels read: every row becomes three bf16 rows whose sum
// is the row exactly (split_rows_bf16_kernel), the bf16 kernels run on those rows, and the partial results of a row are
// added.  Products stay exact, the matrix is read once per launch of sixteen or eight rows.
mi355q_status run_split_rows(mi355q_context* ctx, hipStream_t s, const mi355q_weight* w, const void* x, int x_dtype, void* y,
                             int y_dtype, uint32_t m, uint32_t xs, uint32_t ys, uint32_t flags) {
    const uint32_t n = (uint32_t)w->n, k = (uint32_t)w->k, kp = split_rows_stride(k), parts = split_rows_parts(x_dtype);
    const size_t xbytes = ((size_t)parts * m * kp * 2 + 255) & ~(size_t)255, ybytes = (size_t)parts * m * n * 4;
    if (mi355q_status st = ensure_split_buffer(ctx, xbytes + ybytes)) return st;
    uint16_t* const xp = (uint16_t*)ctx->split_buffer;
    float* const yp = (float*)((char*)ctx->split_buffer + xbytes);
    if (mi355q_status st = launch_split_rows_bf16(s, x, x_dtype, m, k, xs, xp, kp)) return st;
    const WView v = w->view();
    if (!(flags & (MI355Q_FLAG_FORCE_GENERIC | MI355Q_FLAG_FORCE_SMALL_M)) && split_rows_take_stream(v, x_dtype, m)) {
        if (mi355q_status st = launch_qgemm_stream(s, ctx, v, xp, MI355Q_BF16, yp, MI355Q_F32, parts * m, kp, n)) return st;
    } else if (mi355q_status st = run_small_m(ctx, s, w, xp, MI355Q_BF16, yp, MI355Q_F32, parts * m, kp, n, flags)) {
        return st;
    }
    return launch_sum_parts_rows(s, yp, parts, m, n, y, y_dtype, ys);
}

}  // namespace

namespace mi355q {

// Whether m rows of fp32 activations are served as three bf16 rows each on the bf16 decode kernels: no kernel but the
// per-code one reads fp32; taken when a bf16 decode kernel reads the weight and the 3 m rows fit one launch of it --
// three launches where a launch takes sixteen rows (4096 -> 14336 on 4-bit planes: 16-20 us up to five rows, 52 us at
// sixteen, where the dequantise-once route takes 105 us whatever the rows; with launches of eight rows two rows already
// take 35 us).  (f16 rows need no such route: the matrix-core kernels stage them as two bf16 rows themselves.)
bool split_rows_chosen(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride, uint32_t flags) {
    (void)x_stride;
    const uint32_t parts = split_rows_parts(x_dtype);
    if (!parts || (flags & (MI355Q_FLAG_FORCE_GENERIC | MI355Q_FLAG_FORCE_MFMA | MI355Q_FLAG_FORCE_TWO_STEP))) return false;
    // (FORCE_SMALL_M keeps the rows off the streamed-weight kernel: then only the decode kernels count)
    return split_rows_small_batch(w, parts, m) || (!(flags & MI355Q_FLAG_FORCE_SMALL_M) && split_rows_take_stream(w, x_dtype, m));
}

// The split rows fit the small-batch launches of a bf16 decode kernel.
bool split_rows_small_batch(const WView& w, uint32_t parts, uint32_t m) {
    const uint32_t kp = split_rows_stride((uint32_t)w.k);
    if (!decode_kernel_reads(w, MI355Q_BF16, kp)) return false;
    const uint32_t rows = small_batch_rows(w, MI355Q_BF16, kp);
    return (uint64_t)parts * m <= (rows >= 16 ? 3 * rows : rows);
}

// The split rows go to the streamed-weight kernel: up to 32 of them with unrounded weights (blocks in place from three
// fp32 rows' worth, where the dequantise-once route took 100-135 us; the planes from six fp32 rows, one launch instead
// of two or three); more of them, with weights rounded to bf16, only where the small-batch launches do not serve and
// the rows would otherwise take the dequantise-once route, which rounds the weights as well (from sixteen fp32 rows).
bool split_rows_take_stream(const WView& w, int x_dtype, uint32_t m) {
    const uint32_t parts = split_rows_parts(x_dtype);
    if (!parts || (uint64_t)parts * m > kStreamMaxRows) return false;
    const uint32_t pm = parts * m, kp = split_rows_stride((uint32_t)w.k);
    if (!gemm_stream_chosen(w, MI355Q_BF16, pm, kp)) return false;
    if (pm <= 32) return gemm_stream_unrounded(w, pm);
    return !split_rows_small_batch(w, parts, m) && m >= kTwoStepMinRowsOtherwise;
}

mi355q_status dispatch_linear(mi355q_context* ctx, hipStream_t s, const mi355q_weight* w, const void* x, int x_dtype,
                              void* y, int y_dtype, uint32_t m, uint32_t xs, uint32_t ys, uint32_t flags,
                              bool small_m_only) {
    if (mi355q_status st = check_io(w, x, x_dtype, y, y_dtype, m, xs, ys)) return st;
    const WView v = w->view();
    RouteFacts facts{};
    facts.decode_entry = small_m_only;
    facts.x_aligned = (uintptr_t)x % 16 == 0;
    // (asked only where the route is a candidate: the question opens the library)
    facts.library_ok = facts.x_aligned && ((flags & MI355Q_FLAG_FORCE_TWO_STEP) || gemm_two_step_chosen(v, x_dtype, m, xs, flags)) &&
                       gemm_two_step_serves(ctx, v, x_dtype, y_dtype, m, xs, ys);
    // the clock probe cell lives behind the argmax cells of the context's scratch
    unsigned long long* const probe = (flags & MI355Q_FLAG_PROBE_CLOCK) ? ctx->argmax_scratch + 16 : nullptr;
    for (int attempt = 0; attempt < 2; attempt++) {
        switch (linear_route(v, x_dtype, m, xs, flags, facts)) {
        case LinearRoute::kErrorRows:
            return fail(MI355Q_ERR_INVALID_ARGUMENT, "qgemv takes 1 <= M <= 8 (got %u); use qgemm", m);
        case LinearRoute::kErrorFlags:
            return fail(MI355Q_ERR_INVALID_ARGUMENT, "contradictory kernel selection flags");
        case LinearRoute::kErrorTwoStepUnavailable:
            return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the two-dispatch route takes 16-byte aligned activations, K and the row stride multiples of 8");
        case LinearRoute::kErrorNoFusedKernel:
            return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the MFMA GEMM does not accept this format, layout or stride");
        case LinearRoute::kSplitRows:
            return run_split_rows(ctx, s, w, x, x_dtype, y, y_dtype, m, xs, ys, flags);
        case LinearRoute::kTwoStep: {
            const mi355q_status st = launch_qgemm_two_step(s, ctx, v, x, x_dtype, y, y_dtype, m, xs, ys);
            // a library result that fails its check makes the problem unusable: the table is asked again without the library
            if (st != MI355Q_ERR_KERNEL_NOT_FOUND || (flags & MI355Q_FLAG_FORCE_TWO_STEP)) return st;
            facts.library_ok = false;
            continue;
        }
        case LinearRoute::kStream:
            return launch_qgemm_stream(s, ctx, v, x, x_dtype, y, y_dtype, m, xs, ys);
        case LinearRoute::kSmallBatch:
            return run_small_m(ctx, s, w, x, x_dtype, y, y_dtype, m, xs, ys, flags);
        case LinearRoute::kFused:
            return launch_qgemm_mfma(s, ctx, v, x, x_dtype, y, y_dtype, m, xs, ys, probe, flags);
        }
    }
    return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no route serves this projection");
}

// Rows up to which the small-batch kernels, one launch after the other, beat the fused prefill kernel: two launches where
// a launch takes sixteen rows (a Llama-3-8B layer step in bf16: 24 rows 124 us in two launches against 159 us on the
// prefill kernel, 32 rows 136 against 161).
uint32_t small_batch_limit(const WView& w, int x_dtype, uint32_t x_stride) {
    const uint32_t rows = small_batch_rows(w, x_dtype, x_stride);
    if (gemm_stream_eligible(w, x_dtype, rows + 1, x_stride)) {                // the streamed-weight kernel takes over
        // blocks in place: the in-place decode kernel costs 18.7 us at four rows and 35.7 at eight (4096 -> 14336 q4 g64;
        // 31 and 60 on 14336 -> 4096), the streamed kernel with unrounded weights 15.6 and 17.6 whatever the rows
        // (and from the first row where no decode kernel reads the blocks: rows that are not whole 16-byte units)
        // Its cost has a floor of about 10 us (K parts and their sum launch on matrices of few rows), so smaller
        // matrices change over later: 4096 -> 4096 at four rows 10.6 against 8.8 us, at six 10.6 against 14.5;
        // 4096 -> 1024 at eight rows 9.8 against 10.0.
        const bool other_width = w.bits != 4 && w.bits != 8;
        if (w.layout == MI355Q_LAYOUT_STAF_BLOCKS && !other_width && gemm_stream_unrounded(w, 3)) {
            const uint64_t codes = (uint64_t)w.n * w.k;
            const uint32_t first = codes >= kStreamBlocksLargeCodes ? 3 : codes >= kStreamBlocksMediumCodes ? 5 : rows + 1;
            return gemv_staf_eligible(w, x_dtype, 1, x_stride) ? first - 1 : 0;
        }
        // 2, 3, 5 and 6 bits (planes and blocks): the decode kernels take four rows a launch there, so a fifth row is a
        // second launch (4096 -> 14336 q6 g64: 19.4 us at four rows, 29.9 at five, 38.5 at eight, 77.7 at sixteen; the
        // streamed kernel 20.6-21.1 throughout; 4096 -> 4096: 8.4 / 12.9 / 16.2 / 31.8 against 12.3-12.8)
        if (other_width && gemm_stream_unrounded(w, 5)) {
            const uint64_t codes = (uint64_t)w.n * w.k;
            if (w.layout == MI355Q_LAYOUT_STAF_BLOCKS && !gemv_staf_eligible(w, x_dtype, 1, x_stride)) return 0;
            return codes >= kStreamBlocksMediumCodes ? 4 : rows;
        }
        return rows;
    }
    return rows >= 16 ? 2 * rows : rows;
}

// Rows the streamed-weight kernel serves: beyond one small-batch launch, up to its own limit (4096 -> 14336 q4 g64:
// 17 rows 16.6 us where two small-batch launches take 25.8 and the tiled kernel 30.2; 32 rows 17.1 against 33.1 and
// 29.6; 64 rows 21.1 against 33.2 tiled; 96 rows 26.5 against 35.0; 14336 -> 4096: 32 rows 19.3 against 31.4, 96 rows
// 28.0 against 35.4; 4096 -> 4096: 32 rows 12.4 against 17.6, 96 rows 17.9 against 22.7).
bool gemm_stream_chosen(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride) {
    return m <= kStreamMaxRows && gemm_stream_eligible(w, x_dtype, m, x_stride) && m > small_batch_limit(w, x_dtype, x_stride);
}

// The same for two or three matrices that would share a launch: the rows of all of them together decide.
bool gemm_stream_chosen_multi(uint32_t count, const WView* w, int x_dtype, uint32_t m, uint32_t x_stride) {
    if (m > kStreamMaxRows || !gemm_stream_multi_eligible(count, w, x_dtype, m, x_stride)) return false;
    WView all = w[0];
    for (uint32_t i = 1; i < count; i++) all.n += w[i].n;
    return gemm_stream_chosen(all, x_dtype, m, x_stride);
}

uint32_t small_batch_rows(const WView& w, int x_dtype, uint32_t x_stride) {
    const uint32_t most = x_dtype == MI355Q_F16 ? 8 : 16;      // sixteen staged rows: f16 rows are staged as two each
    if (w.layout == MI355Q_LAYOUT_TILE16) return most;
    return gemv_mfma_planes_eligible(w, x_dtype, most, x_stride) ? most : 8;
}

// Whether one of the decode kernels (not the per-code kernel) takes this layout with this activation type.
bool decode_kernel_reads(const WView& w, int x_dtype, uint32_t x_stride) {
    return gemv_tile16_eligible(w, x_dtype, 1, x_stride) || gemv_fast_eligible(w, x_dtype, 1, x_stride) ||
           gemv_staf_eligible(w, x_dtype, 1, x_stride);
}

bool gemm_two_step_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride) {
    (void)x_dtype;                                               // the dense copy takes the activations' type
    return m >= 1 && w.k % 8 == 0 && x_stride % 8 == 0 &&
           (uint64_t)w.n * w.k * 4 <= ((uint64_t)16 << 30);      // the dense copy lives in the context's scratch
}

bool gemm_two_step_chosen(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride, uint32_t flags) {
    if (flags & (MI355Q_FLAG_FORCE_MFMA | MI355Q_FLAG_FORCE_SMALL_M | MI355Q_FLAG_FORCE_GENERIC | MI355Q_FLAG_FORCE_STREAM)) return false;
    if (flags & MI355Q_FLAG_FORCE_TWO_STEP) return true;
    if (!gemm_two_step_eligible(w, x_dtype, m, x_stride)) return false;
    if (gemm_stream_chosen(w, x_dtype, m, x_stride)) return false;      // a few dozen rows on 4- / 8-bit planes
    // long prompts on 4-bit planes: this library's own kernel, up to the rows from which the two dispatches are faster
    // by a tenth and more (M = 3072: 4096 -> 14336 277 us against 314, 14336 -> 4096 282 against 307; M = 2048: 196-216
    // against 202-216 and 224 against 210)
    if (gemm_wide_chosen(w, x_dtype, m, x_stride) && m < kWideRowsBesideLibrary) return false;
    if (!gemm_mfma_eligible(w, x_dtype, m, x_stride)) {
        // no decode kernel reads the weight: from the second row; from the first where the per-code kernel leaves most
        // of its lanes idle (a lane per code of a group: q3 g16 blocks, 4096 -> 14336, take it 465 us at one row
        // against 120 us on this route)
        if (!decode_kernel_reads(w, x_dtype, x_stride)) return m >= 2 || w.group < 64;
        // f16 rows on the matrix-core decode kernels, eight a launch: a Llama-3-8B layer step takes 56-67 us per eight
        // rows there and 255-296 us on this route whatever the rows
        const bool f16_on_matrix_cores = x_dtype == MI355Q_F16 && (gemv_tile16_eligible(w, x_dtype, 8, x_stride) ||
                                                                   gemv_mfma_planes_eligible(w, x_dtype, 8, x_stride));
        const uint32_t least = f16_on_matrix_cores ? kTwoStepMinRowsF16Batches : kTwoStepMinRowsOtherwise;
        const uint32_t one_launch = small_batch_rows(w, x_dtype, x_stride);      // what one small-batch launch still takes
        return m >= least && m > one_launch;
    }
    return m >= (w.k > w.n ? kTwoStepMinRowsLongK : w.n >= kTwoStepWideColumns ? kTwoStepMinRowsWide : kTwoStepMinRowsBesideFused);
}

// The three forms of the route, by rows and activation type:
//   * below sixteen rows (only where no decode kernel reads the weight): fp32 weights, the activations widened to
//     fp32, an fp32 product, the result narrowed to the output type -- the arithmetic of the decode kernels;
//   * fp32 activations into an fp32 result from sixteen rows: bf16 weights, as the reference's gemm_bf16_f32s has
//     them, against the activations split into two bf16 matrices (sixteen bits of every activation), two library
//     products of which the second accumulates (M = 2048, 4096 -> 14336: 0.47 ms against 1.66 ms for an fp32 product);
//   * otherwise: the matrix dequantised to the activations' type and one product in that type.
namespace {
enum class TwoStepForm { kExactF32, kSplitF32, kSameType };
TwoStepForm two_step_form(int x_dtype, int y_dtype, uint32_t m, const WView& w, uint32_t x_stride) {
    if (m < kTwoStepMinRowsOtherwise) return TwoStepForm::kExactF32;
    if (x_dtype == MI355Q_F32 && y_dtype == MI355Q_F32 && w.k % 4 == 0 && x_stride % 4 == 0) return TwoStepForm::kSplitF32;
    return TwoStepForm::kSameType;
}
}  // namespace

bool gemm_two_step_serves(mi355q_context* ctx, const WView& w, int x_dtype, int y_dtype, uint32_t m, uint32_t x_stride,
                          uint32_t y_stride) {
    const uint32_t n = (uint32_t)w.n, k = (uint32_t)w.k;
    switch (two_step_form(x_dtype, y_dtype, m, w, x_stride)) {
    // (results of a padded stride are computed densely in scratch: the library is asked for stride N)
    case TwoStepForm::kExactF32:
        return dense_library_serves(ctx, MI355Q_F32, m, n, k, x_dtype == MI355Q_F32 ? x_stride : k, n, MI355Q_F32);
    case TwoStepForm::kSplitF32: return dense_library_serves(ctx, MI355Q_BF16, m, n, k, k, n, MI355Q_F32);
    default: return dense_library_serves(ctx, x_dtype, m, n, k, x_stride, n, y_dtype);
    }
}

// The library's product into a result whose row stride is not N: with long K (14336; not with 4224 or less) its
// split-K algorithms, the heuristic's first among them, return a wrong matrix into such a result (M = 128, N = 64 or
// 2056, fp32 and bf16, stride N + 5 or N + 8: every run, whatever the workspace holds before, and garbage placed in
// the workspace shows up in the result -- the sum of the parts reads with another row stride than they were written
// with), while results of stride N are right.  So a padded result is computed densely in scratch and copied row by
// row.  `free_ws` is scratch of dense_result_bytes() bytes; `x_second`, when given, is a second activation matrix
// whose product is added to the first's (the low halves of split fp32 rows).
size_t dense_result_bytes(uint32_t m, uint32_t n, uint32_t y_stride, int y_dtype) {
    return y_stride == n ? 0 : (((size_t)m * n * (y_dtype == MI355Q_F32 ? 4 : 2)) + 255) & ~(size_t)255;
}

mi355q_status dense_gemm_into(hipStream_t s, mi355q_context* ctx, int ab_dtype, const void* x, const void* w_dense, void* y,
                              int y_dtype, uint32_t m, uint32_t n, uint32_t k, uint32_t x_stride, uint32_t y_stride,
                              char* free_ws, const void* x_second = nullptr) {
    const size_t tmp_bytes = dense_result_bytes(m, n, y_stride, y_dtype);
    void* const out = tmp_bytes ? (void*)free_ws : y;
    const uint32_t out_stride = tmp_bytes ? n : y_stride;
    if (mi355q_status st = dense_library_gemm(s, ctx, ab_dtype, x, w_dense, out, y_dtype, m, n, k, x_stride, out_stride, false))
        return st;
    if (x_second)
        if (mi355q_status st = dense_library_gemm(s, ctx, ab_dtype, x_second, w_dense, out, y_dtype, m, n, k, x_stride, out_stride,
                                                  true)) return st;
    if (!tmp_bytes) return MI355Q_OK;
    const size_t ysz = y_dtype == MI355Q_F32 ? 4 : 2;
    for (uint32_t m0 = 0; m0 < m; m0 += 65535u) {
        const uint32_t rows = m - m0 < 65535u ? m - m0 : 65535u;
        if (mi355q_status st = launch_convert_rows(s, (const char*)out + (size_t)m0 * n * ysz, y_dtype, n,
                                                   (char*)y + (size_t)m0 * y_stride * ysz, y_dtype, y_stride, rows, n)) return st;
    }
    return MI355Q_OK;
}

// The dense matrix sits at the head of the context's scratch, converted activations and results behind it, the
// library's workspace last.
mi355q_status launch_qgemm_two_step(hipStream_t s, mi355q_context* ctx, const WView& w, const void* x, int x_dtype,
                                    void* y, int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride) {
    const uint32_t n = (uint32_t)w.n, k = (uint32_t)w.k;
    auto round256 = [](size_t b) { return (b + 255) & ~(size_t)255; };
    const TwoStepForm form = two_step_form(x_dtype, y_dtype, m, w, x_stride);
    if (form == TwoStepForm::kExactF32) {
        const bool widen = x_dtype != MI355Q_F32, narrow = y_dtype != MI355Q_F32;
        const size_t wbytes = round256((size_t)n * k * 4), xbytes = widen ? round256((size_t)m * k * 4) : 0;
        const size_t ybytes = narrow ? round256((size_t)m * n * 4) : 0;
        const size_t dense_y = narrow ? 0 : dense_result_bytes(m, n, y_stride, MI355Q_F32);
        if (mi355q_status st = ensure_workspace(ctx, wbytes + xbytes + ybytes + dense_y)) return st;
        char* const base = (char*)ctx->workspace;
        float* const w32 = (float*)base;
        float* const x32 = widen ? (float*)(base + wbytes) : (float*)const_cast<void*>(x);
        float* const y32 = narrow ? (float*)(base + wbytes + xbytes) : (float*)y;
        if (mi355q_status st = launch_dequant_f32(s, w, w32)) return st;
        if (widen)
            if (mi355q_status st = launch_convert_rows(s, x, x_dtype, x_stride, x32, MI355Q_F32, k, m, k)) return st;
        if (mi355q_status st = dense_gemm_into(s, ctx, MI355Q_F32, x32, w32, y32, MI355Q_F32, m, n, k, widen ? k : x_stride,
                                               narrow ? n : y_stride, base + wbytes + xbytes + ybytes)) return st;
        if (narrow) return launch_convert_rows(s, y32, MI355Q_F32, n, y, y_dtype, y_stride, m, n);
        return MI355Q_OK;
    }
    if (form == TwoStepForm::kSplitF32) {
        const size_t wbytes = round256((size_t)n * k * 2), xbytes = round256((size_t)m * k * 2);
        if (mi355q_status st = ensure_workspace(ctx, wbytes + 2 * xbytes + dense_result_bytes(m, n, y_stride, MI355Q_F32))) return st;
        char* const base = (char*)ctx->workspace;
        uint16_t* const w_bf16 = (uint16_t*)base;
        uint16_t* const hi = (uint16_t*)(base + wbytes);
        uint16_t* const lo = (uint16_t*)(base + wbytes + xbytes);
        if (mi355q_status st = launch_dequant_bf16(s, w, w_bf16)) return st;
        if (mi355q_status st = launch_split_f32_bf16x2(s, (const float*)x, m, k, x_stride, hi, lo)) return st;
        return dense_gemm_into(s, ctx, MI355Q_BF16, hi, w_bf16, y, MI355Q_F32, m, n, k, k, y_stride, base + wbytes + 2 * xbytes, lo);
    }
    const size_t esz = x_dtype == MI355Q_F32 ? 4 : 2;
    const size_t dense = round256((size_t)n * k * esz);
    if (mi355q_status st = ensure_workspace(ctx, dense + dense_result_bytes(m, n, y_stride, y_dtype))) return st;
    void* const w_dense = ctx->workspace;
    const mi355q_status st = x_dtype == MI355Q_BF16 ? launch_dequant_bf16(s, w, (uint16_t*)w_dense)
                           : x_dtype == MI355Q_F16 ? launch_dequant_f16(s, w, (uint16_t*)w_dense)
                                                   : launch_dequant_f32(s, w, (float*)w_dense);
    if (st != MI355Q_OK) return st;
    return dense_gemm_into(s, ctx, x_dtype, x, w_dense, y, y_dtype, m, n, k, x_stride, y_stride, (char*)ctx->workspace + dense);
}

// Two or three projections that read the same activations (q+k+v, gate+up).  For M <= 8 on the
// split-plane layout they run as ONE launch whose rows are the rows of all weights together;
// otherwise each projection keeps its own launch on the stream.  Output i has row stride N_i
// (Sources/MetalCompiler/Generator/MetalSourceGenerator+Quantized.swift:166-338).
mi355q_status dispatch_batched(mi355q_context* ctx, hipStream_t s, uint32_t count, const mi355q_weight* const* weights,
                               const void* x, int x_dtype, void* const* ys, int y_dtype, uint32_t m, uint32_t xs,
                               uint32_t flags) {
    if (count != 2 && count != 3)
        return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "batched projection count must be 2 or 3 (got %u)", count);
    if (!weights || !ys) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null weight or output array");
    for (uint32_t i = 0; i < count; i++) {
        if (!weights[i]) return fail(MI355Q_ERR_NULL_HANDLE, "weight handle %u is null", i);
        if (weights[i]->ctx != ctx)
            return fail(MI355Q_ERR_INVALID_ARGUMENT, "weight handle %u belongs to another context", i);
        if (weights[i]->k != weights[0]->k || weights[i]->fmt.scheme_identifier != weights[0]->fmt.scheme_identifier ||
            weights[i]->layout != weights[0]->layout)
            return fail(MI355Q_ERR_SHAPE, "batched projections must share K, scheme and layout");
    }
    WView views[3];
    uint32_t strides[3];
    for (uint32_t i = 0; i < count; i++) {
        uint32_t x_stride = xs, y_stride = 0;
        if (mi355q_status st = check_io(weights[i], x, x_dtype, ys[i], y_dtype, m, x_stride, y_stride)) return st;
        xs = x_stride;
        strides[i] = y_stride;
        views[i] = weights[i]->view();
    }
    switch (shared_route(ctx, count, views, x_dtype, m, xs, flags, (uintptr_t)x % 16 == 0)) {
    case SharedRoute::kStream:
        return launch_qgemm_stream_multi(s, ctx, count, views, x, x_dtype, ys, strides, y_dtype, m, xs);
    case SharedRoute::kMfmaPlanes:
        return launch_gemv_mfma_planes_multi(s, ctx, count, views, x, x_dtype, ys, strides, y_dtype, m, xs);
    case SharedRoute::kDotPlanes:
        return launch_gemv_fast_multi(s, ctx, count, views, x, x_dtype, ys, strides, y_dtype, m, xs, nullptr, nullptr, HeadKeys{});
    case SharedRoute::kTile16:
        return launch_gemv_tile16_multi(s, ctx, count, views, x, x_dtype, ys, strides, y_dtype, m, xs, nullptr, nullptr,
                                        HeadKeys{});
    case SharedRoute::kStafInPlace:
        return launch_gemv_staf_multi(s, ctx, count, views, x, x_dtype, ys, strides, y_dtype, m, xs, nullptr, nullptr, HeadKeys{});
    case SharedRoute::kWide:
        return launch_qgemm_wide_multi(s, ctx, count, views, x, x_dtype, ys, strides, y_dtype, m, xs);
    case SharedRoute::kSplitRows: {
        const uint32_t parts = split_rows_parts(x_dtype);
        const uint32_t k = (uint32_t)views[0].k, kp = split_rows_stride(k);
        const size_t xbytes = ((size_t)parts * m * kp * 2 + 255) & ~(size_t)255;
        size_t ybytes[3] = {0, 0, 0}, total = xbytes;
        for (uint32_t i = 0; i < count; i++) total += ybytes[i] = ((size_t)parts * m * views[i].n * 4 + 255) & ~(size_t)255;
        if (mi355q_status st = ensure_split_buffer(ctx, total)) return st;
        char* const base = (char*)ctx->split_buffer;
        void* yps[3] = {nullptr, nullptr, nullptr};
        size_t at = xbytes;
        for (uint32_t i = 0; i < count; i++) { yps[i] = base + at; at += ybytes[i]; }
        if (mi355q_status st = launch_split_rows_bf16(s, x, x_dtype, m, k, xs, (uint16_t*)base, kp)) return st;
        if (mi355q_status st = dispatch_batched(ctx, s, count, weights, base, MI355Q_BF16, yps, MI355Q_F32, parts * m, kp, flags))
            return st;
        for (uint32_t i = 0; i < count; i++)
            if (mi355q_status st = launch_sum_parts_rows(s, (const float*)yps[i], parts, m, (uint32_t)views[i].n, ys[i], y_dtype,
                                                         strides[i])) return st;
        return MI355Q_OK;
    }
    case SharedRoute::kSteps: {
        const uint32_t step = small_batch_rows(views[0], x_dtype, xs);
        const size_t xsz = x_dtype == MI355Q_F32 ? 4 : 2, ysz = y_dtype == MI355Q_F32 ? 4 : 2;
        for (uint32_t m0 = 0; m0 < m; m0 += step) {
            void* yc[3] = {nullptr, nullptr, nullptr};
            for (uint32_t i = 0; i < count; i++) yc[i] = (char*)ys[i] + (size_t)m0 * strides[i] * ysz;
            if (mi355q_status st = dispatch_batched(ctx, s, count, weights, (const char*)x + (size_t)m0 * xs * xsz, x_dtype, yc,
                                                    y_dtype, m - m0 < step ? m - m0 : step, xs, flags)) return st;
        }
        return MI355Q_OK;
    }
    case SharedRoute::kSeparate:
        break;
    }
    for (uint32_t i = 0; i < count; i++) {
        mi355q_status st = dispatch_linear(ctx, s, weights[i], x, x_dtype, ys[i], y_dtype, m, xs, 0, flags, false);
        if (st != MI355Q_OK) return st;
    }
    return MI355Q_OK;
}

// `keys`: kStaticHeadKeys or kArgmaxPartialCapacity keys for the fused head followed by kArgmaxStandaloneKeys for the
// two-launch arg-max (the context's allocation, or the device array of the entry point that allocates nothing).
mi355q_status dispatch_output_head(mi355q_context* ctx, hipStream_t s, const mi355q_weight* w, const void* x,
                                   int x_dtype, float* logits, int32_t* token, uint32_t flags, HeadKeys keys,
                                   bool no_allocation) {
    if (!x || !token) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null pointer");
    if (!dtype_ok(x_dtype)) return fail(MI355Q_ERR_INVALID_ARGUMENT, "bad dtype tag");
    const WView v = w->view();
    const uint32_t xs = (uint32_t)w->k;
    if (!(flags & MI355Q_FLAG_FORCE_GENERIC) && gemv_fast_eligible(v, x_dtype, 1, xs) && (uintptr_t)x % 16 == 0)
        return launch_gemv_fast(s, ctx, v, x, x_dtype, nullptr, MI355Q_F32, 1, xs, (uint32_t)w->n, logits, token,
                                keys);
    if (!(flags & MI355Q_FLAG_FORCE_GENERIC) && x_dtype == MI355Q_BF16 && gemv_tile16_eligible(v, x_dtype, 1, xs) &&
        gemv_tile16_k_parts(ctx, v, 1) == 1 && (uintptr_t)x % 16 == 0) {
        void* none[1] = {nullptr};
        const uint32_t strides[1] = {(uint32_t)w->n};
        return launch_gemv_tile16_multi(s, ctx, 1, &v, x, x_dtype, none, strides, MI355Q_F32, 1, xs, logits, token,
                                        keys);
    }
    if (!(flags & MI355Q_FLAG_FORCE_GENERIC) && gemv_staf_eligible(v, x_dtype, 1, xs) && (uintptr_t)x % 16 == 0) {
        void* none[1] = {nullptr};
        const uint32_t strides[1] = {(uint32_t)w->n};
        return launch_gemv_staf_multi(s, ctx, 1, &v, x, x_dtype, none, strides, MI355Q_F32, 1, xs, logits, token,
                                      keys);
    }
    // two dispatches, as the reference runs the head: projection to fp32 logits, then argmax
    if (!logits)
        return fail(MI355Q_ERR_INVALID_ARGUMENT,
                    "a logits buffer is required when the fused head kernel does not accept the shape");
    // fp32 activations (three bf16 rows on the bf16 decode kernel) and f16 ones on TILE16 records: the projection's own
    // route for one row (2048 -> 65536 with fp32 activations: the per-code kernel takes hundreds of microseconds)
    // (the routed projections keep scratch in the context, grown on demand: not for the entry point that allocates nothing)
    const bool routed = !no_allocation && !(flags & MI355Q_FLAG_FORCE_GENERIC) && (uintptr_t)x % 16 == 0 &&
                        (split_rows_chosen(v, x_dtype, 1, xs, flags) ||
                         (x_dtype == MI355Q_F16 && gemv_tile16_eligible(v, x_dtype, 1, xs)));
    mi355q_status st = routed ? dispatch_linear(ctx, s, w, x, x_dtype, logits, MI355Q_F32, 1, xs, (uint32_t)w->n, flags, true)
                              : launch_gemv_generic(s, v, x, x_dtype, logits, MI355Q_F32, 1, xs, (uint32_t)w->n);
    if (st != MI355Q_OK) return st;
    return launch_argmax(s, logits, MI355Q_F32, (uint32_t)w->n, token, keys.ptr + keys.capacity);
}

}  // namespace mi355q

extern "C" {

mi355q_status mi355q_qgemv(mi355q_context* ctx, void* stream, const mi355q_weight* w, const void* x_dev,
                           mi355q_dtype x_dtype, void* y_dev, mi355q_dtype y_dtype, uint32_t m,
                           uint32_t x_row_stride, uint32_t y_row_stride, uint32_t flags) {
    if (mi355q_status s = check_launch(ctx, w)) return s;
    ScratchGuard guard(ctx, (hipStream_t)stream);
    if (guard.status) return guard.status;
    return dispatch_linear(ctx, (hipStream_t)stream, w, x_dev, x_dtype, y_dev, y_dtype, m, x_row_stride,
                           y_row_stride, flags, true);
}

mi355q_status mi355q_qgemm(mi355q_context* ctx, void* stream, const mi355q_weight* w, const void* x_dev,
                           mi355q_dtype x_dtype, void* y_dev, mi355q_dtype y_dtype, uint32_t m,
                           uint32_t x_row_stride, uint32_t y_row_stride, uint32_t flags) {
    if (mi355q_status s = check_launch(ctx, w)) return s;
    ScratchGuard guard(ctx, (hipStream_t)stream);
    if (guard.status) return guard.status;
    return dispatch_linear(ctx, (hipStream_t)stream, w, x_dev, x_dtype, y_dev, y_dtype, m, x_row_stride,
                           y_row_stride, flags, false);
}

mi355q_status mi355q_batched_qgemm(mi355q_context* ctx, void* stream, uint32_t count,
                                   const mi355q_weight* const* weights, const void* x_dev, mi355q_dtype x_dtype,
                                   void* const* y_devs, mi355q_dtype y_dtype, uint32_t m, uint32_t x_row_stride,
                                   uint32_t flags) {
    if (!ctx) return fail(MI355Q_ERR_NULL_HANDLE, "context is null");
    MI355Q_HIP(hipSetDevice(ctx->device));
    ScratchGuard guard(ctx, (hipStream_t)stream);
    if (guard.status) return guard.status;
    return dispatch_batched(ctx, (hipStream_t)stream, count, weights, x_dev, x_dtype, y_devs, y_dtype, m,
                            x_row_stride, flags);
}

mi355q_status mi355q_dequant_bf16(mi355q_context* ctx, void* stream, const mi355q_weight* w, void* out_bf16_dev) {
    if (mi355q_status s = check_launch(ctx, w)) return s;
    if (!out_bf16_dev || (uintptr_t)out_bf16_dev % 2) return fail(MI355Q_ERR_INVALID_ARGUMENT, "bad output pointer");
    return launch_dequant_bf16((hipStream_t)stream, w->view(), (uint16_t*)out_bf16_dev);
}

mi355q_status mi355q_dequant_f32(mi355q_context* ctx, void* stream, const mi355q_weight* w, float* out_f32_dev) {
    if (mi355q_status s = check_launch(ctx, w)) return s;
    if (!out_f32_dev || (uintptr_t)out_f32_dev % 4) return fail(MI355Q_ERR_INVALID_ARGUMENT, "bad output pointer");
    return launch_dequant_f32((hipStream_t)stream, w->view(), out_f32_dev);
}

mi355q_status mi355q_gemm_bf16(mi355q_context* ctx, void* stream, const void* a_dev, mi355q_dtype a_dtype,
                               const void* b_bf16_dev, void* c_dev, mi355q_dtype c_dtype, uint32_t m, uint32_t n,
                               uint32_t k, uint32_t a_row_stride, uint32_t c_row_stride) {
    if (!ctx) return fail(MI355Q_ERR_NULL_HANDLE, "context is null");
    if (!a_dev || !b_bf16_dev || !c_dev) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null pointer");
    if (!dtype_ok(a_dtype) || !dtype_ok(c_dtype)) return fail(MI355Q_ERR_INVALID_ARGUMENT, "bad dtype tag");
    if (!m || !n || !k) return fail(MI355Q_ERR_SHAPE, "empty GEMM");
    if (a_row_stride == 0) a_row_stride = k;
    if (c_row_stride == 0) c_row_stride = n;
    if (a_row_stride < k || c_row_stride < n) return fail(MI355Q_ERR_SHAPE, "row stride smaller than the row");
    MI355Q_HIP(hipSetDevice(ctx->device));
    ScratchGuard guard(ctx, (hipStream_t)stream);
    if (guard.status) return guard.status;
    // long products go to the platform's GEMM library (the reference hands them to matmul2d), the rest to this
    // library's own matrix-core kernel
    if (a_dtype == MI355Q_BF16 && m >= kDenseLibraryMinRows && k % 8 == 0 && a_row_stride % 8 == 0 &&
        (uintptr_t)a_dev % 16 == 0 && (uintptr_t)b_bf16_dev % 16 == 0 &&
        dense_library_serves(ctx, MI355Q_BF16, m, n, k, a_row_stride, n, c_dtype)) {
        if (mi355q_status st = ensure_workspace(ctx, mi355q::dense_result_bytes(m, n, c_row_stride, c_dtype))) return st;
        const mi355q_status st = mi355q::dense_gemm_into((hipStream_t)stream, ctx, MI355Q_BF16, a_dev, b_bf16_dev, c_dev, c_dtype,
                                                         m, n, k, a_row_stride, c_row_stride, (char*)ctx->workspace);
        if (st != MI355Q_ERR_KERNEL_NOT_FOUND) return st;        // a library result that failed its check: this library's kernel
    }
    return launch_gemm_bf16_mfma((hipStream_t)stream, ctx, a_dev, a_dtype, (const uint16_t*)b_bf16_dev, c_dev,
                                 c_dtype, m, n, k, a_row_stride, c_row_stride);
}

mi355q_status mi355q_embedding_lookup(mi355q_context* ctx, void* stream, const mi355q_weight* table,
                                      const int32_t* token_ids_dev, uint32_t sequence_length, void* out_dev,
                                      mi355q_dtype out_dtype, uint32_t out_row_stride, int has_embedding_scale,
                                      float embedding_scale) {
    if (mi355q_status s = check_launch(ctx, table)) return s;
    if (!token_ids_dev || !out_dev) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null token or output pointer");
    if (!dtype_ok(out_dtype)) return fail(MI355Q_ERR_INVALID_ARGUMENT, "bad dtype tag");
    if (sequence_length == 0) return fail(MI355Q_ERR_INVALID_ARGUMENT, "sequence length must be >= 1");
    if (sequence_length > 65535) return fail(MI355Q_ERR_SHAPE, "sequence length %u exceeds 65535", sequence_length);
    if (out_row_stride == 0) out_row_stride = (uint32_t)table->k;
    if (out_row_stride < table->k) return fail(MI355Q_ERR_SHAPE, "output row stride smaller than embeddingDim");
    if ((uintptr_t)token_ids_dev % 4 || (uintptr_t)out_dev % (out_dtype == MI355Q_F32 ? 4 : 2))
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "misaligned pointer");
    return launch_embedding_lookup((hipStream_t)stream, table->view(), token_ids_dev, sequence_length, out_dev, out_dtype,
                                   out_row_stride, has_embedding_scale, embedding_scale);
}

mi355q_status mi355q_unpack_codes(mi355q_context* ctx, void* stream, const mi355q_weight* w,
                                  uint8_t* out_codes_dev) {
    if (mi355q_status s = check_launch(ctx, w)) return s;
    if (!out_codes_dev) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null output pointer");
    return launch_unpack_codes((hipStream_t)stream, w->view(), out_codes_dev);
}

mi355q_status mi355q_argmax(mi355q_context* ctx, void* stream, const void* logits_dev, mi355q_dtype dtype,
                            uint32_t vocabulary_size, int32_t* token_out_dev) {
    if (!ctx) return fail(MI355Q_ERR_NULL_HANDLE, "context is null");
    if (!logits_dev || !token_out_dev) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null pointer");
    if (!dtype_ok(dtype)) return fail(MI355Q_ERR_INVALID_ARGUMENT, "bad dtype tag");
    if (vocabulary_size == 0) return fail(MI355Q_ERR_SHAPE, "argmax over an empty vector");
    MI355Q_HIP(hipSetDevice(ctx->device));
    ScratchGuard guard(ctx, (hipStream_t)stream);
    if (guard.status) return guard.status;
    ctx->scratch_touched = true;                              // the keys of the stand-alone arg-max
    return launch_argmax((hipStream_t)stream, logits_dev, dtype, vocabulary_size, token_out_dev,
                         ctx->argmax_partials + kArgmaxPartialCapacity);
}

mi355q_status mi355q_lmhead_argmax(mi355q_context* ctx, void* stream, const mi355q_weight* w, const void* x_dev,
                                   mi355q_dtype x_dtype, float* logits_f32_dev, int32_t* token_out_dev,
                                   uint32_t flags) {
    if (mi355q_status s = check_launch(ctx, w)) return s;
    ScratchGuard guard(ctx, (hipStream_t)stream);
    if (guard.status) return guard.status;
    ctx->scratch_touched = true;                              // one key per workgroup of the head
    return dispatch_output_head(ctx, (hipStream_t)stream, w, x_dev, x_dtype, logits_f32_dev, token_out_dev, flags,
                                HeadKeys{ctx->argmax_partials, kArgmaxPartialCapacity});
}

// The same head with its partial keys in a device array of the library image instead of the context's allocation: no
// device memory is allocated or released on this path (the launches it makes need no workspace and no LDS opt-in).
mi355q_status mi355q_lmhead_argmax_static(mi355q_context* ctx, void* stream, const mi355q_weight* w, const void* x_dev,
                                          mi355q_dtype x_dtype, float* logits_f32_dev, int32_t* token_out_dev,
                                          uint32_t flags) {
    if (mi355q_status s = check_launch(ctx, w)) return s;
    unsigned long long* const keys = static_head_keys(ctx->device);
    if (!keys) return fail(MI355Q_ERR_DEVICE, "the static key array of device %d was not resolved", ctx->device);
    return dispatch_output_head(ctx, (hipStream_t)stream, w, x_dev, x_dtype, logits_f32_dev, token_out_dev, flags,
                                HeadKeys{keys, kStaticHeadKeys}, true);
}

uint32_t mi355q_lmhead_argmax_static_capacity(void) { return kStaticHeadKeys; }

mi355q_status mi355q_clock_probe_read(mi355q_context* ctx, uint64_t* shader_cycles, uint64_t* realtime_ticks) {
    if (!ctx) return fail(MI355Q_ERR_NULL_HANDLE, "context is null");
    if (!shader_cycles || !realtime_ticks) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null output");
    unsigned long long cell[2] = {0, 0};
    MI355Q_HIP(hipSetDevice(ctx->device));
    MI355Q_HIP(hipDeviceSynchronize());
    MI355Q_HIP(hipMemcpy(cell, ctx->argmax_scratch + 16, sizeof cell, hipMemcpyDeviceToHost));
    *shader_cycles = cell[0];
    *realtime_ticks = cell[1];
    return MI355Q_OK;
}

}  // extern "C"

// ---- gated MLP: gate_proj + up_proj + swiglu / gelu_gated --------------------------------------------------------
extern "C" mi355q_status mi355q_gated_activation_apply(mi355q_context* ctx, void* stream, const void* gate_dev,
                                                       const void* up_dev, void* out_dev, mi355q_dtype dtype,
                                                       uint32_t dimension, uint32_t sequence_length,
                                                       uint32_t row_stride, mi355q_gated_activation activation) {
    if (!ctx) return fail(MI355Q_ERR_NULL_HANDLE, "context is null");
    if (!gate_dev || !up_dev || !out_dev) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null buffer");
    if (!dtype_ok(dtype)) return fail(MI355Q_ERR_INVALID_ARGUMENT, "bad dtype tag");
    if (activation != MI355Q_GATED_SILU && activation != MI355Q_GATED_GELU_TANH)
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "unknown gated activation %d", (int)activation);
    if (dimension == 0 || sequence_length == 0) return fail(MI355Q_ERR_INVALID_ARGUMENT, "dimension and sequence length must be >= 1");
    if (row_stride == 0) row_stride = dimension;
    if (row_stride < dimension) return fail(MI355Q_ERR_SHAPE, "row stride %u < dimension %u", row_stride, dimension);
    hipError_t e = hipSetDevice(ctx->device);
    if (e != hipSuccess) return fail(MI355Q_ERR_DEVICE, "hipSetDevice failed: %s", hipGetErrorString(e));
    return launch_gated_activation((hipStream_t)stream, gate_dev, up_dev, out_dev, dtype, dimension, sequence_length, row_stride,
                                   row_stride, row_stride, activation);
}

namespace mi355q {
mi355q_status dispatch_gated(mi355q_context* ctx, hipStream_t s, const mi355q_weight* w_gate, const mi355q_weight* w_up,
                             const void* x_dev, int x_dtype, void* y_dev, int y_dtype, uint32_t m, uint32_t xs, uint32_t ys,
                             int activation, uint32_t flags) {
    if (activation != MI355Q_GATED_SILU && activation != MI355Q_GATED_GELU_TANH)
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "unknown gated activation %d", activation);
    if (w_gate->n != w_up->n || w_gate->k != w_up->k || w_gate->fmt.scheme_identifier != w_up->fmt.scheme_identifier ||
        w_gate->layout != w_up->layout)
        return fail(MI355Q_ERR_SHAPE, "gate and up projections must share N, K, scheme and layout");
    if (x_dtype == MI355Q_F32) return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the gated projection takes bf16 or f16 activations");
    if (mi355q_status st = check_io(w_gate, x_dev, x_dtype, y_dev, y_dtype, m, xs, ys)) return st;
    const WView g = w_gate->view(), u = w_up->view();
    const uint32_t n = (uint32_t)w_gate->n;
    if (!(flags & (MI355Q_FLAG_FORCE_GENERIC | MI355Q_FLAG_FORCE_SMALL_M | MI355Q_FLAG_FORCE_MFMA | MI355Q_FLAG_FORCE_TWO_STEP |
                   MI355Q_FLAG_FORCE_STREAM)) &&
        gemv_gated_eligible(ctx, g, u, x_dtype, m, xs) && (uintptr_t)x_dev % 16 == 0)
        return launch_gemv_gated(s, ctx, g, u, x_dev, x_dtype, y_dev, y_dtype, xs, activation);
    // prompts on 4-bit weights: the wide-tile matrix-core kernel with the activation as its epilogue
    if (gemm_wide_gated_taken(ctx, g, u, x_dtype, m, xs, flags) && (uintptr_t)x_dev % 16 == 0)
        return launch_qgemm_wide_gated(s, ctx, g, u, x_dev, x_dtype, y_dev, y_dtype, m, xs, ys, activation);
    // a few dozen rows: the streamed-weight kernel, gate_proj and up_proj as the two row blocks of every workgroup
    if (gemm_stream_gated_taken(ctx, g, u, x_dtype, m, xs, flags) && (uintptr_t)x_dev % 16 == 0)
        return launch_qgemm_stream_gated(s, ctx, g, u, x_dev, x_dtype, y_dev, y_dtype, m, xs, ys, activation);
    // elsewhere: the two projections as the batched entry point runs them, into scratch of the context, then the
    // elementwise kernel (the reference's own sequence of dispatches)
    const size_t esz = y_dtype == MI355Q_F32 ? 4 : 2;
    const size_t half = ((size_t)m * n * esz + 255) & ~(size_t)255;
    if (mi355q_status st = ensure_gated_buffer(ctx, 2 * half)) return st;
    void* const gate_out = ctx->gated_buffer;
    void* const up_out = (char*)ctx->gated_buffer + half;
    const mi355q_weight* ws[2] = {w_gate, w_up};
    void* ys2[2] = {gate_out, up_out};
    if (mi355q_status st = dispatch_batched(ctx, s, 2, ws, x_dev, x_dtype, ys2, y_dtype, m, xs, flags)) return st;
    return launch_gated_activation(s, gate_out, up_out, y_dev, y_dtype, n, m, n, n, ys, activation);
}
}  // namespace mi355q

extern "C" mi355q_status mi355q_gated_qgemm(mi355q_context* ctx, void* stream, const mi355q_weight* w_gate,
                                            const mi355q_weight* w_up, const void* x_dev, mi355q_dtype x_dtype,
                                            void* y_dev, mi355q_dtype y_dtype, uint32_t m, uint32_t x_row_stride,
                                            uint32_t y_row_stride, mi355q_gated_activation activation, uint32_t flags) {
    if (mi355q_status st = check_launch(ctx, w_gate)) return st;
    if (mi355q_status st = check_launch(ctx, w_up)) return st;
    ScratchGuard guard(ctx, (hipStream_t)stream);
    if (guard.status) return guard.status;
    return dispatch_gated(ctx, (hipStream_t)stream, w_gate, w_up, x_dev, x_dtype, y_dev, y_dtype, m, x_row_stride, y_row_stride,
                          activation, flags);
}
