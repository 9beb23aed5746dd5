// The table of routes: one function from (layout and format of the weight, activation type, rows, row stride, flags) to the
// route a linear projection takes, shared by the launcher (dispatch_linear, run_small_m in api.hip) and the planner
// (planner.cpp).  Stands in for the selection logic the reference spreads over its step builders
// (Sources/MetalCompiler/Compiler/MetalPrefillStepBuilder.swift:463-742, MetalDispatchStepBuilder.swift:640-689,
// Generator/MetalKernelNameResolver.swift:26-140).  The thresholds inside the predicates are measured crossovers,
// stated where each predicate is defined.
#include "common.h"

namespace mi355q {

LinearRoute linear_route(const WView& v, int x_dtype, uint32_t m, uint32_t xs, uint32_t flags, const RouteFacts& f) {
    if (f.decode_entry) {
        if (m > 8) return LinearRoute::kErrorRows;
        if (split_rows_chosen(v, x_dtype, m, xs, flags)) return LinearRoute::kSplitRows;
        // no decode kernel reads this layout with this activation type: dequantise once + the dense library product
        if (gemm_two_step_chosen(v, x_dtype, m, xs, flags) && f.x_aligned && f.library_ok) return LinearRoute::kTwoStep;
        if (!(flags & (MI355Q_FLAG_FORCE_GENERIC | MI355Q_FLAG_FORCE_SMALL_M)) && gemm_stream_chosen(v, x_dtype, m, xs) &&
            gemm_stream_unrounded(v, m) && f.x_aligned)
            return LinearRoute::kStream;
        return LinearRoute::kSmallBatch;
    }
    const uint32_t forced = flags & (MI355Q_FLAG_FORCE_MFMA | MI355Q_FLAG_FORCE_TWO_STEP | MI355Q_FLAG_FORCE_SMALL_M |
                                     MI355Q_FLAG_FORCE_GENERIC);
    if ((forced & (MI355Q_FLAG_FORCE_MFMA | MI355Q_FLAG_FORCE_TWO_STEP)) && (forced & (forced - 1))) return LinearRoute::kErrorFlags;
    if (flags & MI355Q_FLAG_FORCE_STREAM) return forced ? LinearRoute::kErrorFlags : LinearRoute::kStream;
    if (flags & MI355Q_FLAG_FORCE_TWO_STEP)
        return (!gemm_two_step_eligible(v, x_dtype, m, xs) || !f.x_aligned) ? LinearRoute::kErrorTwoStepUnavailable : LinearRoute::kTwoStep;
    if (split_rows_chosen(v, x_dtype, m, xs, flags)) return LinearRoute::kSplitRows;
    // dequantise once, then the dense library GEMM: very long prompts, and every format or layout the fused kernels do not read
    if (gemm_two_step_chosen(v, x_dtype, m, xs, flags) && f.x_aligned && f.library_ok) return LinearRoute::kTwoStep;
    const bool fused_ok = gemm_mfma_eligible(v, x_dtype, m, xs) || gemm_wide_taken(v, x_dtype, m, xs, flags);
    if (flags & MI355Q_FLAG_FORCE_MFMA) return fused_ok ? LinearRoute::kFused : LinearRoute::kErrorNoFusedKernel;
    // a few dozen rows on 4- and 8-bit planes and blocks
    if (!forced && gemm_stream_chosen(v, x_dtype, m, xs) && f.x_aligned) return LinearRoute::kStream;
    // the decode kernels take up to 8 rows per launch, 16 on the matrix cores (and then pay for a second launch too)
    const bool small = (flags & (MI355Q_FLAG_FORCE_SMALL_M | MI355Q_FLAG_FORCE_GENERIC)) ||
                       m <= small_batch_limit(v, x_dtype, xs) || !fused_ok;
    return small ? LinearRoute::kSmallBatch : LinearRoute::kFused;
}

const char* linear_route_name(LinearRoute r) {
    switch (r) {
    case LinearRoute::kErrorRows: return "error:rows";
    case LinearRoute::kErrorFlags: return "error:flags";
    case LinearRoute::kErrorTwoStepUnavailable: return "error:two-step";
    case LinearRoute::kErrorNoFusedKernel: return "error:fused";
    case LinearRoute::kSplitRows: return "split-rows";
    case LinearRoute::kTwoStep: return "two-step";
    case LinearRoute::kStream: return "stream";
    case LinearRoute::kSmallBatch: return "small-batch";
    case LinearRoute::kFused: return "fused";
    }
    return "?";
}

SmallKernel small_kernel(const WView& v, int x_dtype, uint32_t rows, uint32_t xs, uint32_t flags, bool x_aligned) {
    const bool generic = (flags & MI355Q_FLAG_FORCE_GENERIC) || !x_aligned;
    if (generic) return SmallKernel::kGeneric;
    if (gemv_tile16_eligible(v, x_dtype, rows, xs)) return SmallKernel::kTile16;
    if (mfma_planes_pays(v.bits, x_dtype, rows) && gemv_mfma_planes_eligible(v, x_dtype, rows, xs) &&
        !(gemv_rows_batch_pays(1, &v, x_dtype, rows) && gemv_fast_eligible(v, x_dtype, rows, xs)))
        return SmallKernel::kMfmaPlanes;
    if (gemv_fast_eligible(v, x_dtype, rows > 8 ? 8 : rows, xs)) return SmallKernel::kDotPlanes;
    if (gemv_staf_eligible(v, x_dtype, rows, xs)) return SmallKernel::kStafInPlace;
    return SmallKernel::kGeneric;
}

// Rows one launch of the small-batch route takes: sixteen on the matrix-core decode kernels (fewer on TILE16 records when
// K is so long that sixteen staged rows overflow LDS), eight on the dot-product kernels, all of them on the per-code kernel.
uint32_t small_batch_step(const WView& v, int x_dtype, uint32_t m, uint32_t xs, uint32_t flags) {
    const bool generic = flags & MI355Q_FLAG_FORCE_GENERIC;
    const uint32_t all = m < 65535u ? m : 65535u;
    uint32_t step = generic ? 8 : small_batch_rows(v, x_dtype, xs);
    if (!generic && v.layout == MI355Q_LAYOUT_TILE16) {
        step = 16;
        while (step > 1 && !gemv_tile16_eligible(v, x_dtype, step, xs)) step >>= 1;
        // no row count the tile kernel takes (other activation type, stride): the per-code kernel takes all M at once
        if (!gemv_tile16_eligible(v, x_dtype, step, xs)) step = all;
    } else if (generic || !(gemv_fast_eligible(v, x_dtype, 1, xs) || gemv_staf_eligible(v, x_dtype, 1, xs))) {
        step = all;                      // the per-code kernel has no limit of 8 rows
    }
    return step ? step : 1;
}

SharedRoute shared_route(const mi355q_context* ctx, uint32_t count, const WView* views, int x_dtype, uint32_t m, uint32_t xs,
                         uint32_t flags, bool x_aligned) {
    // a forced route is each projection's own affair (honoured or refused there), except the streamed-weight kernel
    // where it takes the matrices together
    if (flags & MI355Q_FLAG_FORCE_TWO_STEP) return SharedRoute::kSeparate;
    if (flags & MI355Q_FLAG_FORCE_STREAM)
        return x_aligned && gemm_stream_multi_eligible(count, views, x_dtype, m, xs) ? SharedRoute::kStream : SharedRoute::kSeparate;
    const bool decode_kernels = !(flags & (MI355Q_FLAG_FORCE_GENERIC | MI355Q_FLAG_FORCE_MFMA));
    bool fused = m <= 8 && decode_kernels, tiled = m <= 16 && decode_kernels, in_place = m <= 8 && decode_kernels;
    bool on_planes = mfma_planes_pays(views[0].bits, x_dtype, m) && m <= 16 && decode_kernels;
    for (uint32_t i = 0; i < count; i++) {
        const WView& v = views[i];
        fused = fused && gemv_fast_eligible(v, x_dtype, m, xs) && v.sb_dtype == views[0].sb_dtype;
        tiled = tiled && gemv_tile16_eligible(v, x_dtype, m, xs) && gemv_tile16_k_parts(ctx, v, staged_rows(x_dtype, m)) == 1 &&
                v.sb_dtype == views[0].sb_dtype;
        in_place = in_place && gemv_staf_eligible(v, x_dtype, m, xs);
        on_planes = on_planes && gemv_mfma_planes_eligible(v, x_dtype, m, xs) &&
                    gemv_mfma_planes_k_parts(ctx, v, staged_rows(x_dtype, m)) == 1 && v.sb_dtype == views[0].sb_dtype &&
                    v.code_stride == views[0].code_stride && v.group == views[0].group;
    }
    if (fused && gemv_rows_batch_pays(count, views, x_dtype, m)) on_planes = false;      // small matrices, three or four rows
    // the streamed-weight kernel, one launch for the two or three matrices: a few dozen rows on 4- / 8-bit planes, and
    // blocks in place from three to nine rows by the size of the matrices together
    const bool no_stream = flags & (MI355Q_FLAG_FORCE_GENERIC | MI355Q_FLAG_FORCE_MFMA | MI355Q_FLAG_FORCE_SMALL_M);
    if (!no_stream && x_aligned && gemm_stream_chosen_multi(count, views, x_dtype, m, xs)) return SharedRoute::kStream;
    if (x_aligned) {
        if (on_planes) return SharedRoute::kMfmaPlanes;
        if (fused) return SharedRoute::kDotPlanes;
        if (tiled) return SharedRoute::kTile16;
        if (in_place) return SharedRoute::kStafInPlace;
    }
    // prompts: the wide-tile prefill kernel over the column tiles of all matrices, where it would take one matrix of
    // their columns together (and the dense library is not the route: from kWideRowsBesideLibrary rows)
    if (x_aligned && !(flags & (MI355Q_FLAG_FORCE_GENERIC | MI355Q_FLAG_FORCE_MFMA | MI355Q_FLAG_FORCE_SMALL_M | MI355Q_FLAG_PROBE_TILED))) {
        if (flags & MI355Q_FLAG_PROBE_WIDE) {
            if (gemm_wide_multi_eligible(count, views, x_dtype, m, xs)) return SharedRoute::kWide;
        } else if (gemm_wide_multi_chosen(count, views, x_dtype, m, xs) && (m < kWideRowsBesideLibrary || library_ruled_out(ctx))) {
            return SharedRoute::kWide;
        }
    }
    // fp32 rows that go to the bf16 kernels as bf16 rows (split_rows_chosen): split once for all projections, one
    // shared bf16 launch on those rows where they fit one, one sum per projection
    const uint32_t parts = split_rows_parts(x_dtype);
    bool split = parts && parts * (uint64_t)m <= 16;
    for (uint32_t i = 0; i < count && split; i++) split = split_rows_chosen(views[i], x_dtype, m, xs, flags);
    if (split) return SharedRoute::kSplitRows;
    // more rows than one shared launch takes, served by the small-batch kernels all the same: the shared launch in steps
    const uint32_t step = small_batch_rows(views[0], x_dtype, xs);
    bool stepped = m > step && !(flags & (MI355Q_FLAG_FORCE_GENERIC | MI355Q_FLAG_FORCE_MFMA | MI355Q_FLAG_FORCE_TWO_STEP));
    for (uint32_t i = 0; i < count && stepped; i++)
        stepped = decode_kernel_reads(views[i], x_dtype, xs) && !split_rows_chosen(views[i], x_dtype, m, xs, flags) &&
                  !gemm_two_step_chosen(views[i], x_dtype, m, xs, flags) &&
                  (m <= small_batch_limit(views[i], x_dtype, xs) ||
                   !(gemm_mfma_eligible(views[i], x_dtype, m, xs) || gemm_wide_taken(views[i], x_dtype, m, xs, flags)));
    return stepped ? SharedRoute::kSteps : SharedRoute::kSeparate;
}

const char* shared_route_name(SharedRoute r) {
    switch (r) {
    case SharedRoute::kStream: return "shared/stream";
    case SharedRoute::kMfmaPlanes: return "shared/mfma-planes";
    case SharedRoute::kDotPlanes: return "shared/dot-planes";
    case SharedRoute::kTile16: return "shared/tile16";
    case SharedRoute::kStafInPlace: return "shared/staf-in-place";
    case SharedRoute::kWide: return "shared/wide";
    case SharedRoute::kSplitRows: return "split-rows";
    case SharedRoute::kSteps: return "steps";
    case SharedRoute::kSeparate: return "separate";
    }
    return "?";
}

const char* small_kernel_name(SmallKernel k) {
    switch (k) {
    case SmallKernel::kTile16: return "tile16";
    case SmallKernel::kMfmaPlanes: return "mfma-planes";
    case SmallKernel::kDotPlanes: return "dot-planes";
    case SmallKernel::kStafInPlace: return "staf-in-place";
    case SmallKernel::kGeneric: return "generic";
    }
    return "?";
}

}  // namespace mi355q
