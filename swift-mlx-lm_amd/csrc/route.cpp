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
