// Planner mirror: launch-shape families, kernel selection and the quantization-plan record.
// Reference: Sources/MetalCompiler/Compiler/MetalCompileContext.swift:5-90,246-260 (shape
// families and GEMV grid), MetalDispatchStepBuilder.swift:640-689 (decode step),
// MetalPrefillStepBuilder.swift:463-742,1866-1893 (prefill steps and fallback reasons),
// MetalQuantizationPlan.swift:290-318 (plan entry).
#include "common.h"

using namespace mi355q;

namespace {

struct Family {
    int32_t id;
    uint32_t simdgroups, tile;
    const char* base;
};

// DecodeProjectionShapeFamily.resolve + preferredSimdgroups + tileElements + kernelBaseName
Family resolve_family(uint32_t n, uint32_t k) {
    if (n >= 65536 && k == 2048) return {MI355Q_FAMILY_VOCAB_DENSE, 16, 2048, "gemv_vocab"};
    if (k == 2048 && n == 2048) return {MI355Q_FAMILY_INPUT2048_SQUARE, 8, 2048, "gemv_2048_sq"};
    if (k == 2048 && n == 6144) return {MI355Q_FAMILY_INPUT2048_6144, 4, 2048, "gemv_2048_6144"};
    if (k == 2048 && n == 8192) return {MI355Q_FAMILY_INPUT2048_8192, 8, 2048, "gemv_2048_8192"};
    if (k == 2048 && n > 2048 && n < 65536) return {MI355Q_FAMILY_INPUT2048_EXPANDED, 8, 2048, "gemv_2048"};
    if (k == 8192 && n >= 2048 && n < 65536) return {MI355Q_FAMILY_INPUT8192_TILED, 8, 1024, "gemv_8192_tiled"};
    if (n >= 32768 && k >= 2048) return {MI355Q_FAMILY_LARGE_DENSE, 8, 512, "gemv_large"};
    return {MI355Q_FAMILY_GENERIC, 4, 256, "gemv"};
}

void fill_common(const mi355q_weight* w, uint32_t m, mi355q_step* s) {
    std::memset(s, 0, sizeof *s);
    const Family f = resolve_family((uint32_t)w->n, (uint32_t)w->k);
    s->shape_family = f.id;
    s->reference_simdgroups = f.simdgroups;
    s->reference_tile_elements = f.tile;
    s->scheme_identifier = w->fmt.scheme_identifier;
    s->layout = w->layout;
    s->input_dimension = (uint32_t)w->k;
    s->output_dimension = (uint32_t)w->n;
    s->sequence_length = m;
    s->weight_bytes = w->n * (w->k / w->fmt.group_size) * w->fmt.bytes_per_block;
    s->flops = 2ull * m * w->k * w->n;
    s->grid[1] = s->grid[2] = s->block[1] = s->block[2] = 1;
}

// Launch record of the decode kernel a small batch runs on: the first slice of the rows, as run_small_m (api.hip)
// cuts them (small_batch_step), on the kernel small_kernel() names.
void plan_small_kernel(const mi355q_weight* w, uint32_t m, int x_dtype, uint32_t x_stride, uint32_t flags, mi355q_step* s) {
    const WView v = w->view();
    const uint32_t step = small_batch_step(v, x_dtype, m, x_stride, flags);
    const uint32_t rows = m < step ? m : step;
    switch (small_kernel(v, x_dtype, rows, x_stride, flags, true)) {
    case SmallKernel::kTile16: {
        const Tile16LaunchShape g = gemv_tile16_shape(w->ctx, (uint32_t)((w->n + 15) / 16), (uint32_t)w->k, staged_rows(x_dtype, rows));
        std::snprintf(s->device_kernel, sizeof s->device_kernel, "gemv_tile16_q%u_g%u", (unsigned)w->fmt.bits, w->fmt.group_size);
        s->grid[0] = g.grid;
        s->block[0] = g.block;
        s->lds_bytes = g.lds_bytes;
        s->rows_per_workgroup = 16;
        return;
    }
    case SmallKernel::kMfmaPlanes: {
        const Tile16LaunchShape g = gemv_mfma_planes_shape(w->ctx, (uint32_t)((w->n + 15) / 16), (uint32_t)w->k,
                                                           (uint32_t)w->fmt.bits, staged_rows(x_dtype, rows));
        std::snprintf(s->device_kernel, sizeof s->device_kernel, "gemv_mfma_planes_q%u_g%u", (unsigned)w->fmt.bits, w->fmt.group_size);
        s->grid[0] = g.wgs_per_part;
        s->grid[1] = g.parts;
        s->block[0] = g.block;
        s->lds_bytes = g.lds_bytes;
        s->rows_per_workgroup = 16 * g.tiles_per_wg * g.passes;
        return;
    }
    case SmallKernel::kDotPlanes: {
        const GemvLaunchShape g = gemv_fast_shape(w->ctx, v, rows > 8 ? 8 : rows, x_dtype);
        std::snprintf(s->device_kernel, sizeof s->device_kernel, "%s_q%u_g%u",
                      std::strcmp(g.kernel, "gemv_rows_kernel") == 0 ? "gemv_rows" : "gemv_planes", (unsigned)w->fmt.bits,
                      w->fmt.group_size);
        s->grid[0] = g.grid;
        s->block[0] = g.block;
        s->lds_bytes = g.lds_bytes;
        s->rows_per_workgroup = g.rows_per_workgroup;
        return;
    }
    case SmallKernel::kStafInPlace: {
        const GemvLaunchShape g = gemv_staf_shape(w->ctx, v, rows > 8 ? 8 : rows);
        std::snprintf(s->device_kernel, sizeof s->device_kernel, "gemv_staf_q%u_g%u", (unsigned)w->fmt.bits, w->fmt.group_size);
        s->grid[0] = g.grid;
        s->block[0] = g.block;
        s->lds_bytes = g.lds_bytes;
        s->rows_per_workgroup = g.rows_per_workgroup;
        return;
    }
    default:
        std::snprintf(s->device_kernel, sizeof s->device_kernel, "gemv_generic");
        s->grid[0] = (uint32_t)((w->n + 3) / 4);
        s->grid[1] = m;
        s->block[0] = 256;
        s->rows_per_workgroup = 4;
        s->used_fallback = 1;
        s->fallback_reason = (flags & MI355Q_FLAG_FORCE_GENERIC) ? MI355Q_FALLBACK_DISABLED_BY_ENVIRONMENT
                                                                 : MI355Q_FALLBACK_UNAVAILABLE_ACCELERATION;
        return;
    }
}

void plan_stream(const mi355q_weight* w, uint32_t rows, const char* prefix, mi355q_step* s) {
    const StreamLaunchShape g = gemm_stream_shape(w->ctx, rows, (uint32_t)w->n, (uint32_t)w->k);
    std::snprintf(s->device_kernel, sizeof s->device_kernel, "%sqgemm_stream_q%u_g%u", prefix, (unsigned)w->fmt.bits, w->fmt.group_size);
    s->grid[0] = g.row_blocks;
    s->grid[1] = g.parts;
    s->block[0] = 768;
    s->lds_bytes = g.lds_bytes;
    s->rows_per_workgroup = 64;
}

// Record of a route that runs on the decode kernels or beside them (what dispatch_linear does for the same route).
void plan_small_m(const mi355q_weight* w, uint32_t m, int x_dtype, uint32_t x_stride, uint32_t flags, LinearRoute route,
                  mi355q_step* s) {
    const WView v = w->view();
    switch (route) {
    case LinearRoute::kSplitRows:
        if (!(flags & (MI355Q_FLAG_FORCE_GENERIC | MI355Q_FLAG_FORCE_SMALL_M)) && split_rows_take_stream(v, x_dtype, m)) {
            // fp32 rows as three bf16 rows each on the streamed-weight kernel, then the sum of the partial results
            plan_stream(w, split_rows_parts(x_dtype) * m, "split_f32_bf16x3+", s);
        } else {
            // ... on the bf16 decode kernel
            plan_small_kernel(w, split_rows_parts(x_dtype) * m, MI355Q_BF16, split_rows_stride((uint32_t)w->k), flags, s);
            char inner[sizeof s->device_kernel];
            std::snprintf(inner, sizeof inner, "%s", s->device_kernel);
            std::snprintf(s->device_kernel, sizeof s->device_kernel, "split_f32_bf16x3+%.30s", inner);
        }
        return;
    case LinearRoute::kStream:
        plan_stream(w, m, "", s);      // blocks in place from three rows: the streamed-weight kernel with unrounded weights
        return;
    case LinearRoute::kTwoStep:
        // no decode kernel reads this layout with this activation type: dequantise once + the dense library product
        // a few rows: fp32 weights and an fp32 product whatever the activation type (the decode kernels' arithmetic)
        std::snprintf(s->device_kernel, sizeof s->device_kernel, "dequant_q%u_g%u_f32+hipblaslt_gemm_f32", (unsigned)w->fmt.bits,
                      w->fmt.group_size);
        std::snprintf(s->kernel_family, sizeof s->kernel_family, "libraryGEMM");
        s->block[0] = 256;
        return;
    default:
        plan_small_kernel(w, m, x_dtype, x_stride, flags, s);
        return;
    }
}

}  // namespace

namespace mi355q {

// Launch record of a shared launch (2 or 3 projections, one set of activations), where shared_route() gives the
// projections one: the rows of all matrices together on the kernel it names.  Other routes leave the record of the
// first projection as it is.
void plan_shared_launch_shape(const mi355q_weight* const* ws, uint32_t count, uint32_t m, int x_dtype, uint32_t x_stride,
                              uint32_t flags, mi355q_step* s) {
    if (count < 2 || count > 3) return;
    WView views[3];
    uint64_t total = 0;
    uint32_t tiles = 0, row_blocks = 0;
    for (uint32_t i = 0; i < count; i++) {
        views[i] = ws[i]->view();
        total += views[i].n;
        tiles += (views[i].n + 15) / 16;
        row_blocks += (views[i].n + 63) / 64;
    }
    if (total > 0xFFFFFFFFull) return;
    const mi355q_context* const ctx = ws[0]->ctx;
    const unsigned bits = (unsigned)ws[0]->fmt.bits, group = ws[0]->fmt.group_size;
    switch (shared_route(ctx, count, views, x_dtype, m, x_stride, flags, true)) {
    case SharedRoute::kStream: {
        const StreamLaunchShape g = gemm_stream_shape_blocks(ctx, m, row_blocks, views[0].k);
        std::snprintf(s->device_kernel, sizeof s->device_kernel, "qgemm_stream_q%u_g%u", bits, group);
        s->grid[0] = g.row_blocks;
        s->grid[1] = g.parts;
        s->block[0] = 768;
        s->lds_bytes = g.lds_bytes;
        s->rows_per_workgroup = 64;
        return;
    }
    case SharedRoute::kWide: {
        const GemmLaunchShape g = gemm_wide_multi_shape(count, views, m, x_dtype);
        std::snprintf(s->device_kernel, sizeof s->device_kernel, "%sqgemm_wide_q%u_g%u", x_dtype == MI355Q_F32 ? "split_f32_bf16x2+" : "",
                      bits, group);
        s->grid[0] = g.grid;
        s->grid[1] = 1;
        s->block[0] = g.block;
        s->lds_bytes = g.lds_bytes;
        s->rows_per_workgroup = g.bn;
        s->used_fallback = 0;
        return;
    }
    case SharedRoute::kMfmaPlanes: {
        const Tile16LaunchShape g = gemv_mfma_planes_shape(ctx, tiles, views[0].k, views[0].bits, staged_rows(x_dtype, m));
        std::snprintf(s->device_kernel, sizeof s->device_kernel, "gemv_mfma_planes_q%u_g%u", bits, group);
        s->grid[0] = g.wgs_per_part;
        s->grid[1] = g.parts;
        s->block[0] = g.block;
        s->lds_bytes = g.lds_bytes;
        s->rows_per_workgroup = 16 * g.tiles_per_wg * g.passes;
        return;
    }
    case SharedRoute::kDotPlanes: {
        WView all = views[0];
        all.n = (uint32_t)total;
        const GemvLaunchShape g = gemv_fast_shape(ctx, all, m, x_dtype);
        std::snprintf(s->device_kernel, sizeof s->device_kernel, "%s_q%u_g%u",
                      std::strcmp(g.kernel, "gemv_rows_kernel") == 0 ? "gemv_rows" : "gemv_planes", bits, group);
        s->grid[0] = g.grid;
        s->block[0] = g.block;
        s->lds_bytes = g.lds_bytes;
        s->rows_per_workgroup = g.rows_per_workgroup;
        return;
    }
    case SharedRoute::kTile16: {
        const Tile16LaunchShape g = gemv_tile16_shape(ctx, tiles, views[0].k, staged_rows(x_dtype, m));
        std::snprintf(s->device_kernel, sizeof s->device_kernel, "gemv_tile16_q%u_g%u", bits, group);
        s->grid[0] = g.grid;
        s->block[0] = g.block;
        s->lds_bytes = g.lds_bytes;
        s->rows_per_workgroup = 16;
        return;
    }
    case SharedRoute::kStafInPlace: {
        WView all = views[0];
        all.n = (uint32_t)total;
        const GemvLaunchShape g = gemv_staf_shape(ctx, all, m);
        std::snprintf(s->device_kernel, sizeof s->device_kernel, "gemv_staf_q%u_g%u", bits, group);
        s->grid[0] = g.grid;
        s->block[0] = g.block;
        s->lds_bytes = g.lds_bytes;
        s->rows_per_workgroup = g.rows_per_workgroup;
        return;
    }
    default:
        return;
    }
}

}  // namespace mi355q

namespace {
// A weight handle that describes a tensor without holding one (aligned addresses that are never read), on a context
// of 256 CUs: enough for the route table and the planner.
void synthetic_weight(mi355q_context* ctx, mi355q_weight* w, const mi355q_format* f, uint32_t layout, uint32_t sb_dtype,
                      uint64_t n_rows, uint64_t k, bool library_available) {
    std::memset((void*)ctx, 0, sizeof *ctx);
    ctx->props.multiProcessorCount = 256;
    ctx->dense_library_forbidden = !library_available;
    std::memset((void*)w, 0, sizeof *w);
    w->ctx = ctx;
    w->fmt = *f;
    w->n = n_rows; w->k = k;
    w->layout = (uint8_t)layout;
    w->sb_dtype = layout == MI355Q_LAYOUT_STAF_BLOCKS ? (uint8_t)MI355Q_F16 : (uint8_t)sb_dtype;
    uint32_t* const fake = (uint32_t*)(uintptr_t)0x10000000;     // aligned, never read
    const uint32_t wpr = (uint32_t)(k * f->bits / 32), bpr = (uint32_t)(k / f->group_size);
    if (layout == MI355Q_LAYOUT_STAF_BLOCKS) w->blocks = fake;
    else if (layout == MI355Q_LAYOUT_TILE16) w->tiles = fake;
    else {
        w->codes = fake; w->sz = fake + wpr; w->scales = fake; w->biases = fake;
        w->code_stride = w->sz_stride = (wpr + bpr + 3u) & ~3u;
    }
}
}  // namespace

extern "C" {

mi355q_status mi355q_shape_family_resolve(uint32_t output_dimension, uint32_t input_dimension, int32_t* out_family,
                                          uint32_t* out_simdgroups, uint32_t* out_tile_elements,
                                          char* out_kernel_base_name, size_t name_cap) {
    const Family f = resolve_family(output_dimension, input_dimension);
    if (out_family) *out_family = f.id;
    if (out_simdgroups) *out_simdgroups = f.simdgroups;
    if (out_tile_elements) *out_tile_elements = f.tile;
    if (out_kernel_base_name && name_cap) std::snprintf(out_kernel_base_name, name_cap, "%s", f.base);
    return MI355Q_OK;
}

mi355q_status mi355q_plan_decode_step(const mi355q_weight* w, uint32_t m, mi355q_dtype x_dtype, uint32_t flags,
                                      mi355q_step* out) {
    if (!w) return fail(MI355Q_ERR_NULL_HANDLE, "weight handle is null");
    if (!out) return fail(MI355Q_ERR_INVALID_ARGUMENT, "out pointer is null");
    if (m < 1 || m > 8) return fail(MI355Q_ERR_INVALID_ARGUMENT, "decode step takes 1 <= M <= 8");
    fill_common(w, m, out);
    out->path = MI355Q_PATH_DECODE_PROJECTION;
    out->input_row_stride = (uint32_t)w->k;
    // decode => format.gemvKernelName (MetalKernelNameResolver.swift:85-140)
    std::snprintf(out->kernel_name, sizeof out->kernel_name, "%s", w->fmt.gemv_kernel_name);
    std::snprintf(out->kernel_family, sizeof out->kernel_family, "q%uG%uGEMV", (unsigned)w->fmt.bits,
                  w->fmt.group_size);
    RouteFacts facts{};
    facts.decode_entry = true;
    facts.library_ok = !library_ruled_out(w->ctx);
    facts.x_aligned = true;
    plan_small_m(w, m, x_dtype, (uint32_t)w->k, flags, linear_route(w->view(), x_dtype, m, (uint32_t)w->k, flags, facts), out);
    return MI355Q_OK;
}

mi355q_status mi355q_plan_prefill_steps(const mi355q_weight* w, uint32_t maximum_sequence_length,
                                        uint32_t input_row_stride, mi355q_dtype x_dtype, int is_last_token,
                                        uint32_t flags, mi355q_step* out_steps, uint32_t* out_count) {
    if (!w) return fail(MI355Q_ERR_NULL_HANDLE, "weight handle is null");
    if (!out_steps || !out_count) return fail(MI355Q_ERR_INVALID_ARGUMENT, "out pointer is null");
    if (maximum_sequence_length == 0) return fail(MI355Q_ERR_INVALID_ARGUMENT, "maximumSequenceLength must be >= 1");
    if (input_row_stride == 0) input_row_stride = (uint32_t)w->k;
    if (input_row_stride < w->k) return fail(MI355Q_ERR_SHAPE, "inputRowStride smaller than inputDimension");
    *out_count = 1;
    mi355q_step* s = &out_steps[0];
    const WView v = w->view();

    if (is_last_token) {
        // mode = .lastToken: the head runs the decode kernel on one row
        fill_common(w, 1, s);
        s->path = MI355Q_PATH_PREFILL_PROJECTION;
        s->input_row_stride = input_row_stride;
        std::snprintf(s->kernel_name, sizeof s->kernel_name, "%s", w->fmt.gemv_kernel_name);
        std::snprintf(s->kernel_family, sizeof s->kernel_family, "q%uG%uGEMV", (unsigned)w->fmt.bits,
                      w->fmt.group_size);
        RouteFacts one{};
        one.decode_entry = true;
        one.library_ok = !library_ruled_out(w->ctx);
        one.x_aligned = true;
        plan_small_m(w, 1, x_dtype, input_row_stride, flags, linear_route(v, x_dtype, 1, input_row_stride, flags, one), s);
        s->used_fallback = 1;
        s->fallback_reason = MI355Q_FALLBACK_LAST_TOKEN_USES_DECODE_KERNEL;
        return MI355Q_OK;
    }

    const uint32_t m = maximum_sequence_length;
    // the same table the launcher reads (route.cpp): the library counts as there unless it is ruled out for the context
    RouteFacts facts{};
    facts.decode_entry = false;
    facts.library_ok = !library_ruled_out(w->ctx);
    facts.x_aligned = true;
    const LinearRoute route = linear_route(v, x_dtype, m, input_row_stride, flags, facts);
    if (route == LinearRoute::kTwoStep) {
        // dequant_q{b}_g{g}_bf16 into the scratch matrix, then the dense GEMM (MetalPrefillStepBuilder's two-dispatch
        // route; the dense product is the platform library's, as the reference's is matmul2d)
        *out_count = 2;
        mi355q_step* d = &out_steps[0];
        fill_common(w, m, d);
        d->path = MI355Q_PATH_PREFILL_PROJECTION;
        d->input_row_stride = input_row_stride;
        d->flops = 0;
        // fp32 activations from sixteen rows: bf16 weights against the activations split into two bf16 matrices (two
        // library products); below, an fp32 product of fp32 weights
        const bool exact = m < kTwoStepMinRowsOtherwise;       // a few rows: fp32 weights, fp32 product, any activation type
        const bool split = x_dtype == MI355Q_F32 && !exact;
        const char* const type_name = exact ? "f32" : x_dtype == MI355Q_F16 ? "f16" : "bf16";
        std::snprintf(d->kernel_name, sizeof d->kernel_name, "%s", w->fmt.dequant_to_bfloat_kernel_name);
        std::snprintf(d->device_kernel, sizeof d->device_kernel, "dequant_q%u_g%u_%s", (unsigned)w->fmt.bits,
                      w->fmt.group_size, type_name);
        std::snprintf(d->kernel_family, sizeof d->kernel_family, "dequantToBFloat");
        d->block[0] = 256;
        s = &out_steps[1];
        fill_common(w, m, s);
        s->path = MI355Q_PATH_PREFILL_PROJECTION;
        s->input_row_stride = input_row_stride;
        s->weight_bytes = (uint64_t)w->n * w->k * (exact ? 4 : 2);     // the dense operand it reads
        std::snprintf(s->kernel_name, sizeof s->kernel_name, "gemm_bf16_f32s");
        std::snprintf(s->device_kernel, sizeof s->device_kernel, split ? "hipblaslt_gemm_%s_x2" : "hipblaslt_gemm_%s", type_name);
        std::snprintf(s->kernel_family, sizeof s->kernel_family, "libraryGEMM");
        return MI355Q_OK;
    }
    fill_common(w, m, s);
    s->path = MI355Q_PATH_PREFILL_PROJECTION;
    s->input_row_stride = input_row_stride;
    if (route == LinearRoute::kStream) {
        // weights streamed through registers into the matrix cores: the direct quantized GEMM at a few dozen rows
        std::snprintf(s->kernel_name, sizeof s->kernel_name, "%s", w->fmt.gemm_kernel_name_f32s);
        std::snprintf(s->device_kernel, sizeof s->device_kernel, "qgemm_stream_q%u_g%u", (unsigned)w->fmt.bits,
                      w->fmt.group_size);
        std::snprintf(s->kernel_family, sizeof s->kernel_family, "mfmaGEMM");
        const StreamLaunchShape g = gemm_stream_shape(w->ctx, m, (uint32_t)w->n, (uint32_t)w->k);
        s->block[0] = 768;
        s->grid[0] = g.row_blocks;
        s->grid[1] = g.parts;
        s->lds_bytes = g.lds_bytes;
        s->rows_per_workgroup = 64;
        return MI355Q_OK;
    }
    if (route == LinearRoute::kFused) {
        // fused dequant + matrix-core contraction: the stand-in for dequant_q*_bf16 + gemm_bf16_f32s
        std::snprintf(s->kernel_name, sizeof s->kernel_name, "%s", w->fmt.gemm_kernel_name_f32s);
        std::snprintf(s->device_kernel, sizeof s->device_kernel, "qgemm_mfma_q%u_g%u", (unsigned)w->fmt.bits,
                      w->fmt.group_size);
        std::snprintf(s->kernel_family, sizeof s->kernel_family, "mfmaGEMM");
        const bool wide = gemm_wide_taken(v, x_dtype, m, input_row_stride, flags);
        if (wide)
            std::snprintf(s->device_kernel, sizeof s->device_kernel, "%sqgemm_wide_q%u_g%u", x_dtype == MI355Q_F32 ? "split_f32_bf16x2+" : "",
                          (unsigned)w->fmt.bits, w->fmt.group_size);
        const GemmLaunchShape g = wide ? gemm_wide_shape(m, (uint32_t)w->n, gemm_wide_k((uint32_t)w->k, x_dtype))
                                       : gemm_mfma_shape(w->ctx, m, (uint32_t)w->n, (uint32_t)w->k);
        s->block[0] = g.block;
        s->grid[0] = g.grid;
        s->grid[1] = wide ? 1 : g.splits;            // the wide-tile kernel numbers the parts of K inside its one grid axis
        s->lds_bytes = g.lds_bytes;
        s->rows_per_workgroup = g.bn;
        return MI355Q_OK;
    }
    // the decode kernels with the sequence signature (gemm_q{b}_g{g}[_f32s]): small batches, split fp32 rows, and the
    // weights no matrix-core kernel reads (recorded as a fallback, with the reference's reason)
    std::snprintf(s->kernel_name, sizeof s->kernel_name, "%s",
                  x_dtype == MI355Q_F32 ? w->fmt.gemm_kernel_name_f32s : w->fmt.gemm_kernel_name);
    std::snprintf(s->kernel_family, sizeof s->kernel_family, "q%uG%uGEMM", (unsigned)w->fmt.bits,
                  w->fmt.group_size);
    plan_small_m(w, m, x_dtype, input_row_stride, flags, route, s);
    const bool want_small = (flags & (MI355Q_FLAG_FORCE_SMALL_M | MI355Q_FLAG_FORCE_GENERIC)) ||
                            (!(flags & MI355Q_FLAG_FORCE_MFMA) && m <= small_batch_limit(v, x_dtype, input_row_stride)) ||
                            route == LinearRoute::kSplitRows;
    const bool fused_ok = gemm_mfma_eligible(v, x_dtype, m, input_row_stride) || gemm_wide_taken(v, x_dtype, m, input_row_stride, flags);
    if (!want_small && !fused_ok) {
        s->used_fallback = 1;
        s->fallback_reason = (input_row_stride != w->k) ? MI355Q_FALLBACK_INPUT_STRIDE_MISMATCH
                                                        : MI355Q_FALLBACK_UNAVAILABLE_ACCELERATION;
    }
    return MI355Q_OK;
}

// Measurement / test aid: the route table on a synthetic weight, no device needed.  `launcher_out` is what
// dispatch_linear and run_small_m would run ("route" or "route/kernel"), `planner_out` the device kernels the plan
// records name, joined by '+'.
mi355q_status mi355q_probe_route(uint8_t scheme_identifier, uint32_t layout, uint32_t sb_dtype, uint64_t n_rows, uint64_t k,
                                 mi355q_dtype x_dtype, uint32_t m, uint32_t x_row_stride, uint32_t flags, int decode_entry,
                                 int library_available, char* launcher_out, char* planner_out, size_t cap) {
    const mi355q_format* f = find_format_scheme(scheme_identifier);
    if (!f) return fail(MI355Q_ERR_UNSUPPORTED_FORMAT, "unsupported scheme 0x%02x", scheme_identifier);
    if (!launcher_out || !planner_out || cap < 16) return fail(MI355Q_ERR_INVALID_ARGUMENT, "output buffers");
    if (!n_rows || !k || k % f->group_size) return fail(MI355Q_ERR_SHAPE, "K must be a whole number of groups");
    if (layout != MI355Q_LAYOUT_STAF_BLOCKS && (k * f->bits) % 32) return fail(MI355Q_ERR_SHAPE, "planes need whole words per row");
    if (layout == MI355Q_LAYOUT_TILE16 && (f->bits != 4 || f->group_size != 64 || k % 128))
        return fail(MI355Q_ERR_UNSUPPORTED_FORMAT, "TILE16 holds q4 g64 with K %% 128 == 0");
    if (x_row_stride == 0) x_row_stride = (uint32_t)k;
    mi355q_context ctx;
    mi355q_weight w;
    synthetic_weight(&ctx, &w, f, layout, sb_dtype, n_rows, k, library_available != 0);
    const WView v = w.view();
    RouteFacts facts{};
    facts.decode_entry = decode_entry != 0;
    facts.library_ok = library_available != 0;
    facts.x_aligned = true;
    const LinearRoute r = linear_route(v, x_dtype, m, x_row_stride, flags, facts);
    const char* detail = "";
    if (r == LinearRoute::kSmallBatch) {
        const uint32_t step = small_batch_step(v, x_dtype, m, x_row_stride, flags);
        detail = small_kernel_name(small_kernel(v, x_dtype, m < step ? m : step, x_row_stride, flags, true));
    } else if (r == LinearRoute::kFused) {
        detail = gemm_wide_taken(v, x_dtype, m, x_row_stride, flags) ? "wide" : "tiled";
    } else if (r == LinearRoute::kSplitRows) {
        if (!(flags & (MI355Q_FLAG_FORCE_GENERIC | MI355Q_FLAG_FORCE_SMALL_M)) && split_rows_take_stream(v, x_dtype, m)) detail = "stream";
        else {
            const uint32_t pm = split_rows_parts(x_dtype) * m, kp = split_rows_stride((uint32_t)k);
            const uint32_t step = small_batch_step(v, MI355Q_BF16, pm, kp, flags);
            detail = small_kernel_name(small_kernel(v, MI355Q_BF16, pm < step ? pm : step, kp, flags, true));
        }
    }
    std::snprintf(launcher_out, cap, "%s%s%s", linear_route_name(r), *detail ? "/" : "", detail);
    planner_out[0] = 0;
    mi355q_step steps[2];
    uint32_t count = 0;
    mi355q_status st;
    if (decode_entry) { st = mi355q_plan_decode_step(&w, m, x_dtype, flags, &steps[0]); count = 1; }
    else st = mi355q_plan_prefill_steps(&w, m, x_row_stride, x_dtype, 0, flags, steps, &count);
    if (st != MI355Q_OK) { std::snprintf(planner_out, cap, "error"); return MI355Q_OK; }
    size_t at = 0;
    for (uint32_t i = 0; i < count && at < cap; i++)
        at += (size_t)std::snprintf(planner_out + at, cap - at, "%s%s", i ? "+" : "", steps[i].device_kernel);
    return MI355Q_OK;
}

// The same for two or three projections that share their activations (q+k+v, gate+up): what dispatch_batched would run
// (shared_route) and the device kernel the plan record of the shared launch names.
mi355q_status mi355q_probe_shared_route(uint8_t scheme_identifier, uint32_t layout, uint32_t sb_dtype, uint32_t count,
                                        const uint64_t* n_rows, uint64_t k, mi355q_dtype x_dtype, uint32_t m,
                                        uint32_t x_row_stride, uint32_t flags, char* launcher_out, char* planner_out, size_t cap) {
    const mi355q_format* f = find_format_scheme(scheme_identifier);
    if (!f) return fail(MI355Q_ERR_UNSUPPORTED_FORMAT, "unsupported scheme 0x%02x", scheme_identifier);
    if (!launcher_out || !planner_out || cap < 16 || !n_rows) return fail(MI355Q_ERR_INVALID_ARGUMENT, "output buffers");
    if (count != 2 && count != 3) return fail(MI355Q_ERR_INVALID_ARGUMENT, "two or three projections");
    if (!k || k % f->group_size) return fail(MI355Q_ERR_SHAPE, "K must be a whole number of groups");
    if (layout != MI355Q_LAYOUT_STAF_BLOCKS && (k * f->bits) % 32) return fail(MI355Q_ERR_SHAPE, "planes need whole words per row");
    if (layout == MI355Q_LAYOUT_TILE16 && (f->bits != 4 || f->group_size != 64 || k % 128))
        return fail(MI355Q_ERR_UNSUPPORTED_FORMAT, "TILE16 holds q4 g64 with K %% 128 == 0");
    if (x_row_stride == 0) x_row_stride = (uint32_t)k;
    mi355q_context ctx;
    mi355q_weight w[3];
    const mi355q_weight* ws[3] = {&w[0], &w[1], &w[2]};
    WView views[3];
    for (uint32_t i = 0; i < count; i++) {
        if (!n_rows[i]) return fail(MI355Q_ERR_SHAPE, "empty projection");
        synthetic_weight(&ctx, &w[i], f, layout, sb_dtype, n_rows[i], k, true);
        views[i] = w[i].view();
    }
    const SharedRoute r = shared_route(&ctx, count, views, x_dtype, m, x_row_stride, flags, true);
    std::snprintf(launcher_out, cap, "%s", shared_route_name(r));
    mi355q_step steps[2];
    uint32_t n_steps = 0;
    mi355q_status st;
    if (m <= 8) { st = mi355q_plan_decode_step(&w[0], m, x_dtype, flags, &steps[0]); n_steps = 1; }
    else st = mi355q_plan_prefill_steps(&w[0], m, x_row_stride, x_dtype, 0, flags, steps, &n_steps);
    if (st != MI355Q_OK || !n_steps) { std::snprintf(planner_out, cap, "error"); return MI355Q_OK; }
    plan_shared_launch_shape(ws, count, m, x_dtype, x_row_stride, flags, &steps[0]);
    std::snprintf(planner_out, cap, "%s", steps[0].device_kernel);
    return MI355Q_OK;
}

}  // extern "C"
