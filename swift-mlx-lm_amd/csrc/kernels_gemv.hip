// Host-side selection and launch of the split-plane decode GEMV (kernels: gemv_planes.inl).
#include <cstdlib>

#include "gemv_planes.inl"

namespace mi355q {

mi355q_status launch_gemv_planes_q2(hipStream_t, const GemvArgs&, int, int, int, bool, uint32_t, size_t);
mi355q_status launch_gemv_planes_q3(hipStream_t, const GemvArgs&, int, int, int, bool, uint32_t, size_t);
mi355q_status launch_gemv_planes_q4(hipStream_t, const GemvArgs&, int, int, int, bool, uint32_t, size_t);
mi355q_status launch_gemv_planes_q5(hipStream_t, const GemvArgs&, int, int, int, bool, uint32_t, size_t);
mi355q_status launch_gemv_planes_q6(hipStream_t, const GemvArgs&, int, int, int, bool, uint32_t, size_t);
mi355q_status launch_gemv_planes_q8(hipStream_t, const GemvArgs&, int, int, int, bool, uint32_t, size_t);

namespace {

constexpr size_t kLdsBudget = 144 * 1024;  // of the 160 KiB per CU; the rest is left for the runtime

struct Geo { int wpl, cpl; };
Geo geo_for(uint32_t bits) {
    switch (bits) {
    case 2: return {GemvGeo<2>::WPL, GemvGeo<2>::CPL};
    case 3: return {GemvGeo<3>::WPL, GemvGeo<3>::CPL};
    case 4: return {GemvGeo<4>::WPL, GemvGeo<4>::CPL};
    case 5: return {GemvGeo<5>::WPL, GemvGeo<5>::CPL};
    case 6: return {GemvGeo<6>::WPL, GemvGeo<6>::CPL};
    case 8: return {GemvGeo<8>::WPL, GemvGeo<8>::CPL};
    default: return {0, 0};
    }
}

size_t lds_bytes(const WView& w, int mt) {
    const Geo g = geo_for(w.bits);
    const size_t kc = 64 * (size_t)g.cpl;
    const size_t nc = (w.k + kc - 1) / kc;
    const size_t sr = (size_t)g.cpl < w.group ? g.cpl : w.group;
    const size_t nsr = g.cpl / sr;
    return (size_t)mt * nc * 64 * ((size_t)(g.cpl / 8) * 16 + nsr * 4);
}

int env_int(const char* name, int fallback) {
    const char* v = std::getenv(name);
    return (v && *v) ? std::atoi(v) : fallback;
}

// Largest activation batch (1, 2, 4 or 8) whose staged activations fit the LDS budget.
int max_mt(const WView& w) {
    for (int mt = 8; mt >= 1; mt >>= 1)
        if (lds_bytes(w, mt) <= kLdsBudget) return mt;
    return 0;
}

struct Choice { int r, mt; uint32_t grid, nrb, nc; size_t lds; };

Choice choose(const mi355q_context* ctx, const WView& w, uint32_t m, bool argmax) {
    Choice c{};
    c.mt = m <= 1 ? 1 : m <= 2 ? 2 : m <= 4 ? 4 : 8;
    if (c.mt == 1) {
        // rows per wavefront: more rows in flight per lane once there are enough rows to go round
        c.r = w.n >= 8192 ? 4 : (w.n >= 2048 ? 2 : 1);
        const int forced = env_int("MI355Q_GEMV_ROWS_PER_WAVE", 0);
        if (forced == 1 || forced == 2 || forced == 4) c.r = forced;
    } else {
        c.r = c.mt == 8 ? 1 : 2;
    }
    (void)argmax;
    const Geo g = geo_for(w.bits);
    const size_t kc = 64 * (size_t)g.cpl;
    c.nc = (uint32_t)((w.k + kc - 1) / kc);
    c.nrb = (w.n + 4 * c.r - 1) / (4 * c.r);
    c.lds = lds_bytes(w, c.mt);
    int per_cu = env_int("MI355Q_GEMV_WGS_PER_CU", 4);
    const size_t fit = c.lds ? (160 * 1024) / c.lds : 8;
    if ((size_t)per_cu > fit) per_cu = (int)(fit ? fit : 1);
    if (per_cu < 1) per_cu = 1;
    const uint32_t cap = (uint32_t)ctx->props.multiProcessorCount * (uint32_t)per_cu;
    c.grid = c.nrb < cap ? c.nrb : cap;
    if (c.grid == 0) c.grid = 1;
    return c;
}

}  // namespace

bool gemv_fast_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride) {
    if (w.layout != MI355Q_LAYOUT_PLANES || x_dtype != MI355Q_BF16) return false;
    if (m < 1 || m > 8) return false;
    const Geo g = geo_for(w.bits);
    if (!g.cpl) return false;
    if (w.k % (uint32_t)g.cpl) return false;       // rows are whole lane chunks
    if (x_stride % 8) return false;                // 128-bit activation loads
    if ((uintptr_t)w.codes % 16) return false;     // 128-bit code loads
    if (max_mt(w) == 0) return false;
    return true;
}

GemvLaunchShape gemv_fast_shape(const mi355q_context* ctx, const WView& w, uint32_t m) {
    const int fit = max_mt(w);
    const uint32_t mm = (fit && m > (uint32_t)fit) ? (uint32_t)fit : m;
    const Choice c = choose(ctx, w, mm, false);
    GemvLaunchShape s;
    s.grid = c.grid;
    s.block = 256;
    s.lds_bytes = (uint32_t)c.lds;
    s.rows_per_workgroup = (uint32_t)(4 * c.r);
    s.kernel = "gemv_planes_kernel";
    return s;
}

mi355q_status launch_gemv_fast(hipStream_t s, const mi355q_context* ctx, const WView& w, const void* x, void* y,
                               int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride, float* logits_f32,
                               int32_t* token_out, unsigned long long* argmax_scratch) {
    if ((uintptr_t)x % 16) return fail(MI355Q_ERR_INVALID_ARGUMENT, "activation pointer must be 16-byte aligned");
    const bool argmax = token_out != nullptr;
    if (argmax && m != 1) return fail(MI355Q_ERR_INVALID_ARGUMENT, "fused argmax needs M == 1");
    const int fit = max_mt(w);
    if (!fit) return fail(MI355Q_ERR_SHAPE, "K=%u does not fit the activation staging budget", w.k);
    const size_t ysz = y_dtype == MI355Q_F32 ? 4 : 2;
    // activation batches larger than what fits in LDS are processed in slices of `fit` rows
    for (uint32_t m0 = 0; m0 < m; m0 += (uint32_t)fit) {
        const uint32_t mm = (m - m0) < (uint32_t)fit ? (m - m0) : (uint32_t)fit;
        const Choice c = choose(ctx, w, mm, argmax);
        GemvArgs a{};
        a.codes = w.codes;
        a.scales = w.scales;
        a.biases = w.biases;
        a.x = (const uint16_t*)x + (size_t)m0 * x_stride;
        a.y = y ? (void*)((char*)y + (size_t)m0 * y_stride * ysz) : nullptr;
        a.logits = logits_f32;
        a.token_out = token_out;
        a.scratch = argmax_scratch;
        a.n = w.n; a.k = w.k; a.m = mm;
        a.x_stride = x_stride; a.y_stride = y_stride;
        a.words_per_row = w.words_per_row; a.blocks_per_row = w.blocks_per_row;
        a.nc = c.nc; a.nrb = c.nrb;
        a.y_dtype = (uint32_t)y_dtype; a.sb_dtype = w.sb_dtype;
        mi355q_status st;
        switch (w.bits) {
        case 2: st = launch_gemv_planes_q2(s, a, (int)w.group, c.r, c.mt, argmax, c.grid, c.lds); break;
        case 3: st = launch_gemv_planes_q3(s, a, (int)w.group, c.r, c.mt, argmax, c.grid, c.lds); break;
        case 4: st = launch_gemv_planes_q4(s, a, (int)w.group, c.r, c.mt, argmax, c.grid, c.lds); break;
        case 5: st = launch_gemv_planes_q5(s, a, (int)w.group, c.r, c.mt, argmax, c.grid, c.lds); break;
        case 6: st = launch_gemv_planes_q6(s, a, (int)w.group, c.r, c.mt, argmax, c.grid, c.lds); break;
        case 8: st = launch_gemv_planes_q8(s, a, (int)w.group, c.r, c.mt, argmax, c.grid, c.lds); break;
        default: st = fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no split-plane GEMV for %u-bit codes", w.bits);
        }
        if (st != MI355Q_OK) return st;
    }
    return MI355Q_OK;
}

}  // namespace mi355q
