// Host-side selection and launch of the split-plane decode GEMV (kernels: gemv_planes.inl).
#include <cstdlib>

#include "gemv_planes.inl"

namespace mi355q {

mi355q_status launch_gemv_planes_q2(hipStream_t, const GemvArgs&, int, const GemvCfg&);
mi355q_status launch_gemv_planes_q3(hipStream_t, const GemvArgs&, int, const GemvCfg&);
mi355q_status launch_gemv_planes_q4(hipStream_t, const GemvArgs&, int, const GemvCfg&);
mi355q_status launch_gemv_planes_q5(hipStream_t, const GemvArgs&, int, const GemvCfg&);
mi355q_status launch_gemv_planes_q6(hipStream_t, const GemvArgs&, int, const GemvCfg&);
mi355q_status launch_gemv_planes_q8(hipStream_t, const GemvArgs&, int, const GemvCfg&);

#ifdef MI355Q_GEMV_TIMELINE
unsigned long long* g_gemv_timeline = nullptr;      // measurement build only
extern "C" __attribute__((visibility("default"))) void mi355q_probe_set_timeline(unsigned long long* p) { g_gemv_timeline = p; }
#endif

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

// Staged activations of mt rows: pairs, then per sub-run the sum of the activations and, in f16 arithmetic on
// 2- and 4-bit codes, the class-weighted sum next to it.
size_t lds_bytes(const WView& w, int mt, int xa) {
    const Geo g = geo_for(w.bits);
    const size_t kc = 64 * (size_t)g.cpl;
    const size_t nc = (w.k + kc - 1) / kc;
    const size_t sr = (size_t)g.cpl < w.group ? g.cpl : w.group;
    const size_t nsr = g.cpl / sr;
    // two sums per lane chunk where fields are used in place (f16: 2 and 4 bits; bf16, rows kernel: 3 bits)
    const size_t nf = ((xa == 1 && (w.bits == 2 || w.bits == 4)) || (xa == 0 && w.bits == 3)) ? 2 : 1;
    return (size_t)mt * nc * 64 * ((size_t)(g.cpl / 8) * 16 + nsr * nf * 4);
}

// Largest activation batch per launch (1, 2 or 4) whose staged activations fit the LDS budget.
// Batches of 5 to 8 rows run as two launches: an 8-row variant of this kernel needs more registers
// than a wavefront has.
int max_mt(const WView& w) {
    // q2 g16 carries four scale groups per lane chunk: its 4-row variant does not fit the register file
    for (int mt = (w.bits == 2 && w.group == 16) ? 2 : 4; mt >= 1; mt >>= 1)
        if (lds_bytes(w, mt, 1) <= kLdsBudget) return mt;
    return 0;
}

// Variant and launch shape for one call (measured on MI355X).
GemvCfg choose(const mi355q_context* ctx, const WView& w, uint32_t m, bool argmax, int x_dtype) {
    GemvCfg c{};
    c.argmax = argmax;
    c.xa = x_dtype == MI355Q_F16 ? 1 : 0;
    c.mt = m <= 1 ? 1 : m <= 2 ? 2 : 4;
    const Geo g = geo_for(w.bits);
    const size_t kc = 64 * (size_t)g.cpl;
    c.nc = (uint32_t)((w.k + kc - 1) / kc);
    // One activation row and rows of 1, 2, 3, 4 or 7 K-steps: the static-structure kernel.  A wavefront takes two rows
    // (four of one K-step) in one pass, every load issued up front, fewer while that would leave less than sixteen
    // wavefronts per CU (measured, q4 g64: 28672 rows of two K-steps 12.1-12.3 us with two rows per wavefront,
    // 12.4-14.0 with four, 13.8-14.1 with one; 14336 rows 7.5 / 8.2 / 8.0 us; 4096 rows 4.2 us either way; 14336 rows
    // of four K-steps, q8 g32: 12.2 us with two rows, 14.4 with one; q6 g64 10.0 / 10.1; q3 g64 8.1 / 8.8).
    // Two to four activation rows (4 bits, bf16): the same kernel with every row on each unpacked code pair (28672 rows
    // of two K-steps at two rows: 18.4 us on the general kernel, 15.7 us here; a further row costs the dot products
    // alone).  Three and four rows where gemv_rows_batch_pays() says so (the callers ask).
    const bool two_rows = m >= 2 && m <= 4 && !argmax && !c.xa && w.bits == 4;
    if (two_rows) c.mt = (int)m;
    if ((c.mt == 1 || two_rows) && gemv_rows_has_format((int)w.bits, (int)w.group) &&
        (!c.xa || gemv_rows_has_f16((int)w.bits, (int)w.group)) && (c.nc <= 4 || (c.nc == 7 && w.bits != 8))) {
        const uint32_t least_waves = (uint32_t)ctx->props.multiProcessorCount * 16u;
        uint32_t rpw = c.nc == 1 ? 4 : c.nc <= 4 ? 2 : 1;
        while (rpw > 1 && w.n / rpw < least_waves) rpw >>= 1;
        int br = (int)rpw;                                                          // one pass
#ifdef MI355Q_GEMV_TIMELINE
        if (const char* e = std::getenv("TL_RPW")) rpw = (uint32_t)std::atoi(e);      // measurement build only
        br = (int)rpw;
        if (const char* e = std::getenv("TL_BR")) br = std::atoi(e);
#endif
        if (argmax && !gemv_rows_has_argmax((int)c.nc, br)) br = c.nc == 1 ? 4 : 2;   // the head's variants
        rpw = (rpw + br - 1) / br * br;
        // very tall matrices: more passes rather than more than 65535 workgroups
        while ((w.n + rpw * 4 - 1) / (rpw * 4) > 65535u && rpw + br <= 64) rpw += br;
        if (rpw <= 64 && gemv_rows_has_shape((int)c.nc, br) && (!argmax || gemv_rows_has_argmax((int)c.nc, br)) &&
            (!two_rows || (gemv_rows_has_batch((int)w.bits, (int)w.group, (int)c.nc, br, c.mt) && lds_bytes(w, c.mt, 0) <= kLdsBudget))) {
            c.rows = true;
            c.nct = (int)c.nc;
            c.br = br;
            c.r = 1;
            c.waves = gemv_rows_waves(c.nct);
            c.rows_per_wave = rpw;
            c.lds = lds_bytes(w, c.mt, c.xa);
            const uint32_t rows_per_wg = rpw * (uint32_t)c.waves;
            c.grid = (w.n + rows_per_wg - 1) / rows_per_wg;
            if (c.grid == 0) c.grid = 1;
            return c;
        }
    }
    c.mt = m <= 1 ? 1 : m <= 2 ? 2 : 4;                      // the general kernel's batches
    const uint64_t weight_bytes = (uint64_t)w.n * (w.k / w.group) * (4 + w.group * w.bits / 8);
    const bool big = weight_bytes >= (24ull << 20);
    if (c.mt == 1) {
        // Measured on MI355X (q4 g64): large matrices of short rows (one or two K-steps) run best with 4
        // wavefronts per workgroup, and with rows of one K-step they keep their activation slice in
        // registers; everything else runs best with 8 wavefronts reading the slice from LDS
        // (2048 -> 8192: 4.3 us against 5.5 us with the large-matrix shape).
        c.xreg = (c.nc == 1 && big) ? 1 : 0;
        c.r = 1;
        c.waves = (c.nc <= 2 && big) ? 4 : 8;
        // long rows (more than two K-steps: 14336 -> 4096): sixteen wavefronts share one staged copy of the long
        // activation vector (8.8 us against 9.2 us with eight)
        if (c.nc > 2 && big) c.waves = 16;
    } else {
        c.xreg = 0;
        c.r = gemv_batch_rows((int)w.bits, (int)w.group, c.mt);
        c.waves = 4;
    }
    c.lds = lds_bytes(w, c.mt, c.xa);
    // rows per wavefront: aim for 32 wavefronts on every CU at M = 1, 16 for batches, each owning a whole
    // number of R-row steps
    const uint32_t target = (uint32_t)ctx->props.multiProcessorCount * (c.mt == 1 ? 32u : 16u);
    uint32_t rpw = (w.n + target - 1) / target;
    rpw = (rpw + c.r - 1) / c.r * c.r;
    if (rpw < (uint32_t)c.r) rpw = c.r;
    c.rows_per_wave = rpw;
    // ring depth: four pipeline steps in flight, two when a wavefront only has two or three
    const uint32_t nsteps = rpw / (uint32_t)c.r * c.nc;
    if (c.mt == 1) c.depth = (nsteps >= 4 && (big || c.nc > 2)) ? 4 : 2;
    else c.depth = gemv_batch_depth((int)w.bits, (int)w.group, c.mt);
    const uint32_t rows_per_wg = rpw * (uint32_t)c.waves;
    c.grid = (w.n + rows_per_wg - 1) / rows_per_wg;
    if (c.grid == 0) c.grid = 1;
    return c;
}

}  // namespace

bool gemv_fast_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride) {
    if (w.layout != MI355Q_LAYOUT_PLANES || (x_dtype != MI355Q_BF16 && x_dtype != MI355Q_F16)) return false;
    if (m < 1 || m > 8) return false;
    const Geo g = geo_for(w.bits);
    if (!g.cpl) return false;
    if (w.k % (uint32_t)g.cpl) return false;       // rows are whole lane chunks
    if (x_stride % 8) return false;                // 128-bit activation loads
    if ((uintptr_t)w.codes % 16 || w.code_stride % 4) return false;     // 128-bit code loads
    if (!w.sz) return false;
    if (max_mt(w) == 0) return false;
    return true;
}

GemvLaunchShape gemv_fast_shape(const mi355q_context* ctx, const WView& w, uint32_t m, int x_dtype) {
    const int fit = max_mt(w);
    const uint32_t mm = (fit && m > (uint32_t)fit) ? (uint32_t)fit : m;
    const GemvCfg c = choose(ctx, w, mm, false, x_dtype);
    GemvLaunchShape s;
    s.grid = c.grid;
    s.block = (uint32_t)c.waves * 64;
    s.lds_bytes = (uint32_t)c.lds;
    s.rows_per_workgroup = c.rows_per_wave * (uint32_t)c.waves;
    s.kernel = c.rows ? "gemv_rows_kernel" : "gemv_planes_kernel";
    return s;
}

// Up to three weights sharing K, format and activations in one launch.  `w[0]` supplies the format;
// the caller has checked that the others match.
mi355q_status launch_gemv_fast_multi(hipStream_t s, const mi355q_context* ctx, uint32_t count, const WView* w,
                                     const void* x, int x_dtype, void* const* y, const uint32_t* y_strides, int y_dtype,
                                     uint32_t m, uint32_t x_stride, float* logits_f32, int32_t* token_out,
                                     HeadKeys keys) {
    if (count < 1 || count > (uint32_t)kGemvMaxSegments)
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "1..%d weights per fused launch", kGemvMaxSegments);
    if ((uintptr_t)x % 16) return fail(MI355Q_ERR_INVALID_ARGUMENT, "activation pointer must be 16-byte aligned");
    const bool argmax = token_out != nullptr;
    if (argmax && (m != 1 || count != 1)) return fail(MI355Q_ERR_INVALID_ARGUMENT, "fused argmax needs M == 1");
    if (logits_f32 && count != 1) return fail(MI355Q_ERR_INVALID_ARGUMENT, "fp32 logits need a single weight");
    WView all = w[0];                       // same geometry, rows of every segment together
    uint64_t total = 0;
    for (uint32_t i = 0; i < count; i++) total += w[i].n;
    if (total > 0xFFFFFFFFull) return fail(MI355Q_ERR_SHAPE, "too many rows");
    all.n = (uint32_t)total;
    const int fit = max_mt(all);
    if (!fit) return fail(MI355Q_ERR_SHAPE, "K=%u does not fit the activation staging budget", all.k);
    const size_t ysz = y_dtype == MI355Q_F32 ? 4 : 2;
    // activation batches larger than what fits in LDS are processed in slices of `fit` rows
    for (uint32_t m0 = 0; m0 < m; m0 += (uint32_t)fit) {
        const uint32_t mm = (m - m0) < (uint32_t)fit ? (m - m0) : (uint32_t)fit;
        GemvCfg c = choose(ctx, all, mm, argmax, x_dtype);
        GemvArgs a{};
        uint32_t waves = 0;
        for (uint32_t i = 0; i < (uint32_t)kGemvMaxSegments; i++) {
            const uint32_t j = i < count ? i : count - 1;
            if (i < count) waves += (w[i].n + c.rows_per_wave - 1) / c.rows_per_wave;
            a.codes[i] = w[j].codes;
            a.sz[i] = w[j].sz;
            a.y[i] = y[j] ? (void*)((char*)y[j] + (size_t)m0 * y_strides[j] * ysz) : nullptr;
            a.y_stride[i] = y_strides[j];
            a.seg_rows[i] = w[j].n;
            a.wave_end[i] = waves;
        }
        const uint32_t grid = (waves + (uint32_t)c.waves - 1) / (uint32_t)c.waves;
        a.x = (const uint16_t*)x + (size_t)m0 * x_stride;
        a.logits = logits_f32;
        a.token_out = token_out;
        a.scratch = keys.ptr;
        a.k = all.k; a.m = mm;
        a.x_stride = x_stride;
        a.code_stride = all.code_stride; a.sz_stride = all.sz_stride;
        a.nc = c.nc; a.rows_per_wave = c.rows_per_wave;
        a.y_dtype = (uint32_t)y_dtype; a.sb_dtype = all.sb_dtype; a.x_dtype = (uint32_t)x_dtype;
#ifdef MI355Q_GEMV_TIMELINE
        a.timeline = g_gemv_timeline;
#endif
        c.grid = grid;                        // whole wavefronts per matrix: a few more than rows / rows_per_wave
        if (argmax && grid > keys.capacity)
            return fail(MI355Q_ERR_SHAPE, "the fused output head keeps one partial key per workgroup: %u workgroups exceed %u",
                        grid, keys.capacity);
        mi355q_status st;
        switch (all.bits) {
        case 2: st = launch_gemv_planes_q2(s, a, (int)all.group, c); break;
        case 3: st = launch_gemv_planes_q3(s, a, (int)all.group, c); break;
        case 4: st = launch_gemv_planes_q4(s, a, (int)all.group, c); break;
        case 5: st = launch_gemv_planes_q5(s, a, (int)all.group, c); break;
        case 6: st = launch_gemv_planes_q6(s, a, (int)all.group, c); break;
        case 8: st = launch_gemv_planes_q8(s, a, (int)all.group, c); break;
        default: st = fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no split-plane GEMV for %u-bit codes", all.bits);
        }
        if (st != MI355Q_OK) return st;
        if (argmax)
            if (mi355q_status fin = launch_argmax_finish(s, keys.ptr, grid, token_out)) return fin;
    }
    return MI355Q_OK;
}

// Gate and up projection of ONE activation row with the gated activation as epilogue: the rows kernel over 2 N
// "virtual rows" (2 r = row r of gate, 2 r + 1 = row r of up), launch shape chosen as for a matrix of 2 N rows.
namespace {
bool gated_cfg(const mi355q_context* ctx, const WView& gate, const WView& up, int x_dtype, uint32_t x_stride, GemvCfg& c) {
    if (!gemv_fast_eligible(gate, x_dtype, 1, x_stride) || !gemv_fast_eligible(up, x_dtype, 1, x_stride)) return false;
    if (gate.n != up.n || gate.k != up.k || gate.bits != up.bits || gate.group != up.group || gate.sb_dtype != up.sb_dtype ||
        gate.code_stride != up.code_stride || gate.sz_stride != up.sz_stride) return false;
    if ((uint64_t)gate.n * 2 > 0xFFFFFFFFull) return false;
    WView all = gate;
    all.n = gate.n * 2;
    c = choose(ctx, all, 1, false, x_dtype);
    if (!c.rows) return false;                             // rows of a length the static-structure kernel does not take
    if (c.rows_per_wave & 1u) {                            // a wavefront owns whole (gate, up) pairs
        c.rows_per_wave += (uint32_t)c.br;
        if ((c.rows_per_wave & 1u) || c.rows_per_wave > 64) return false;
    }
    c.gated = true;
    return true;
}
}  // namespace

bool gemv_gated_eligible(const mi355q_context* ctx, const WView& gate, const WView& up, int x_dtype, uint32_t m, uint32_t x_stride) {
    GemvCfg c{};
    return m == 1 && gated_cfg(ctx, gate, up, x_dtype, x_stride, c);
}

mi355q_status launch_gemv_gated(hipStream_t s, const mi355q_context* ctx, const WView& gate, const WView& up, const void* x,
                                int x_dtype, void* y, int y_dtype, uint32_t x_stride, int activation) {
    GemvCfg c{};
    if (!gated_cfg(ctx, gate, up, x_dtype, x_stride, c))
        return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no one-launch gated projection for these weights");
    if ((uintptr_t)x % 16) return fail(MI355Q_ERR_INVALID_ARGUMENT, "activation pointer must be 16-byte aligned");
    GemvArgs a{};
    const uint32_t vrows = gate.n * 2;
    const uint32_t waves = (vrows + c.rows_per_wave - 1) / c.rows_per_wave;
    for (int i = 0; i < kGemvMaxSegments; i++) {
        a.codes[i] = i == 0 ? gate.codes : up.codes;
        a.sz[i] = i == 0 ? gate.sz : up.sz;
        a.y[i] = y;
        a.y_stride[i] = gate.n;
        a.seg_rows[i] = vrows;
        a.wave_end[i] = waves;
    }
    a.x = (const uint16_t*)x;
    a.k = gate.k; a.m = 1;
    a.x_stride = x_stride;
    a.code_stride = gate.code_stride; a.sz_stride = gate.sz_stride;
    a.nc = c.nc; a.rows_per_wave = c.rows_per_wave;
    a.y_dtype = (uint32_t)y_dtype; a.sb_dtype = gate.sb_dtype; a.x_dtype = (uint32_t)x_dtype;
    a.gated = (uint32_t)activation;
    c.grid = (waves + (uint32_t)c.waves - 1) / (uint32_t)c.waves;
    switch (gate.bits) {
    case 2: return launch_gemv_planes_q2(s, a, (int)gate.group, c);
    case 3: return launch_gemv_planes_q3(s, a, (int)gate.group, c);
    case 4: return launch_gemv_planes_q4(s, a, (int)gate.group, c);
    case 5: return launch_gemv_planes_q5(s, a, (int)gate.group, c);
    case 6: return launch_gemv_planes_q6(s, a, (int)gate.group, c);
    case 8: return launch_gemv_planes_q8(s, a, (int)gate.group, c);
    default: break;
    }
    return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no split-plane GEMV for %u-bit codes", gate.bits);
}

mi355q_status launch_gemv_fast(hipStream_t s, const mi355q_context* ctx, const WView& w, const void* x, int x_dtype,
                               void* y, int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride, float* logits_f32,
                               int32_t* token_out, HeadKeys keys) {
    void* ys[1] = {y};
    const uint32_t strides[1] = {y_stride};
    return launch_gemv_fast_multi(s, ctx, 1, &w, x, x_dtype, ys, strides, y_dtype, m, x_stride, logits_f32, token_out,
                                  keys);
}

}  // namespace mi355q
