// Context, device memory, streams, events and packed-weight handles.
#include <new>
#include <vector>

#include <mutex>
#include <unordered_map>

#include "common.h"

using namespace mi355q;

// Partial keys of mi355q_lmhead_argmax_static, the entry point that allocates nothing: a device array in the library
// image (each GPU the library runs on holds its own copy, 258 KiB, until the process ends).  Host code never uses the
// array's name as an address: the address on a device is resolved once, with that device current, when the first context
// is created there, and only that pointer is handed to kernels.
static __device__ __align__(256) unsigned long long scratch[kStaticHeadKeys + kArgmaxStandaloneKeys];

namespace {
constexpr int kMaxDevices = 64;
unsigned long long* g_static_keys[kMaxDevices] = {};
std::mutex g_static_keys_mutex;

// with `device` current
mi355q_status resolve_static_keys(int device) {
    if (device < 0 || device >= kMaxDevices) return fail(MI355Q_ERR_INVALID_ARGUMENT, "device index %d beyond %d", device, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_static_keys_mutex);
    if (g_static_keys[device]) return MI355Q_OK;
    void* ptr = nullptr;
    MI355Q_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return fail(MI355Q_ERR_DEVICE, "hipGetSymbolAddress returned a null address for the static key array");
    g_static_keys[device] = (unsigned long long*)ptr;
    return MI355Q_OK;
}
}  // namespace

namespace mi355q {
unsigned long long* static_head_keys(int device) {
    if (device < 0 || device >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(g_static_keys_mutex);
    return g_static_keys[device];
}
}  // namespace mi355q

namespace mi355q {

namespace {
mi355q_status grow_scratch(mi355q_context* ctx, void*& buffer, size_t& have, size_t bytes, size_t granule) {
    if (bytes <= have) return MI355Q_OK;
    // A launch recorded in a HIP graph keeps the address it was captured with, so an outgrown buffer stays allocated
    // until the context goes; growth at least doubles, which bounds the retired buffers to the size of the live one.
    size_t want = bytes > 2 * have ? bytes : 2 * have;
    want = (want + granule - 1) & ~(granule - 1);
    if (buffer && ctx->retired_count >= kRetiredWorkspaces)
        return fail(MI355Q_ERR_OUT_OF_MEMORY, "scratch buffer outgrown %d times", kRetiredWorkspaces);
    void* grown = nullptr;
    MI355Q_HIP(hipMalloc(&grown, want));
    if (buffer) ctx->retired[ctx->retired_count++] = buffer;
    buffer = grown;
    have = want;
    return MI355Q_OK;
}
}  // namespace

// An entry point that uses the scratch only notes its stream (an event recorded behind every such call costs a caller on
// one stream about 3 us a call: the launches no longer run back to back).  When a call on a second stream arrives, the
// first stream is asked whether it has run dry -- everything it holds by then, which is at least the work that used the
// scratch.  A stream destroyed through this library leaves an event in its place (scratch_marked).
ScratchGuard::ScratchGuard(mi355q_context* c, hipStream_t s) : ctx(c), stream(s), status(MI355Q_OK) {
    if (!ctx) return;
    ctx->scratch_touched = false;
    if (!ctx->scratch_pending || ctx->scratch_stream == s || !s || !ctx->scratch_stream) return;
    hipError_t q;
    if (ctx->scratch_marked) {
        q = hipEventQuery(ctx->scratch_event);
    } else {
        // a stream that is being captured runs nothing; one that is gone (destroyed by its owner, which the runtime
        // answers with an error) has nothing left to order against
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(ctx->scratch_stream, &capture) != hipSuccess || capture != hipStreamCaptureStatusNone)
            q = hipSuccess;
        else
            q = hipStreamQuery(ctx->scratch_stream);
    }
    (void)hipGetLastError();
    if (q == hipErrorNotReady) {
        status = fail(MI355Q_ERR_INVALID_ARGUMENT,
                      "the context's scratch is still in use by work on another stream: one stream per context at a time "
                      "(synchronise the first stream, or give each stream a context of its own)");
        return;
    }
    ctx->scratch_pending = false;
    ctx->scratch_marked = false;
}

ScratchGuard::~ScratchGuard() {
    if (!ctx || status != MI355Q_OK || !ctx->scratch_touched) return;
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (stream && (hipStreamIsCapturing(stream, &capture) != hipSuccess || capture != hipStreamCaptureStatusNone)) {
        (void)hipGetLastError();
        return;
    }
    ctx->scratch_stream = stream;
    ctx->scratch_pending = true;
    ctx->scratch_marked = false;
}

mi355q_status ensure_workspace(mi355q_context* ctx, size_t bytes) {
    ctx->scratch_touched = true;
    return grow_scratch(ctx, ctx->workspace, ctx->workspace_bytes, bytes, (size_t)1 << 22);
}

mi355q_status ensure_split_buffer(mi355q_context* ctx, size_t bytes) {
    ctx->scratch_touched = true;
    return grow_scratch(ctx, ctx->split_buffer, ctx->split_bytes, bytes, (size_t)1 << 20);
}

mi355q_status ensure_gated_buffer(mi355q_context* ctx, size_t bytes) {
    ctx->scratch_touched = true;
    return grow_scratch(ctx, ctx->gated_buffer, ctx->gated_bytes, bytes, (size_t)1 << 20);
}

}  // namespace mi355q

namespace {

// ---- host float16 <-> float32 (round-to-nearest-even), used only while preparing weights ----
inline uint32_t as_u32(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float as_f32(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }

uint16_t host_f32_to_f16(float f) {
    const uint32_t u = as_u32(f);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t a = u & 0x7FFFFFFFu;
    if (a >= 0x7F800000u) return (uint16_t)(sign | (a > 0x7F800000u ? 0x7E00u | ((a >> 13) & 0x3FFu) : 0x7C00u));
    if (a >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);  // rounds to >= 65520 -> inf
    if (a < 0x38800000u) {                                    // below the smallest normal half
        // scale so that the half subnormal grid becomes the integer grid; the fp32 add rounds RNE
        const float scaled = as_f32(a) * 16777216.0f;         // * 2^24 (exact)
        const float magic = 8388608.0f;                       // 2^23: ulp == 1 from here up
        const float r = (scaled + magic) - magic;
        return (uint16_t)(sign | (uint16_t)r);
    }
    const uint32_t rebias = a - 0x38000000u;                  // exponent 127 -> 15
    uint32_t half = rebias >> 13;
    const uint32_t rem = rebias & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++;
    return (uint16_t)(sign | half);
}

float host_bf16_to_f32(uint16_t h) { return as_f32((uint32_t)h << 16); }

float host_f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    if (e == 0x1Fu) return as_f32(sign | 0x7F800000u | (m << 13));
    if (e) return as_f32(sign | ((e + 112u) << 23) | (m << 13));
    const float v = (float)m * 5.9604644775390625e-8f;        // subnormal: m * 2^-24 (exact)
    return sign ? -v : v;
}

// A bf16 scale or bias as the converter would store it (narrowed to f16, round to nearest even), written back as
// bf16.  The narrowed value always has a bf16 spelling: inside the f16 normal range the 8 significant bits of a bf16
// survive, below it rounding to the f16 subnormal grid can only drop bits, above it the result is infinity.  So a
// plane of these values decodes to exactly what the f16 header of the block layout decodes to.
uint16_t host_bf16_through_f16(uint16_t h) {
    return (uint16_t)(as_u32(host_f16_to_f32(host_f32_to_f16(host_bf16_to_f32(h)))) >> 16);
}

float host_load_sb(const void* p, size_t i, int dtype) {
    if (dtype == MI355Q_F32) return ((const float*)p)[i];
    if (dtype == MI355Q_BF16) return host_bf16_to_f32(((const uint16_t*)p)[i]);
    return 0.0f;  // F16 is never widened on the host
}

// scale/bias plane normalised to f16 bits (the converter's normalizeScaleToFloat16)
uint16_t host_sb_as_f16(const void* p, size_t i, int dtype) {
    if (dtype == MI355Q_F16) return ((const uint16_t*)p)[i];
    return host_f32_to_f16(host_load_sb(p, i, dtype));
}

mi355q_status check_shape(const mi355q_format* f, uint64_t n, uint64_t k) {
    if (n == 0 || k == 0) return fail(MI355Q_ERR_SHAPE, "empty weight: N=%llu K=%llu",
                                      (unsigned long long)n, (unsigned long long)k);
    if (n > 0x7FFFFFFFull || k > 0x7FFFFFFFull)
        return fail(MI355Q_ERR_SHAPE, "dimension exceeds 2^31-1");
    if (k % f->group_size)
        return fail(MI355Q_ERR_SHAPE, "K=%llu is not a multiple of group size %u",
                    (unsigned long long)k, f->group_size);
    if ((uint64_t)f->group_size * f->bits % 8)
        return fail(MI355Q_ERR_SHAPE, "group_size x bits is not a whole number of bytes");
    return MI355Q_OK;
}

void repack_rows(const mi355q_format* f, size_t n, size_t k, const uint32_t* codes,
                 const void* scales, const void* biases, int sb_dtype, uint8_t* out) {
    const size_t bpr = k / f->group_size;
    const size_t row_bytes = k * f->bits / 8;
    const size_t group_bytes = (size_t)f->group_size * f->bits / 8;
    const uint8_t* src = (const uint8_t*)codes;
    for (size_t r = 0; r < n; r++)
        for (size_t b = 0; b < bpr; b++) {
            uint8_t* dst = out + (r * bpr + b) * f->bytes_per_block;
            const uint16_t s = host_sb_as_f16(scales, r * bpr + b, sb_dtype);
            const uint16_t z = host_sb_as_f16(biases, r * bpr + b, sb_dtype);
            std::memcpy(dst, &s, 2);
            std::memcpy(dst + 2, &z, 2);
            std::memcpy(dst + 4, src + r * row_bytes + b * group_bytes, group_bytes);
        }
}

mi355q_weight* new_weight(mi355q_context* ctx, const mi355q_format* f, uint64_t n, uint64_t k) {
    mi355q_weight* w = new (std::nothrow) mi355q_weight;
    if (!w) return nullptr;
    std::memset(w, 0, sizeof *w);
    w->ctx = ctx;
    w->fmt = *f;
    w->n = n;
    w->k = k;
    return w;
}

mi355q_status upload_new(void** dev, const void* host, size_t bytes) {
    MI355Q_HIP(hipMalloc(dev, bytes));
    hipError_t e = hipMemcpy(*dev, host, bytes, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        (void)hipFree(*dev);
        *dev = nullptr;
        return fail(MI355Q_ERR_DEVICE, "hipMemcpy (upload) failed: %s", hipGetErrorString(e));
    }
    return MI355Q_OK;
}

// Packed (scale, bias) words of a split-plane weight, filled once on the device from the two
// 16-bit planes.  `dst` is either the sz part of the row-interleaved buffer or a plane of its own.
mi355q_status fill_sz(mi355q_weight* w) {
    const uint32_t bpr = (uint32_t)(w->k / w->fmt.group_size);
    const size_t groups = (size_t)w->n * bpr;
    if (mi355q_status st = launch_pack_sz(nullptr, (const uint16_t*)w->scales, (const uint16_t*)w->biases,
                                          (uint32_t*)w->sz, groups, bpr, w->sz_stride))
        return st;
    MI355Q_HIP(hipStreamSynchronize(nullptr));
    return MI355Q_OK;
}

// Borrowed planes: the caller's code plane stays where it is; sz is an owned plane of its own.
mi355q_status build_sz_plane(mi355q_weight* w) {
    const uint32_t bpr = (uint32_t)(w->k / w->fmt.group_size);
    w->code_stride = (uint32_t)(w->k * w->fmt.bits / 32);
    w->sz_stride = bpr;
    w->sz_separate = 1;
    MI355Q_HIP(hipMalloc(&w->sz, (size_t)w->n * bpr * 4));
    return fill_sz(w);
}

// Owned planes: one buffer of rows [code words | sz words | pad to 16 bytes].  The host code plane
// is copied with a pitched copy; scales/biases must already be on the device.
mi355q_status build_rows(mi355q_weight* w, const void* codes_host) {
    const uint32_t wpr = (uint32_t)(w->k * w->fmt.bits / 32), bpr = (uint32_t)(w->k / w->fmt.group_size);
    const uint32_t stride = (wpr + bpr + 3u) & ~3u;
    w->code_stride = stride;
    w->sz_stride = stride;
    w->sz_separate = 0;
    w->codes_bytes = (size_t)w->n * stride * 4;
    MI355Q_HIP(hipMalloc(&w->codes, w->codes_bytes));
    w->sz = (uint32_t*)w->codes + wpr;
    if (stride != wpr + bpr) MI355Q_HIP(hipMemset(w->codes, 0, w->codes_bytes));   // padding words
    MI355Q_HIP(hipMemcpy2D(w->codes, (size_t)stride * 4, codes_host, (size_t)wpr * 4, (size_t)wpr * 4, (size_t)w->n,
                           hipMemcpyHostToDevice));
    return fill_sz(w);
}

// TILE16: build the split-plane rows first, re-tile them on the device, drop the rows.
mi355q_status check_tile16(const mi355q_format* f, uint64_t k) {
    if (f->bits != 4 || f->group_size != 64)
        return fail(MI355Q_ERR_UNSUPPORTED_FORMAT, "the TILE16 layout holds 4-bit codes in groups of 64 (got q%u g%u)",
                    (unsigned)f->bits, f->group_size);
    if (k % 128) return fail(MI355Q_ERR_SHAPE, "the TILE16 layout needs K %% 128 == 0 (K=%llu)", (unsigned long long)k);
    return MI355Q_OK;
}

mi355q_status planes_to_tile16(mi355q_weight* w) {
    w->layout = MI355Q_LAYOUT_PLANES;
    const mi355q::WView v = w->view();
    w->tiles_bytes = (size_t)((w->n + 15) / 16) * (w->k / 128) * 1152;
    MI355Q_HIP(hipMalloc(&w->tiles, w->tiles_bytes));
    if (mi355q_status st = launch_tile16_pack(nullptr, v, (uint32_t*)w->tiles)) return st;
    MI355Q_HIP(hipStreamSynchronize(nullptr));
    (void)hipFree(w->codes);  w->codes = nullptr; w->sz = nullptr; w->codes_bytes = 0;
    (void)hipFree(w->scales); w->scales = nullptr;
    (void)hipFree(w->biases); w->biases = nullptr;
    w->layout = MI355Q_LAYOUT_TILE16;
    return MI355Q_OK;
}

mi355q_status need_ctx(mi355q_context* ctx) {
    if (!ctx) return fail(MI355Q_ERR_NULL_HANDLE, "context is null");
    hipError_t e = hipSetDevice(ctx->device);
    if (e != hipSuccess) return fail(MI355Q_ERR_DEVICE, "hipSetDevice failed: %s", hipGetErrorString(e));
    return MI355Q_OK;
}

}  // namespace

namespace mi355q {
// hipFuncSetAttribute belongs to a function on one device: remember the largest size asked per (function, device)
mi355q_status raise_lds_limit(const void* kernel, size_t lds_bytes) {
    static std::mutex mu;
    static std::unordered_map<uint64_t, size_t> raised;
    int device = 0;
    MI355Q_HIP(hipGetDevice(&device));
    const uint64_t key = (uint64_t)(uintptr_t)kernel * 64u + (uint64_t)(device & 63);
    std::lock_guard<std::mutex> lock(mu);
    auto it = raised.find(key);
    if (it != raised.end() && it->second >= lds_bytes) return MI355Q_OK;
    MI355Q_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
    raised[key] = lds_bytes;
    return MI355Q_OK;
}
}  // namespace mi355q

extern "C" {

// ---------------------------------------------------------------------------------- context
mi355q_status mi355q_context_create(int device_index, mi355q_context** out) {
    if (!out) return fail(MI355Q_ERR_INVALID_ARGUMENT, "context out pointer is null");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
        return fail(MI355Q_ERR_DEVICE, "no HIP device available (%s); this library has no CPU path",
                    e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    if (device_index < 0 || device_index >= count)
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "device index %d out of range [0,%d)", device_index, count);
    MI355Q_HIP(hipSetDevice(device_index));
    mi355q_context* ctx = new (std::nothrow) mi355q_context;
    if (!ctx) return fail(MI355Q_ERR_OUT_OF_MEMORY, "host allocation failed");
    std::memset(ctx, 0, sizeof *ctx);
    ctx->device = device_index;
    e = hipGetDeviceProperties(&ctx->props, device_index);
    if (e != hipSuccess) {
        delete ctx;
        return fail(MI355Q_ERR_DEVICE, "hipGetDeviceProperties failed: %s", hipGetErrorString(e));
    }
    if (std::strncmp(ctx->props.gcnArchName, "gfx950", 6) != 0) {
        std::string arch = ctx->props.gcnArchName;
        delete ctx;
        return fail(MI355Q_ERR_DEVICE, "device arch %s is not gfx950; the kernels are built for MI355X only",
                    arch.c_str());
    }
    if (mi355q_status st = resolve_static_keys(device_index)) {     // the device is current
        delete ctx;
        return st;
    }
    e = hipMalloc((void**)&ctx->argmax_scratch, 256);
    if (e == hipSuccess) e = hipMemset(ctx->argmax_scratch, 0, 256);
    if (e == hipSuccess) e = hipMalloc((void**)&ctx->argmax_partials, (size_t)(kArgmaxPartialCapacity + kArgmaxStandaloneKeys) * 8);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&ctx->scratch_event, hipEventDisableTiming);
    if (e != hipSuccess) {
        if (ctx->scratch_event) (void)hipEventDestroy(ctx->scratch_event);
        if (ctx->argmax_scratch) (void)hipFree(ctx->argmax_scratch);
        if (ctx->argmax_partials) (void)hipFree(ctx->argmax_partials);
        delete ctx;
        return fail(MI355Q_ERR_DEVICE, "scratch allocation failed: %s", hipGetErrorString(e));
    }
    *out = ctx;
    return MI355Q_OK;
}

mi355q_status mi355q_context_scratch_bytes(mi355q_context* ctx, uint64_t out_bytes[3]) {
    if (!ctx || !out_bytes) return fail(MI355Q_ERR_NULL_HANDLE, "context or output is null");
    out_bytes[0] = ctx->workspace_bytes;
    out_bytes[1] = ctx->split_bytes;
    out_bytes[2] = ctx->gated_bytes;
    return MI355Q_OK;
}

void mi355q_probe_wide_shape(uint32_t tile_rows, uint32_t k_parts) { gemm_wide_force_shape(tile_rows, k_parts); }

mi355q_status mi355q_context_set_library_use(mi355q_context* ctx, int enabled) {
    if (!ctx) return fail(MI355Q_ERR_NULL_HANDLE, "context is null");
    ctx->dense_library_forbidden = !enabled;
    return MI355Q_OK;
}

mi355q_status mi355q_context_destroy(mi355q_context* ctx) {
    if (!ctx) return fail(MI355Q_ERR_NULL_HANDLE, "context is null");
    (void)hipSetDevice(ctx->device);
    (void)hipDeviceSynchronize();
    mi355q::dense_library_release(ctx);
    if (ctx->scratch_event) (void)hipEventDestroy(ctx->scratch_event);
    if (ctx->argmax_scratch) (void)hipFree(ctx->argmax_scratch);
    if (ctx->argmax_partials) (void)hipFree(ctx->argmax_partials);
    if (ctx->workspace) (void)hipFree(ctx->workspace);
    if (ctx->split_buffer) (void)hipFree(ctx->split_buffer);
    if (ctx->gated_buffer) (void)hipFree(ctx->gated_buffer);
    for (int i = 0; i < ctx->retired_count; i++) (void)hipFree(ctx->retired[i]);
    delete ctx;
    return MI355Q_OK;
}

mi355q_status mi355q_device_query(mi355q_context* ctx, mi355q_device_info* out) {
    if (!ctx) return fail(MI355Q_ERR_NULL_HANDLE, "context is null");
    if (!out) return fail(MI355Q_ERR_INVALID_ARGUMENT, "out pointer is null");
    std::memset(out, 0, sizeof *out);
    std::snprintf(out->name, sizeof out->name, "%s", ctx->props.name);
    std::snprintf(out->arch, sizeof out->arch, "%s", ctx->props.gcnArchName);
    out->compute_units = ctx->props.multiProcessorCount;
    out->wavefront_size = ctx->props.warpSize;
    out->lds_bytes_per_workgroup = (int32_t)ctx->props.sharedMemPerBlock;
    out->hbm_bytes = ctx->props.totalGlobalMem;
    out->hbm_peak_gbps = 8000.0;
    out->mfma_bf16_peak_tflops = 2500.0;
    return MI355Q_OK;
}

// ------------------------------------------------------------------------------ device memory
mi355q_status mi355q_buffer_alloc(mi355q_context* ctx, size_t bytes, void** out_dev) {
    if (mi355q_status s = need_ctx(ctx)) return s;
    if (!out_dev || bytes == 0) return fail(MI355Q_ERR_INVALID_ARGUMENT, "bad buffer_alloc arguments");
    MI355Q_HIP(hipMalloc(out_dev, bytes));
    return MI355Q_OK;
}

mi355q_status mi355q_buffer_free(mi355q_context* ctx, void* dev) {
    if (mi355q_status s = need_ctx(ctx)) return s;
    if (!dev) return MI355Q_OK;
    MI355Q_HIP(hipFree(dev));
    return MI355Q_OK;
}

mi355q_status mi355q_buffer_upload(mi355q_context* ctx, void* dst_dev, const void* src_host, size_t bytes) {
    if (mi355q_status s = need_ctx(ctx)) return s;
    if (!dst_dev || !src_host) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null pointer in buffer_upload");
    if (bytes == 0) return MI355Q_OK;
    MI355Q_HIP(hipMemcpy(dst_dev, src_host, bytes, hipMemcpyHostToDevice));
    return MI355Q_OK;
}

mi355q_status mi355q_buffer_download(mi355q_context* ctx, void* dst_host, const void* src_dev, size_t bytes) {
    if (mi355q_status s = need_ctx(ctx)) return s;
    if (!dst_host || !src_dev) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null pointer in buffer_download");
    if (bytes == 0) return MI355Q_OK;
    MI355Q_HIP(hipMemcpy(dst_host, src_dev, bytes, hipMemcpyDeviceToHost));
    return MI355Q_OK;
}

__global__ void fill_words_kernel(uint32_t* dst, uint32_t word, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = word;
}

// A fill kernel rather than hipMemsetAsync, so that callers may capture it in a HIP graph.
mi355q_status mi355q_buffer_fill(mi355q_context* ctx, void* stream, void* dst_dev, uint32_t word, size_t n_words) {
    if (mi355q_status s = need_ctx(ctx)) return s;
    if (!dst_dev) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null pointer in buffer_fill");
    if (n_words == 0) return MI355Q_OK;
    size_t blocks = (n_words + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    fill_words_kernel<<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>((uint32_t*)dst_dev, word, n_words);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

// ------------------------------------------------------------------------- streams and events
mi355q_status mi355q_stream_create(mi355q_context* ctx, void** out_stream) {
    if (mi355q_status s = need_ctx(ctx)) return s;
    if (!out_stream) return fail(MI355Q_ERR_INVALID_ARGUMENT, "stream out pointer is null");
    hipStream_t st;
    MI355Q_HIP(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));  // default priority
    *out_stream = (void*)st;
    return MI355Q_OK;
}
mi355q_status mi355q_stream_destroy(mi355q_context* ctx, void* stream) {
    if (mi355q_status s = need_ctx(ctx)) return s;
    if (stream && ctx->scratch_pending && ctx->scratch_stream == (hipStream_t)stream && !ctx->scratch_marked) {
        // the stream that last used the scratch goes: if it still holds work, an event takes its place
        if (hipStreamQuery((hipStream_t)stream) != hipErrorNotReady) {
            (void)hipGetLastError();
            ctx->scratch_pending = false;
        } else if (hipEventRecord(ctx->scratch_event, (hipStream_t)stream) == hipSuccess) {
            ctx->scratch_marked = true;
            ctx->scratch_stream = (hipStream_t)(uintptr_t)1;       // (no live stream: a new one may get the old address)
        } else {
            (void)hipGetLastError();
            ctx->scratch_pending = false;
        }
    }
    if (stream) MI355Q_HIP(hipStreamDestroy((hipStream_t)stream));
    return MI355Q_OK;
}
mi355q_status mi355q_stream_synchronize(mi355q_context* ctx, void* stream) {
    if (mi355q_status s = need_ctx(ctx)) return s;
    MI355Q_HIP(hipStreamSynchronize((hipStream_t)stream));
    return MI355Q_OK;
}
mi355q_status mi355q_event_create(mi355q_context* ctx, void** out_event) {
    if (mi355q_status s = need_ctx(ctx)) return s;
    if (!out_event) return fail(MI355Q_ERR_INVALID_ARGUMENT, "event out pointer is null");
    hipEvent_t ev;
    MI355Q_HIP(hipEventCreate(&ev));
    *out_event = (void*)ev;
    return MI355Q_OK;
}
mi355q_status mi355q_event_destroy(mi355q_context* ctx, void* event) {
    if (mi355q_status s = need_ctx(ctx)) return s;
    if (event) MI355Q_HIP(hipEventDestroy((hipEvent_t)event));
    return MI355Q_OK;
}
mi355q_status mi355q_event_record(mi355q_context* ctx, void* event, void* stream) {
    if (mi355q_status s = need_ctx(ctx)) return s;
    if (!event) return fail(MI355Q_ERR_NULL_HANDLE, "event is null");
    MI355Q_HIP(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
    return MI355Q_OK;
}
mi355q_status mi355q_event_synchronize(mi355q_context* ctx, void* event) {
    if (mi355q_status s = need_ctx(ctx)) return s;
    if (!event) return fail(MI355Q_ERR_NULL_HANDLE, "event is null");
    MI355Q_HIP(hipEventSynchronize((hipEvent_t)event));
    return MI355Q_OK;
}
mi355q_status mi355q_event_elapsed_ms(mi355q_context* ctx, void* start, void* stop, float* out_ms) {
    if (mi355q_status s = need_ctx(ctx)) return s;
    if (!start || !stop || !out_ms) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null argument in event_elapsed_ms");
    MI355Q_HIP(hipEventElapsedTime(out_ms, (hipEvent_t)start, (hipEvent_t)stop));
    return MI355Q_OK;
}

// ------------------------------------------------------------------------------- host repack
mi355q_status mi355q_repack_mlx_to_staf(uint8_t scheme_identifier, size_t n_rows, size_t packed_words_per_row,
                                        const uint32_t* codes_host, const void* scales_host,
                                        const void* biases_host, mi355q_dtype sb_dtype,
                                        uint8_t* out_blocks_host, size_t out_capacity) {
    const mi355q_format* f = find_format_scheme(scheme_identifier);
    if (!f) return fail(MI355Q_ERR_UNSUPPORTED_FORMAT, "unsupported scheme 0x%02x", scheme_identifier);
    if (!codes_host || !scales_host || !biases_host || !out_blocks_host)
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "null pointer in repack_mlx_to_staf");
    if ((int)sb_dtype < 0 || (int)sb_dtype > 2) return fail(MI355Q_ERR_INVALID_ARGUMENT, "bad scale dtype");
    // K from the packed width, as the converter derives it: bytesPerRow*8/bits
    const size_t k = packed_words_per_row * 32 / f->bits;
    if (k == 0 || (packed_words_per_row * 32) % f->bits)
        return fail(MI355Q_ERR_SHAPE, "packed width %zu words is not a whole number of %u-bit codes",
                    packed_words_per_row, (unsigned)f->bits);
    if (mi355q_status s = check_shape(f, n_rows, k)) return s;
    const size_t need = n_rows * (k / f->group_size) * f->bytes_per_block;
    if (out_capacity < need)
        return fail(MI355Q_ERR_SIZE_MISMATCH, "output capacity %zu < required %zu bytes", out_capacity, need);
    repack_rows(f, n_rows, k, codes_host, scales_host, biases_host, (int)sb_dtype, out_blocks_host);
    return MI355Q_OK;
}

// ------------------------------------------------------------------------------ weight handles
mi355q_status mi355q_weight_prepare_mlx(mi355q_context* ctx, uint8_t scheme_identifier, uint64_t n_rows,
                                        uint64_t k, const uint32_t* codes_host, const void* scales_host,
                                        const void* biases_host, mi355q_dtype sb_dtype,
                                        mi355q_layout layout, mi355q_weight** out) {
    if (!out) return fail(MI355Q_ERR_INVALID_ARGUMENT, "weight out pointer is null");
    *out = nullptr;
    if (mi355q_status s = need_ctx(ctx)) return s;
    const mi355q_format* f = find_format_scheme(scheme_identifier);
    if (!f) return fail(MI355Q_ERR_UNSUPPORTED_FORMAT, "unsupported scheme 0x%02x", scheme_identifier);
    if (!codes_host || !scales_host || !biases_host) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null plane pointer");
    if ((int)sb_dtype < 0 || (int)sb_dtype > 2) return fail(MI355Q_ERR_INVALID_ARGUMENT, "bad scale dtype");
    if (layout != MI355Q_LAYOUT_STAF_BLOCKS && layout != MI355Q_LAYOUT_PLANES && layout != MI355Q_LAYOUT_TILE16)
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "bad layout");
    if (mi355q_status s = check_shape(f, n_rows, k)) return s;
    if (layout == MI355Q_LAYOUT_TILE16)
        if (mi355q_status s = check_tile16(f, k)) return s;
    if ((k * f->bits) % 32)
        return fail(MI355Q_ERR_SHAPE, "MLX planes need K*bits to be a whole number of 32-bit words (K=%llu bits=%u)",
                    (unsigned long long)k, (unsigned)f->bits);
    mi355q_weight* w = new_weight(ctx, f, n_rows, k);
    if (!w) return fail(MI355Q_ERR_OUT_OF_MEMORY, "host allocation failed");
    w->owns = 1;
    w->layout = (uint8_t)layout;
    const size_t groups = (size_t)n_rows * (k / f->group_size);
    mi355q_status st = MI355Q_OK;
    if (layout == MI355Q_LAYOUT_STAF_BLOCKS) {
        std::vector<uint8_t> blocks(groups * f->bytes_per_block);
        repack_rows(f, n_rows, k, codes_host, scales_host, biases_host, (int)sb_dtype, blocks.data());
        w->sb_dtype = MI355Q_F16;
        w->blocks_bytes = blocks.size();
        st = upload_new(&w->blocks, blocks.data(), blocks.size());
    } else {
        w->sb_bytes = groups * 2;
        {
            if (sb_dtype == MI355Q_F32) {  // normalised to f16 like the converter
                std::vector<uint16_t> s16(groups), z16(groups);
                for (size_t i = 0; i < groups; i++) {
                    s16[i] = host_sb_as_f16(scales_host, i, MI355Q_F32);
                    z16[i] = host_sb_as_f16(biases_host, i, MI355Q_F32);
                }
                w->sb_dtype = MI355Q_F16;
                st = upload_new(&w->scales, s16.data(), w->sb_bytes);
                if (st == MI355Q_OK) st = upload_new(&w->biases, z16.data(), w->sb_bytes);
            } else if (sb_dtype == MI355Q_BF16) {  // kept as bf16, holding the values the converter's f16 would hold
                std::vector<uint16_t> sb(groups), zb(groups);
                for (size_t i = 0; i < groups; i++) {
                    sb[i] = host_bf16_through_f16(((const uint16_t*)scales_host)[i]);
                    zb[i] = host_bf16_through_f16(((const uint16_t*)biases_host)[i]);
                }
                w->sb_dtype = MI355Q_BF16;
                st = upload_new(&w->scales, sb.data(), w->sb_bytes);
                if (st == MI355Q_OK) st = upload_new(&w->biases, zb.data(), w->sb_bytes);
            } else {
                w->sb_dtype = (uint8_t)sb_dtype;
                st = upload_new(&w->scales, scales_host, w->sb_bytes);
                if (st == MI355Q_OK) st = upload_new(&w->biases, biases_host, w->sb_bytes);
            }
        }
    }
    if (st == MI355Q_OK && layout != MI355Q_LAYOUT_STAF_BLOCKS) st = build_rows(w, codes_host);
    if (st == MI355Q_OK && layout == MI355Q_LAYOUT_TILE16) st = planes_to_tile16(w);
    if (st != MI355Q_OK) {
        mi355q_weight_destroy(w);
        return st;
    }
    *out = w;
    return MI355Q_OK;
}

mi355q_status mi355q_weight_prepare_staf(mi355q_context* ctx, uint8_t scheme_identifier, uint64_t n_rows,
                                         uint64_t k, const uint8_t* blocks_host, size_t payload_bytes,
                                         mi355q_layout layout, mi355q_weight** out) {
    if (!out) return fail(MI355Q_ERR_INVALID_ARGUMENT, "weight out pointer is null");
    *out = nullptr;
    if (mi355q_status s = need_ctx(ctx)) return s;
    const mi355q_format* f = find_format_scheme(scheme_identifier);
    if (!f) return fail(MI355Q_ERR_UNSUPPORTED_FORMAT, "unsupported scheme 0x%02x", scheme_identifier);
    if (!blocks_host) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null block pointer");
    if (layout != MI355Q_LAYOUT_STAF_BLOCKS && layout != MI355Q_LAYOUT_PLANES && layout != MI355Q_LAYOUT_TILE16)
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "bad layout");
    if (mi355q_status s = check_shape(f, n_rows, k)) return s;
    if (layout == MI355Q_LAYOUT_TILE16)
        if (mi355q_status s = check_tile16(f, k)) return s;
    const size_t groups = (size_t)n_rows * (k / f->group_size);
    if (payload_bytes != groups * f->bytes_per_block)
        return fail(MI355Q_ERR_SIZE_MISMATCH, "payload is %zu bytes, expected %zu", payload_bytes,
                    groups * f->bytes_per_block);
    if (layout != MI355Q_LAYOUT_STAF_BLOCKS && (k * f->bits) % 32)
        return fail(MI355Q_ERR_SHAPE, "the planes layout needs K*bits to be a whole number of 32-bit words");
    mi355q_weight* w = new_weight(ctx, f, n_rows, k);
    if (!w) return fail(MI355Q_ERR_OUT_OF_MEMORY, "host allocation failed");
    w->owns = 1;
    w->layout = (uint8_t)layout;
    w->sb_dtype = MI355Q_F16;
    mi355q_status st;
    std::vector<uint8_t> planes_codes;           // de-interleaved code plane (host), PLANES only
    if (layout == MI355Q_LAYOUT_STAF_BLOCKS) {
        w->blocks_bytes = payload_bytes;
        st = upload_new(&w->blocks, blocks_host, payload_bytes);
    } else {
        const size_t bpr = k / f->group_size;
        const size_t row_bytes = k * f->bits / 8, group_bytes = (size_t)f->group_size * f->bits / 8;
        std::vector<uint8_t>& codes = planes_codes;
        codes.resize((size_t)n_rows * row_bytes);
        std::vector<uint16_t> s16(groups), z16(groups);
        for (size_t r = 0; r < n_rows; r++)
            for (size_t b = 0; b < bpr; b++) {
                const uint8_t* src = blocks_host + (r * bpr + b) * f->bytes_per_block;
                std::memcpy(&s16[r * bpr + b], src, 2);
                std::memcpy(&z16[r * bpr + b], src + 2, 2);
                std::memcpy(codes.data() + r * row_bytes + b * group_bytes, src + 4, group_bytes);
            }
        w->sb_bytes = groups * 2;
        st = upload_new(&w->scales, s16.data(), w->sb_bytes);
        if (st == MI355Q_OK) st = upload_new(&w->biases, z16.data(), w->sb_bytes);
    }
    if (st == MI355Q_OK && layout != MI355Q_LAYOUT_STAF_BLOCKS) st = build_rows(w, planes_codes.data());
    if (st == MI355Q_OK && layout == MI355Q_LAYOUT_TILE16) st = planes_to_tile16(w);
    if (st != MI355Q_OK) {
        mi355q_weight_destroy(w);
        return st;
    }
    *out = w;
    return MI355Q_OK;
}

mi355q_status mi355q_weight_wrap_staf(mi355q_context* ctx, uint8_t scheme_identifier, uint64_t n_rows,
                                      uint64_t k, const void* blocks_dev, size_t payload_bytes,
                                      mi355q_weight** out) {
    if (!out) return fail(MI355Q_ERR_INVALID_ARGUMENT, "weight out pointer is null");
    *out = nullptr;
    if (!ctx) return fail(MI355Q_ERR_NULL_HANDLE, "context is null");
    const mi355q_format* f = find_format_scheme(scheme_identifier);
    if (!f) return fail(MI355Q_ERR_UNSUPPORTED_FORMAT, "unsupported scheme 0x%02x", scheme_identifier);
    if (!blocks_dev) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null device pointer");
    if (mi355q_status s = check_shape(f, n_rows, k)) return s;
    const size_t need = (size_t)n_rows * (k / f->group_size) * f->bytes_per_block;
    if (payload_bytes != need)
        return fail(MI355Q_ERR_SIZE_MISMATCH, "payload is %zu bytes, expected %zu", payload_bytes, need);
    if ((uintptr_t)blocks_dev % 4)
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "STAF payload must be 4-byte aligned on the device");
    mi355q_weight* w = new_weight(ctx, f, n_rows, k);
    if (!w) return fail(MI355Q_ERR_OUT_OF_MEMORY, "host allocation failed");
    w->layout = MI355Q_LAYOUT_STAF_BLOCKS;
    w->sb_dtype = MI355Q_F16;
    w->blocks = const_cast<void*>(blocks_dev);
    w->blocks_bytes = payload_bytes;
    *out = w;
    return MI355Q_OK;
}

mi355q_status mi355q_weight_wrap_planes(mi355q_context* ctx, uint8_t scheme_identifier, uint64_t n_rows,
                                        uint64_t k, const void* codes_dev, const void* scales_dev,
                                        const void* biases_dev, mi355q_dtype sb_dtype, mi355q_weight** out) {
    if (!out) return fail(MI355Q_ERR_INVALID_ARGUMENT, "weight out pointer is null");
    *out = nullptr;
    if (!ctx) return fail(MI355Q_ERR_NULL_HANDLE, "context is null");
    const mi355q_format* f = find_format_scheme(scheme_identifier);
    if (!f) return fail(MI355Q_ERR_UNSUPPORTED_FORMAT, "unsupported scheme 0x%02x", scheme_identifier);
    if (!codes_dev || !scales_dev || !biases_dev) return fail(MI355Q_ERR_INVALID_ARGUMENT, "null device pointer");
    if (sb_dtype != MI355Q_F16 && sb_dtype != MI355Q_BF16)
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "device scale/bias planes must be f16 or bf16");
    if (mi355q_status s = check_shape(f, n_rows, k)) return s;
    if ((k * f->bits) % 32) return fail(MI355Q_ERR_SHAPE, "K*bits must be a whole number of 32-bit words");
    if ((uintptr_t)codes_dev % 4 || (uintptr_t)scales_dev % 2 || (uintptr_t)biases_dev % 2)
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "misaligned plane pointer");
    mi355q_weight* w = new_weight(ctx, f, n_rows, k);
    if (!w) return fail(MI355Q_ERR_OUT_OF_MEMORY, "host allocation failed");
    w->layout = MI355Q_LAYOUT_PLANES;
    w->sb_dtype = (uint8_t)sb_dtype;
    w->codes = const_cast<void*>(codes_dev);
    w->scales = const_cast<void*>(scales_dev);
    w->biases = const_cast<void*>(biases_dev);
    w->codes_bytes = (size_t)n_rows * (k * f->bits / 32) * 4;
    w->sb_bytes = (size_t)n_rows * (k / f->group_size) * 2;
    // the borrowed planes stay where they are; the packed (scale, bias) words are an extra owned buffer
    if (hipSetDevice(ctx->device) != hipSuccess) {
        delete w;
        return fail(MI355Q_ERR_DEVICE, "hipSetDevice failed");
    }
    if (mi355q_status st = build_sz_plane(w)) {
        if (w->sz) (void)hipFree(w->sz);
        delete w;
        return st;
    }
    *out = w;
    return MI355Q_OK;
}

mi355q_status mi355q_weight_query(const mi355q_weight* w, mi355q_weight_info* out) {
    if (!w) return fail(MI355Q_ERR_NULL_HANDLE, "weight handle is null");
    if (!out) return fail(MI355Q_ERR_INVALID_ARGUMENT, "out pointer is null");
    std::memset(out, 0, sizeof *out);
    out->scheme_identifier = w->fmt.scheme_identifier;
    out->bits = w->fmt.bits;
    out->layout = w->layout;
    out->sb_dtype = w->sb_dtype;
    out->group_size = w->fmt.group_size;
    out->n_rows = w->n;
    out->k = w->k;
    out->weight_bytes = w->n * (w->k / w->fmt.group_size) * w->fmt.bytes_per_block;
    out->blocks_dev = w->blocks;
    out->codes_dev = w->codes;
    out->scales_dev = w->scales;
    out->biases_dev = w->biases;
    out->owns_memory = w->owns;
    return MI355Q_OK;
}

mi355q_status mi355q_weight_destroy(mi355q_weight* w) {
    if (!w) return fail(MI355Q_ERR_NULL_HANDLE, "weight handle is null");
    (void)hipSetDevice(w->ctx->device);
    if (w->owns) {
        if (w->blocks) (void)hipFree(w->blocks);
        if (w->codes) (void)hipFree(w->codes);
        if (w->scales) (void)hipFree(w->scales);
        if (w->biases) (void)hipFree(w->biases);
        if (w->tiles) (void)hipFree(w->tiles);
    }
    if (w->sz && w->sz_separate) (void)hipFree(w->sz);
    delete w;
    return MI355Q_OK;
}

// ---- STAF container on the device ----------------------------------------------------------------
mi355q_status mi355q_staf_upload(mi355q_context* ctx, const mi355q_staf* staf, void** base_dev_out, uint64_t* bytes_out) {
    if (!base_dev_out) return fail(MI355Q_ERR_INVALID_ARGUMENT, "output pointer is null");
    *base_dev_out = nullptr;
    if (!ctx || !staf) return fail(MI355Q_ERR_NULL_HANDLE, "context or container is null");
    uint64_t bytes = 0;
    const void* region = mi355q_staf_payload_region(staf, &bytes);
    void* dev = nullptr;
    if (mi355q_status st = mi355q_buffer_alloc(ctx, (size_t)bytes, &dev)) return st;
    // pageable host memory (the file mapping): a synchronous copy, staged by the runtime
    const hipError_t e = hipMemcpy(dev, region, (size_t)bytes, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        (void)hipFree(dev);
        return fail(MI355Q_ERR_DEVICE, "copy of the payload region failed: %s", hipGetErrorString(e));
    }
    *base_dev_out = dev;
    if (bytes_out) *bytes_out = bytes;
    return MI355Q_OK;
}

mi355q_status mi355q_staf_weight(mi355q_context* ctx, const mi355q_staf* staf, const void* base_dev, const char* name,
                                 mi355q_layout layout, mi355q_weight** out) {
    if (!out) return fail(MI355Q_ERR_INVALID_ARGUMENT, "weight out pointer is null");
    *out = nullptr;
    if (!ctx || !staf) return fail(MI355Q_ERR_NULL_HANDLE, "context or container is null");
    mi355q_staf_entry t;
    if (mi355q_status st = mi355q_staf_find(staf, name, &t)) return st;
    const mi355q_format* f = find_format_scheme(t.scheme_identifier);
    if (!f) return fail(MI355Q_ERR_UNSUPPORTED_FORMAT, "tensor '%s' has scheme 0x%02x, which is not a packed format", name,
                        (unsigned)t.scheme_identifier);
    if (t.dimension_count != 2)
        return fail(MI355Q_ERR_SHAPE, "tensor '%s' has %u dimensions; a packed projection has 2", name, (unsigned)t.dimension_count);
    const uint64_t n = t.shape[0], k = (uint64_t)t.shape[1] * 32 / f->bits;      // STAFWriter.swift:250-258
    if (layout == MI355Q_LAYOUT_STAF_BLOCKS) {
        if (!base_dev) return fail(MI355Q_ERR_INVALID_ARGUMENT, "the row-major layout needs the uploaded payload region");
        return mi355q_weight_wrap_staf(ctx, t.scheme_identifier, n, k, (const char*)base_dev + t.buffer_offset,
                                       (size_t)t.payload_size, out);
    }
    uint64_t bytes = 0;
    const uint8_t* region = (const uint8_t*)mi355q_staf_payload_region(staf, &bytes);
    return mi355q_weight_prepare_staf(ctx, t.scheme_identifier, n, k, region + t.buffer_offset, (size_t)t.payload_size,
                                      layout, out);
}

}  // extern "C"
