// Dense GEMM (bf16, f16 or fp32 operands) of the two-dispatch prefill route through hipBLASLt.
//
// The reference's second prefill route is  dequant_q{b}_g{g}_bf16  into a scratch matrix, then the platform's own
// matmul2d primitive on the dense operands (Sources/MetalCompiler/Generator/MetalSourceGenerator+Linear.swift:18-81,
// bindings Sources/MetalCompiler/Compiler/MetalPrefillStepBuilder.swift:928-955).  Here the dequantisation is this
// library's kernel and the dense product is the platform's GEMM library.  hipBLASLt is opened with dlopen on first
// use, so libmi355_qlinear.so itself has no link-time dependency on it and callers that never reach this route never
// load it; when it cannot be opened the route reports itself unavailable and the fused kernel serves the call.
//
// Operands, in the library's column-major terms:  Y^T [N x M, ld ys] = W^T-as-stored [K x N, ld K]^T * X^T [K x M, ld xs].
#include "common.h"

#include <dlfcn.h>
#include <hipblaslt/hipblaslt.h>

#include <cmath>
#include <mutex>
#include <vector>

namespace mi355q {
namespace {

struct Api {
    void* so = nullptr;
    bool tried = false;
    decltype(&hipblasLtCreate) create = nullptr;
    decltype(&hipblasLtDestroy) destroy = nullptr;
    decltype(&hipblasLtMatrixLayoutCreate) layout_create = nullptr;
    decltype(&hipblasLtMatrixLayoutDestroy) layout_destroy = nullptr;
    decltype(&hipblasLtMatmulDescCreate) desc_create = nullptr;
    decltype(&hipblasLtMatmulDescDestroy) desc_destroy = nullptr;
    decltype(&hipblasLtMatmulDescSetAttribute) desc_set = nullptr;
    decltype(&hipblasLtMatmulPreferenceCreate) pref_create = nullptr;
    decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy = nullptr;
    decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set = nullptr;
    decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic = nullptr;
    decltype(&hipblasLtMatmul) matmul = nullptr;
};

Api g_api;
std::mutex g_api_mu;

template <typename F>
bool resolve(void* so, const char* name, F& out) {
    out = (F)dlsym(so, name);
    return out != nullptr;
}

const Api* api() {
    std::lock_guard<std::mutex> lock(g_api_mu);
    if (g_api.tried) return g_api.so ? &g_api : nullptr;
    g_api.tried = true;
    void* so = dlopen("libhipblaslt.so.1", RTLD_NOW | RTLD_LOCAL);
    if (!so) so = dlopen("/opt/rocm/lib/libhipblaslt.so.1", RTLD_NOW | RTLD_LOCAL);
    if (!so) so = dlopen("libhipblaslt.so", RTLD_NOW | RTLD_LOCAL);
    if (!so) return nullptr;
    Api a;
    const bool ok = resolve(so, "hipblasLtCreate", a.create) && resolve(so, "hipblasLtDestroy", a.destroy) &&
                    resolve(so, "hipblasLtMatrixLayoutCreate", a.layout_create) &&
                    resolve(so, "hipblasLtMatrixLayoutDestroy", a.layout_destroy) &&
                    resolve(so, "hipblasLtMatmulDescCreate", a.desc_create) &&
                    resolve(so, "hipblasLtMatmulDescDestroy", a.desc_destroy) &&
                    resolve(so, "hipblasLtMatmulDescSetAttribute", a.desc_set) &&
                    resolve(so, "hipblasLtMatmulPreferenceCreate", a.pref_create) &&
                    resolve(so, "hipblasLtMatmulPreferenceDestroy", a.pref_destroy) &&
                    resolve(so, "hipblasLtMatmulPreferenceSetAttribute", a.pref_set) &&
                    resolve(so, "hipblasLtMatmulAlgoGetHeuristic", a.heuristic) &&
                    resolve(so, "hipblasLtMatmul", a.matmul);
    if (!ok) return nullptr;
    a.so = so;
    a.tried = true;
    g_api = a;
    return &g_api;
}

hipDataType data_type(int dtype) {
    return dtype == MI355Q_F32 ? HIP_R_32F : dtype == MI355Q_BF16 ? HIP_R_16BF : HIP_R_16F;
}

constexpr int kCandidates = 8;
constexpr size_t kMaxProblems = 256;     // problems remembered per context
constexpr int kCheckSamples = 64;       // result elements recomputed as plain dot products on a problem's first call

// One problem the context has met: its descriptors and the algorithm the library's heuristic ranks first.
struct Problem {
    uint32_t m, n, k, xs, ys;
    int ab_dtype, y_dtype;
    bool usable;
    hipblasLtMatmulDesc_t desc;
    hipblasLtMatrixLayout_t a, b, c;
    hipblasLtMatmulAlgo_t algo;                       // the one in use: the heuristic's first until `timed`
    hipblasLtMatmulAlgo_t ranked[kCandidates];        // what the heuristic returned, in its order
    int candidates;
    bool timed;                                       // the candidates have been timed on the device
    bool verified;                                    // the algorithm in use has been checked against plain dot products
};

}  // namespace

struct DenseLibrary {
    const Api* api;
    hipblasLtHandle_t handle;
    std::vector<Problem> problems;
    float* check;                                     // device cells: two spare, then kCheckSamples (product, magnitude,
                                                      // result) triples
    void* workspace;                                  // the library's own: kDenseLibraryWorkspace bytes, zeroed once, written
                                                      // by nothing else
};

namespace {

DenseLibrary* library_of(mi355q_context* ctx) {
    if (ctx->dense_library) return ctx->dense_library;
    if (ctx->dense_library_failed || ctx->dense_library_forbidden) return nullptr;
    const Api* a = api();
    hipblasLtHandle_t h = nullptr;
    if (!a || a->create(&h) != HIPBLAS_STATUS_SUCCESS) {
        ctx->dense_library_failed = true;
        return nullptr;
    }
    // The workspace is the library's alone and starts out zeroed: split-K algorithms keep partial results there.
    float* check = nullptr;
    void* workspace = nullptr;
    if (hipMalloc((void**)&check, (2 + 3 * kCheckSamples) * sizeof(float)) != hipSuccess ||
        hipMalloc(&workspace, kDenseLibraryWorkspace) != hipSuccess || hipMemset(workspace, 0, kDenseLibraryWorkspace) != hipSuccess) {
        (void)hipGetLastError();
        if (check) (void)hipFree(check);
        if (workspace) (void)hipFree(workspace);
        a->destroy(h);
        ctx->dense_library_failed = true;
        return nullptr;
    }
    ctx->dense_library = new DenseLibrary{a, h, {}, check, workspace};
    return ctx->dense_library;
}

__device__ __forceinline__ float dense_element(const void* p, int dtype, size_t at) {
    if (dtype == MI355Q_F32) return ((const float*)p)[at];
    if (dtype == MI355Q_BF16) return __uint_as_float((uint32_t)((const uint16_t*)p)[at] << 16);
    return (float)((const _Float16*)p)[at];
}

// kCheckSamples result elements, spread over the matrix with its corners among them, recomputed as plain fp32 dot
// products of the dense operands: one workgroup each; out[3 i ..] = (product, sum of magnitudes, what the result holds).
__global__ __launch_bounds__(256) void dense_check_kernel(const void* __restrict__ w, const void* __restrict__ x, int ab_dtype,
                                                         const void* __restrict__ y, int y_dtype, uint32_t m, uint32_t n,
                                                         uint32_t k, uint32_t xs, uint32_t ys, float* __restrict__ out) {
    const uint32_t i = blockIdx.x;
    uint32_t row, col;
    if (i < 4) { row = (i & 1) ? m - 1 : 0; col = (i & 2) ? n - 1 : 0; }
    else {
        uint32_t h = i * 2654435761u; h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
        row = h % m; col = (h >> 8) * 40503u % n;
    }
    float dot = 0.f, mag = 0.f;
    for (uint32_t t = threadIdx.x; t < k; t += 256) {
        const float p = dense_element(w, ab_dtype, (size_t)col * k + t) * dense_element(x, ab_dtype, (size_t)row * xs + t);
        dot += p; mag += p < 0.f ? -p : p;
    }
    __shared__ float part[2][256];
    part[0][threadIdx.x] = dot; part[1][threadIdx.x] = mag;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) { part[0][threadIdx.x] += part[0][threadIdx.x + s]; part[1][threadIdx.x] += part[1][threadIdx.x + s]; }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        out[3 * i] = part[0][0]; out[3 * i + 1] = part[1][0];
        out[3 * i + 2] = dense_element(y, y_dtype, (size_t)row * ys + col);
    }
}

// Whether the result in y is the product, by the samples above.  Synchronises the stream.
bool dense_result_verified(hipStream_t s, DenseLibrary* lib, int ab_dtype, const void* x, const void* w, const void* y, int y_dtype,
                           uint32_t m, uint32_t n, uint32_t k, uint32_t xs, uint32_t ys) {
    float host[3 * kCheckSamples];
    dense_check_kernel<<<dim3(kCheckSamples), dim3(256), 0, s>>>(w, x, ab_dtype, y, y_dtype, m, n, k, xs, ys, lib->check + 2);
    if (hipGetLastError() != hipSuccess || hipStreamSynchronize(s) != hipSuccess ||
        hipMemcpy(host, lib->check + 2, sizeof host, hipMemcpyDeviceToHost) != hipSuccess) return false;
    // fp32 sums in another order differ by a few 1e-6 of the magnitudes (1e-3 with 16-bit operands' products summed in
    // fp32 is far above that); a 16-bit result adds its own rounding
    const float out_step = y_dtype == MI355Q_F32 ? 0.f : y_dtype == MI355Q_BF16 ? 1.f / 128.f : 1.f / 1024.f;
    for (int i = 0; i < kCheckSamples; i++) {
        const float dot = host[3 * i], mag = host[3 * i + 1], got = host[3 * i + 2];
        const float slack = 2e-4f * mag + out_step * std::fabs(dot) + 1e-30f;
        if (!(std::fabs(got - dot) <= slack)) return false;
    }
    return true;
}

Problem* find_problem(DenseLibrary* lib, int ab_dtype, uint32_t m, uint32_t n, uint32_t k, uint32_t xs, uint32_t ys,
                      int y_dtype) {
    for (Problem& p : lib->problems)
        if (p.m == m && p.n == n && p.k == k && p.xs == xs && p.ys == ys && p.ab_dtype == ab_dtype && p.y_dtype == y_dtype)
            return &p;
    const Api* a = lib->api;
    // the oldest problems go when the list is full (their descriptors with them)
    if (lib->problems.size() >= kMaxProblems) {
        Problem& old = lib->problems.front();
        if (old.desc) a->desc_destroy(old.desc);
        if (old.a) a->layout_destroy(old.a);
        if (old.b) a->layout_destroy(old.b);
        if (old.c) a->layout_destroy(old.c);
        lib->problems.erase(lib->problems.begin());
    }
    Problem p{};
    p.m = m; p.n = n; p.k = k; p.xs = xs; p.ys = ys; p.ab_dtype = ab_dtype; p.y_dtype = y_dtype;
    const hipblasOperation_t op_t = HIPBLAS_OP_T, op_n = HIPBLAS_OP_N;
    hipblasLtMatmulPreference_t pref = nullptr;
    const uint64_t most = kDenseLibraryWorkspace;
    bool ok = a->desc_create(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS &&
              a->desc_set(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_t, sizeof op_t) == HIPBLAS_STATUS_SUCCESS &&
              a->desc_set(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof op_n) == HIPBLAS_STATUS_SUCCESS &&
              a->layout_create(&p.a, data_type(ab_dtype), k, n, k) == HIPBLAS_STATUS_SUCCESS &&
              a->layout_create(&p.b, data_type(ab_dtype), k, m, xs) == HIPBLAS_STATUS_SUCCESS &&
              a->layout_create(&p.c, data_type(y_dtype), n, m, ys) == HIPBLAS_STATUS_SUCCESS &&
              a->pref_create(&pref) == HIPBLAS_STATUS_SUCCESS &&
              a->pref_set(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &most, sizeof most) == HIPBLAS_STATUS_SUCCESS;
    if (ok) {
        hipblasLtMatmulHeuristicResult_t found[kCandidates];
        int count = 0;
        ok = a->heuristic(lib->handle, p.desc, p.a, p.b, p.c, p.c, pref, kCandidates, found, &count) == HIPBLAS_STATUS_SUCCESS;
        p.candidates = 0;
        for (int i = 0; ok && i < count; i++)
            if (found[i].state == HIPBLAS_STATUS_SUCCESS && found[i].workspaceSize <= kDenseLibraryWorkspace)
                p.ranked[p.candidates++] = found[i].algo;
        ok = ok && p.candidates > 0;
        if (ok) p.algo = p.ranked[0];
    }
    if (pref) a->pref_destroy(pref);
    p.usable = ok;
    lib->problems.push_back(p);      // an unusable problem is remembered too: the question is not asked again
    return &lib->problems.back();
}

}  // namespace

bool dense_library_serves(mi355q_context* ctx, int ab_dtype, uint32_t m, uint32_t n, uint32_t k, uint32_t x_stride,
                          uint32_t y_stride, int y_dtype) {
    DenseLibrary* lib = library_of(ctx);
    if (!lib) return false;
    return find_problem(lib, ab_dtype, m, n, k, x_stride, y_stride, y_dtype)->usable;
}

mi355q_status dense_library_gemm(hipStream_t s, mi355q_context* ctx, int ab_dtype, const void* x, const void* w_bf16,
                                 void* y, int y_dtype, uint32_t m, uint32_t n, uint32_t k, uint32_t x_stride,
                                 uint32_t y_stride, bool accumulate) {
    DenseLibrary* lib = library_of(ctx);
    if (!lib) return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the dense GEMM library (hipBLASLt) could not be opened");
    Problem* p = find_problem(lib, ab_dtype, m, n, k, x_stride, y_stride, y_dtype);
    if (!p->usable)
        return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the dense GEMM library has no algorithm for M=%u N=%u K=%u", m, n, k);
    const float one = 1.0f, zero = accumulate ? 1.0f : 0.0f;     // `zero` is beta
    // First eager call of a problem: time the candidates the heuristic ranked (its first is often not the fastest at
    // these shapes) on the caller's operands and keep the quickest.  Not while the stream is being captured: a
    // capture takes the algorithm in use, so run a problem once before capturing it.
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing(s, &capture);
    // Prompt lengths come in all sizes: the timing pass (24 products and a few synchronisations) runs once per
    // (N, K, types) and power-of-two range of M; other lengths in a range already timed keep the heuristic's first.
    if (!p->timed && p->candidates > 1 && capture == hipStreamCaptureStatusNone && !accumulate) {
        auto range = [](uint32_t rows) { uint32_t r = 0; while ((1u << r) < rows) r++; return r; };
        for (const Problem& q : lib->problems)
            if (&q != p && q.timed && q.n == n && q.k == k && q.ab_dtype == ab_dtype && q.y_dtype == y_dtype && range(q.m) == range(m)) {
                p->timed = true;
                break;
            }
    }
    if (!p->timed && p->candidates > 1 && capture == hipStreamCaptureStatusNone && !accumulate) {
        p->timed = true;
        hipEvent_t e0 = nullptr, e1 = nullptr;
        if (lib->check && hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess) {
            float best = 0.f;
            int best_i = -1;
            for (int i = 0; i < p->candidates; i++) {
                bool ran = true;
                float ms = 0.f;
                for (int rep = 0; rep < 3 && ran; rep++) {         // the first run warms up, the last two are timed
                    if (rep == 1) (void)hipEventRecord(e0, s);
                    ran = lib->api->matmul(lib->handle, p->desc, &one, w_bf16, p->a, x, p->b, &zero, y, p->c, y, p->c,
                                           &p->ranked[i], lib->workspace, kDenseLibraryWorkspace, s) == HIPBLAS_STATUS_SUCCESS;
                }
                if (!ran) continue;
                if (hipEventRecord(e1, s) != hipSuccess) continue;
                // A candidate is kept only if its result is the product: ranked algorithms have returned wrong matrices
                // (into results whose row stride is not N with a long K, every split-K algorithm does, the heuristic's
                // first among them).  Sampled elements are recomputed as plain dot products.
                if (!dense_result_verified(s, lib, ab_dtype, x, w_bf16, y, y_dtype, m, n, k, x_stride, y_stride)) continue;
                if (hipEventElapsedTime(&ms, e0, e1) != hipSuccess) continue;
                if (best_i < 0 || ms < best) { best = ms; best_i = i; }
            }
            p->verified = true;
            if (best_i < 0) {
                // not one candidate multiplies this problem right
                (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
                p->usable = false;
                return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the dense GEMM library returned wrong matrices for M=%u N=%u K=%u", m, n, k);
            }
            if (best_i >= 0) p->algo = p->ranked[best_i];
        }
        if (e0) (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
    }
    const hipblasStatus_t st = lib->api->matmul(lib->handle, p->desc, &one, w_bf16, p->a, x, p->b, &zero, y, p->c, y, p->c,
                                                &p->algo, lib->workspace, kDenseLibraryWorkspace, s);
    if (st != HIPBLAS_STATUS_SUCCESS)
        return fail(MI355Q_ERR_DEVICE, "hipblasLtMatmul failed with status %d (M=%u N=%u K=%u)", (int)st, m, n, k);
    // First eager call of a problem that timed nothing (one candidate, or no check cells): the algorithm in use is
    // checked all the same.  A wrong matrix makes the problem unusable: the caller's other routes serve it.
    if (!p->verified && capture == hipStreamCaptureStatusNone && !accumulate) {
        p->verified = true;
        if (!dense_result_verified(s, lib, ab_dtype, x, w_bf16, y, y_dtype, m, n, k, x_stride, y_stride)) {
            p->usable = false;
            return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the dense GEMM library returned a wrong matrix for M=%u N=%u K=%u", m, n, k);
        }
    }
    return MI355Q_OK;
}

void dense_library_release(mi355q_context* ctx) {
    DenseLibrary* lib = ctx->dense_library;
    if (!lib) return;
    for (Problem& p : lib->problems) {
        if (p.desc) lib->api->desc_destroy(p.desc);
        if (p.a) lib->api->layout_destroy(p.a);
        if (p.b) lib->api->layout_destroy(p.b);
        if (p.c) lib->api->layout_destroy(p.c);
    }
    if (lib->check) (void)hipFree(lib->check);
    if (lib->workspace) (void)hipFree(lib->workspace);
    lib->api->destroy(lib->handle);
    delete lib;
    ctx->dense_library = nullptr;
}

}  // namespace mi355q
