// Prefill GEMM on the matrix cores (placeholder translation unit: selection reports "not
// eligible" until the MFMA kernels land, so every shape takes the small-M kernels).
#include "common.h"

namespace mi355q {

bool gemm_mfma_eligible(const WView&, int, uint32_t, uint32_t) { return false; }

mi355q_status launch_qgemm_mfma(hipStream_t, const mi355q_context*, const WView&, const void*, int, void*, int,
                                uint32_t, uint32_t, uint32_t) {
    return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "MFMA GEMM kernel is not built");
}

mi355q_status launch_gemm_bf16_mfma(hipStream_t, const mi355q_context*, const void*, int, const uint16_t*, void*,
                                    int, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t) {
    return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "MFMA GEMM kernel is not built");
}

}  // namespace mi355q
