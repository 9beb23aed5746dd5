// Instantiates the split-plane GEMV kernels for one bit width (QBITS) and exports one launcher.
// Included by gemv_q{2,3,4,5,6,8}.hip so that the widths compile in parallel.
#include "gemv_planes.inl"

namespace mi355q {

namespace {

template <int BITS, int GROUP, int R, int MT, bool ARGMAX, int WAVES, int D, int XREG>
mi355q_status launch_one(hipStream_t s, const GemvArgs& a, uint32_t grid, size_t lds) {
    auto kern = gemv_planes_kernel<BITS, GROUP, R, MT, ARGMAX, WAVES, D, XREG>;
    if (lds > 64 * 1024) {
        // opt in to more than the default 64 KiB of dynamic LDS (gfx950 has 160 KiB per CU)
        MI355Q_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    }
    kern<<<dim3(grid), dim3(WAVES * 64), lds, s>>>(a);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

#define MI355Q_TRY(R_, MT_, AM_, WV_, D_, XR_)                                                            \
    if (c.r == R_ && c.mt == MT_ && c.argmax == AM_ && c.waves == WV_ && c.depth == D_ && c.xreg == XR_) \
        return launch_one<BITS, GROUP, R_, MT_, AM_, WV_, D_, XR_>(s, a, c.grid, c.lds);

template <int BITS, int GROUP>
mi355q_status launch_group(hipStream_t s, const GemvArgs& a, const GemvCfg& c) {
#ifdef MI355Q_GEMV_EXPERIMENT
    // tuning build: the (R, waves, depth, xreg) grid for one format
    MI355Q_TRY(1, 1, false, 4, 2, 0) MI355Q_TRY(1, 1, false, 4, 4, 0) MI355Q_TRY(1, 1, false, 4, 8, 0)
    MI355Q_TRY(2, 1, false, 4, 2, 0) MI355Q_TRY(2, 1, false, 4, 4, 0) MI355Q_TRY(2, 1, false, 4, 8, 0)
    MI355Q_TRY(1, 1, false, 8, 2, 0) MI355Q_TRY(1, 1, false, 8, 4, 0) MI355Q_TRY(1, 1, false, 8, 8, 0)
    MI355Q_TRY(2, 1, false, 8, 2, 0) MI355Q_TRY(2, 1, false, 8, 4, 0) MI355Q_TRY(2, 1, false, 8, 8, 0)
    MI355Q_TRY(1, 1, false, 16, 2, 0) MI355Q_TRY(1, 1, false, 16, 4, 0) MI355Q_TRY(1, 1, false, 16, 8, 0)
    MI355Q_TRY(1, 1, false, 4, 2, 1) MI355Q_TRY(1, 1, false, 4, 4, 1) MI355Q_TRY(1, 1, false, 4, 8, 1)
    MI355Q_TRY(1, 1, false, 4, 2, 2) MI355Q_TRY(1, 1, false, 4, 4, 2) MI355Q_TRY(1, 1, false, 4, 8, 2)
    MI355Q_TRY(1, 1, false, 8, 2, 1) MI355Q_TRY(1, 1, false, 8, 4, 1) MI355Q_TRY(1, 1, false, 8, 8, 1)
    MI355Q_TRY(1, 1, false, 8, 2, 2) MI355Q_TRY(1, 1, false, 8, 4, 2) MI355Q_TRY(1, 1, false, 8, 8, 2)
    MI355Q_TRY(1, 1, false, 16, 2, 1) MI355Q_TRY(1, 1, false, 16, 4, 1) MI355Q_TRY(1, 1, false, 16, 8, 1)
    MI355Q_TRY(1, 1, false, 16, 2, 2) MI355Q_TRY(1, 1, false, 16, 4, 2) MI355Q_TRY(1, 1, false, 16, 8, 2)
#else
    // M == 1 (decode): register-resident activations for rows of one K-step, LDS-resident otherwise
    MI355Q_TRY(1, 1, false, 4, 2, 1) MI355Q_TRY(1, 1, false, 4, 4, 1)
    MI355Q_TRY(1, 1, false, 4, 2, 0) MI355Q_TRY(1, 1, false, 4, 4, 0)
    MI355Q_TRY(1, 1, false, 8, 2, 0) MI355Q_TRY(1, 1, false, 8, 4, 0)
    MI355Q_TRY(1, 1, false, 16, 2, 0) MI355Q_TRY(1, 1, false, 16, 4, 0)
#endif
    // the same with the fused arg-max tail (LM head)
    MI355Q_TRY(1, 1, true, 4, 2, 1) MI355Q_TRY(1, 1, true, 4, 4, 1)
    MI355Q_TRY(1, 1, true, 4, 2, 0) MI355Q_TRY(1, 1, true, 4, 4, 0)
    MI355Q_TRY(1, 1, true, 8, 2, 0) MI355Q_TRY(1, 1, true, 8, 4, 0)
    MI355Q_TRY(1, 1, true, 16, 2, 0) MI355Q_TRY(1, 1, true, 16, 4, 0)
    // small batches (M = 2, 3-4)
    constexpr int R2 = gemv_batch_rows(BITS, GROUP, 2), R4 = gemv_batch_rows(BITS, GROUP, 4);
    constexpr int D2 = gemv_batch_depth(BITS, GROUP, 2), D4 = gemv_batch_depth(BITS, GROUP, 4);
    MI355Q_TRY(R2, 2, false, 4, D2, 0) MI355Q_TRY(R4, 4, false, 4, D4, 0)
    return fail(MI355Q_ERR_KERNEL_NOT_FOUND,
                "no split-plane GEMV variant for q%d g%d R=%d MT=%d argmax=%d waves=%d depth=%d xreg=%d", BITS, GROUP,
                c.r, c.mt, (int)c.argmax, c.waves, c.depth, c.xreg);
}

#undef MI355Q_TRY

}  // namespace

#define MI355Q_GEMV_LAUNCHER_NAME2(b) launch_gemv_planes_q##b
#define MI355Q_GEMV_LAUNCHER_NAME(b) MI355Q_GEMV_LAUNCHER_NAME2(b)

mi355q_status MI355Q_GEMV_LAUNCHER_NAME(QBITS)(hipStream_t s, const GemvArgs& a, int group, const GemvCfg& c) {
    switch (group) {
#if QBITS == 2 || QBITS == 3 || QBITS == 6
    case 16: return launch_group<QBITS, 16>(s, a, c);
#endif
#if QBITS != 4
    case 32: return launch_group<QBITS, 32>(s, a, c);
#endif
    case 64: return launch_group<QBITS, 64>(s, a, c);
#if QBITS == 4 || QBITS == 8
    case 128: return launch_group<QBITS, 128>(s, a, c);
#endif
    default: break;
    }
    return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no split-plane GEMV for q%d g%d", QBITS, group);
}

}  // namespace mi355q
