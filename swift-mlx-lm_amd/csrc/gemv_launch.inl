// Instantiates the split-plane GEMV kernels for one bit width (QBITS) and exports one launcher.
// Included by gemv_q{2,3,4,5,6,8}.hip so that the widths compile in parallel.
#include "gemv_planes.inl"

namespace mi355q {

namespace {

template <int BITS, int GROUP, int R, int MT, bool ARGMAX>
mi355q_status launch_one(hipStream_t s, const GemvArgs& a, uint32_t grid, size_t lds) {
    auto kern = gemv_planes_kernel<BITS, GROUP, R, MT, ARGMAX>;
    if (lds > 64 * 1024) {
        // opt in to more than the default 64 KiB of dynamic LDS (gfx950 has 160 KiB per CU)
        MI355Q_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    }
    kern<<<dim3(grid), dim3(256), lds, s>>>(a);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

template <int BITS, int GROUP>
mi355q_status launch_group(hipStream_t s, const GemvArgs& a, int r, int mt, bool argmax, uint32_t grid, size_t lds) {
    if (mt == 1) {
        if (argmax) {
            if (r == 1) return launch_one<BITS, GROUP, 1, 1, true>(s, a, grid, lds);
            if (r == 2) return launch_one<BITS, GROUP, 2, 1, true>(s, a, grid, lds);
            if (r == 4) return launch_one<BITS, GROUP, 4, 1, true>(s, a, grid, lds);
        } else {
            if (r == 1) return launch_one<BITS, GROUP, 1, 1, false>(s, a, grid, lds);
            if (r == 2) return launch_one<BITS, GROUP, 2, 1, false>(s, a, grid, lds);
            if (r == 4) return launch_one<BITS, GROUP, 4, 1, false>(s, a, grid, lds);
        }
    } else if (!argmax) {
        if (mt == 2 && r == 2) return launch_one<BITS, GROUP, 2, 2, false>(s, a, grid, lds);
        if (mt == 4 && r == 2) return launch_one<BITS, GROUP, 2, 4, false>(s, a, grid, lds);
        if (mt == 8 && r == 1) return launch_one<BITS, GROUP, 1, 8, false>(s, a, grid, lds);
    }
    return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no split-plane GEMV variant for q%d g%d R=%d MT=%d argmax=%d", BITS,
                GROUP, r, mt, (int)argmax);
}

}  // namespace

#define MI355Q_GEMV_LAUNCHER_NAME2(b) launch_gemv_planes_q##b
#define MI355Q_GEMV_LAUNCHER_NAME(b) MI355Q_GEMV_LAUNCHER_NAME2(b)

mi355q_status MI355Q_GEMV_LAUNCHER_NAME(QBITS)(hipStream_t s, const GemvArgs& a, int group, int r, int mt,
                                               bool argmax, uint32_t grid, size_t lds) {
    switch (group) {
#if QBITS == 2 || QBITS == 3 || QBITS == 6
    case 16: return launch_group<QBITS, 16>(s, a, r, mt, argmax, grid, lds);
#endif
#if QBITS != 4
    case 32: return launch_group<QBITS, 32>(s, a, r, mt, argmax, grid, lds);
#endif
    case 64: return launch_group<QBITS, 64>(s, a, r, mt, argmax, grid, lds);
#if QBITS == 4 || QBITS == 8
    case 128: return launch_group<QBITS, 128>(s, a, r, mt, argmax, grid, lds);
#endif
    default: break;
    }
    return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no split-plane GEMV for q%d g%d", QBITS, group);
}

}  // namespace mi355q
