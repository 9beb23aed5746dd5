// Instantiates the split-plane GEMV kernels for one bit width (QBITS) and exports one launcher.
// Included by gemv_q{2,3,4,5,6,8}.hip so that the widths compile in parallel.
#include "gemv_rows.inl"

namespace mi355q {

namespace {

template <typename K>
mi355q_status launch_kernel(K kern, hipStream_t s, const GemvArgs& a, uint32_t grid, uint32_t block, size_t lds) {
    if (lds > 64 * 1024) {
        // opt in to more than the default 64 KiB of dynamic LDS (gfx950 has 160 KiB per CU): once per kernel and device
        if (mi355q_status st = raise_lds_limit((const void*)kern, lds)) return st;
    }
    kern<<<dim3(grid), dim3(block), lds, s>>>(a);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

// ---- the general kernel (any row length, small batches) ---------------------------------------------------
template <int BITS, int GROUP, int R, int MT, bool ARGMAX, int WAVES, int D, int XREG>
mi355q_status launch_one(hipStream_t s, const GemvArgs& a, const GemvCfg& c) {
    if (c.xa) return launch_kernel(gemv_planes_kernel<BITS, GROUP, R, MT, ARGMAX, WAVES, D, XREG, 1>, s, a, c.grid, WAVES * 64, c.lds);
    return launch_kernel(gemv_planes_kernel<BITS, GROUP, R, MT, ARGMAX, WAVES, D, XREG, 0>, s, a, c.grid, WAVES * 64, c.lds);
}

#define MI355Q_TRY(R_, MT_, AM_, WV_, D_, XR_)                                                            \
    if (c.r == R_ && c.mt == MT_ && c.argmax == AM_ && c.waves == WV_ && c.depth == D_ && c.xreg == XR_) \
        return launch_one<BITS, GROUP, R_, MT_, AM_, WV_, D_, XR_>(s, a, c);

template <int BITS, int GROUP>
mi355q_status launch_general(hipStream_t s, const GemvArgs& a, const GemvCfg& c) {
    // M == 1 (decode): register-resident activations for rows of one K-step, LDS-resident otherwise
    MI355Q_TRY(1, 1, false, 4, 2, 1) MI355Q_TRY(1, 1, false, 4, 4, 1)
    MI355Q_TRY(1, 1, false, 4, 2, 0) MI355Q_TRY(1, 1, false, 4, 4, 0)
    MI355Q_TRY(1, 1, false, 8, 2, 0) MI355Q_TRY(1, 1, false, 8, 4, 0)
    MI355Q_TRY(1, 1, false, 16, 2, 0) MI355Q_TRY(1, 1, false, 16, 4, 0)
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

// ---- the static-structure kernel (M == 1, rows of 1, 2, 3, 4 or 7 K-steps) -----------------------------------
template <int BITS, int GROUP, int NCT, int BR, int WAVES>
mi355q_status launch_rows(hipStream_t s, const GemvArgs& a, const GemvCfg& c) {
    const bool sbbf = a.sb_dtype == MI355Q_BF16;
    const uint32_t block = WAVES * 64;
    if (c.mt > 1) {
        if (!c.argmax && !c.gated && !c.xa) {
            if constexpr (gemv_rows_has_batch(BITS, GROUP, NCT, BR, 2)) {
                if (c.mt == 2) {
                    if (sbbf) return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 0, true, false, false, 2>, s, a, c.grid, block, c.lds);
                    return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 0, false, false, false, 2>, s, a, c.grid, block, c.lds);
                }
            }
            if constexpr (gemv_rows_has_batch(BITS, GROUP, NCT, BR, 3)) {
                if (c.mt == 3) {
                    if (sbbf) return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 0, true, false, false, 3>, s, a, c.grid, block, c.lds);
                    return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 0, false, false, false, 3>, s, a, c.grid, block, c.lds);
                }
                if (c.mt == 4) {
                    if (sbbf) return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 0, true, false, false, 4>, s, a, c.grid, block, c.lds);
                    return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 0, false, false, false, 4>, s, a, c.grid, block, c.lds);
                }
            }
        }
        return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no %d-row variant of the row kernel for q%d g%d steps=%d rows=%d", c.mt, BITS, GROUP, NCT, BR);
    }
    if (c.gated) {
        if (c.argmax) return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the gated row kernel has no arg-max tail");
        if (c.xa) {
            if constexpr (gemv_rows_has_f16(BITS, GROUP)) {
                if (sbbf) return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 1, true, false, true>, s, a, c.grid, block, c.lds);
                return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 1, false, false, true>, s, a, c.grid, block, c.lds);
            }
            return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no f16 variant of the row kernel for q%d g%d", BITS, GROUP);
        }
        if (sbbf) return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 0, true, false, true>, s, a, c.grid, block, c.lds);
        return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 0, false, false, true>, s, a, c.grid, block, c.lds);
    }
    if (c.argmax) {
        if constexpr (gemv_rows_has_argmax(NCT, BR)) {
            if (c.xa) {
                if constexpr (gemv_rows_has_f16(BITS, GROUP)) {
                    if (sbbf) return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 1, true, true>, s, a, c.grid, block, c.lds);
                    return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 1, false, true>, s, a, c.grid, block, c.lds);
                }
            } else {
                if (sbbf) return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 0, true, true>, s, a, c.grid, block, c.lds);
                return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 0, false, true>, s, a, c.grid, block, c.lds);
            }
        }
        return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no fused arg-max variant of the row kernel for q%d g%d steps=%d rows=%d", BITS, GROUP, NCT, BR);
    }
    if (c.xa) {
        if constexpr (gemv_rows_has_f16(BITS, GROUP)) {
            if (sbbf) return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 1, true, false>, s, a, c.grid, block, c.lds);
            return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 1, false, false>, s, a, c.grid, block, c.lds);
        }
        return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no f16 variant of the row kernel for q%d g%d", BITS, GROUP);
    }
    if (sbbf) return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 0, true, false>, s, a, c.grid, block, c.lds);
    return launch_kernel(gemv_rows_kernel<BITS, GROUP, NCT, BR, WAVES, 0, false, false>, s, a, c.grid, block, c.lds);
}

#define MI355Q_TRY_ROWS(NCT_, BR_) \
    if (c.nct == NCT_ && c.br == BR_) return launch_rows<BITS, GROUP, NCT_, BR_, gemv_rows_waves(NCT_)>(s, a, c);

template <int BITS, int GROUP>
mi355q_status launch_group(hipStream_t s, const GemvArgs& a, const GemvCfg& c) {
    if (!c.rows) return launch_general<BITS, GROUP>(s, a, c);
    if constexpr (gemv_rows_has_format(BITS, GROUP)) {
        MI355Q_TRY_ROWS(1, 1) MI355Q_TRY_ROWS(1, 2) MI355Q_TRY_ROWS(1, 4) MI355Q_TRY_ROWS(1, 8)
        MI355Q_TRY_ROWS(2, 1) MI355Q_TRY_ROWS(2, 2) MI355Q_TRY_ROWS(2, 4)
        MI355Q_TRY_ROWS(3, 1) MI355Q_TRY_ROWS(3, 2)
        MI355Q_TRY_ROWS(4, 1) MI355Q_TRY_ROWS(4, 2)
        if constexpr (BITS != 8) { MI355Q_TRY_ROWS(7, 1) }   // 8-bit codes at sixteen wavefronts do not fit the register file
    }
    return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no row-kernel variant for q%d g%d steps=%d rows=%d", BITS, GROUP, c.nct, c.br);
}

#undef MI355Q_TRY_ROWS

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
