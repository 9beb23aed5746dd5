// Decode GEMV that reads STAF interleaved blocks in place ([f16 scale][f16 zero][packed codes], one
// block per group), bf16 or f16 activations, 1 <= M <= 8: the path of a weight that was wrapped or uploaded
// from a model file without being repacked.
//
//   * a block is 4 + GROUP*BITS/8 bytes (36 for q4 g64), so a lane cannot fetch "its" block with one
//     aligned vector load.  A wavefront instead copies a span of 64 consecutive blocks of one row --
//     one contiguous byte range -- from memory straight into LDS with 128-bit direct-to-LDS loads
//     (no register staging), and every lane then reads its own block back with 32-bit LDS reads:
//     1 + GROUP*BITS/32 dwords at a stride that is odd for the common formats (q4 and q8 at every
//     group size, every width at g64), so their reads are free of bank conflicts;
//   * a wavefront owns a run of consecutive rows and keeps D spans in flight in a private LDS ring;
//     the direct-to-LDS loads are invisible to the compiler's wait-counter bookkeeping, so the
//     kernel waits on the vector-memory counter itself: every span is exactly NDMA load
//     instructions, each issued with at least one lane active (lanes past the end of the buffer read
//     a clamped address; their bytes belong to blocks no lane uses), which makes "at most NDMA
//     loads outstanding per younger span" mean "the oldest span has landed";
//   * arithmetic is that of the split-plane kernel: activations staged once per workgroup in LDS in
//     the pair order the unpacker produces together with the per-block sums, 2..6-bit codes turned
//     into bf16 (128+q) pairs for v_dot2_f32_bf16, 8-bit codes through fp32 FMA, the affine form
//     s*sum(q*x) + z*sum(x) per block, one wavefront reduction per output row.  With f16 activations every
//     width, 8 bits included, becomes f16 (1024+q) pairs (exact: one unit in the last place is 1 from 1024
//     to 2048) for v_dot2_f32_f16.
//
// Replaces gemv_q{b}_g{g} reading the STAF payload directly
// (Sources/MetalCompiler/Generator/MetalSourceGenerator+Quantized.swift:496-575; block layout:
// Sources/MetalCompiler/STAF/QuantizationFormat.swift:1284-1312).
#include "gemv_planes.inl"

namespace mi355q {

namespace {

#define MI355Q_LDS_PTR(p) ((__attribute__((address_space(3))) uint8_t*)(p))

// One launch covers up to three weight matrices that share K, format and activations (q+k+v, gate+up): wavefronts
// are dealt to the matrices whole, matrix i owns the wavefronts [wave_end[i-1], wave_end[i]).
struct StafArgs {
    const uint8_t* blocks[kGemvMaxSegments];
    void* y[kGemvMaxSegments];                 // [M, y_stride[i]] in y_dtype (may be null when only logits are wanted)
    uint32_t wave_end[kGemvMaxSegments];       // cumulative wavefront counts; unused entries repeat the last
    uint32_t seg_rows[kGemvMaxSegments];       // N_i
    uint32_t y_stride[kGemvMaxSegments];
    const uint16_t* x;       // bf16 or f16 [M, x_stride] (the kernel's XA argument says which)
    float* logits;           // optional fp32 [N] copy (M == 1, single matrix)
    unsigned long long* scratch;   // ARGMAX only: one packed (ordered value, ~row) key per workgroup
    uint64_t row_bytes;      // blocks_per_row * bytes per block (a multiple of 16)
    uint32_t k, m;
    uint32_t x_stride, y_dtype;
    uint32_t blocks_per_row;
    uint32_t nsp;            // spans per row = ceil(blocks_per_row / 64)
    uint32_t rows_per_span;  // 64 / blocks_per_row when a row is a power-of-two fraction of a span (then nsp == 1), else 1
    uint32_t rows_per_wave;  // a multiple of rows_per_span
};

template <int BITS, int GROUP>
struct StafGeo {
    static constexpr int WPB = GROUP * BITS / 32;           // code words per block
    static constexpr int BW = 1 + WPB;                      // dwords per block
    static constexpr int SPAN = 64 * BW * 4;                // bytes of 64 blocks
    static constexpr int NDMA = (SPAN + 1023) / 1024;       // 64 lanes x 16 bytes per load instruction
    static constexpr int SLOT = SPAN;                       // ring slot (a multiple of 256 bytes)
    static constexpr int Q = GROUP / 8;                     // staged activation pieces (8 elements each) per block
};

// XREG: rows are one span long (K <= 64 * GROUP) and M == 1: every lane keeps its block's activations and their sum
// in registers instead of re-reading them from LDS at every row.
// XA = 0: bf16 activations.  XA = 1: f16 activations.
template <int BITS, int GROUP, int MT, int WAVES, int D, bool ARGMAX, bool XREG, int XA>
__global__ __launch_bounds__(WAVES * 64) void gemv_staf_kernel(const StafArgs a) {
    static_assert(!XREG || MT == 1, "register-resident activations are for M == 1");
    using G = StafGeo<BITS, GROUP>;
    constexpr int WPB = G::WPB, BW = G::BW, SPAN = G::SPAN, NDMA = G::NDMA, SLOT = G::SLOT, Q = G::Q;
    constexpr bool DOT2 = BITS <= 6 || XA == 1;             // 128 + q is exact in bf16 up to 6 bits, 1024 + q in f16 up to 8
    constexpr float OFS = XA == 1 ? 1024.0f : 128.0f;
    constexpr uint32_t kOnes = XA == 1 ? 0x3C003C00u : 0x3F803F80u;
    static_assert(GROUP * BITS % 32 == 0 && GROUP % 8 == 0, "blocks are whole words");
    static_assert(NDMA * (D - 1) < 64, "the vector-memory counter has 6 bits");

    extern __shared__ __align__(16) uint8_t lds[];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t NSP = a.nsp;
    u32x4* const xs = (u32x4*)lds;                                          // [m][span][piece][lane]
    float* const sxs = (float*)(lds + (size_t)MT * NSP * Q * 1024);         // [m][span][lane]
    uint8_t* const ring = lds + (size_t)MT * NSP * (Q * 1024 + 256) + (size_t)wave * D * SLOT;
    const uint32_t ring_lds = (uint32_t)(uintptr_t)MI355Q_LDS_PTR(ring);

    // the matrix this wavefront works on (scalar select chain); wavefronts past the last matrix fall on rows past
    // its end: their loads are clamped and nothing is stored
    const uint32_t gw = blockIdx.x * WAVES + wave;
    const uint32_t seg = gw < a.wave_end[0] ? 0u : (gw < a.wave_end[1] ? 1u : 2u);
    // Mask arithmetic over all three entries instead of a select: a select of kernel-argument fields becomes one
    // scalar load from a selected address, which waits for the load of wave_end first -- a second trip to the constant
    // cache in front of the first weight loads.
    const uint32_t k0 = seg == 0 ? ~0u : 0u, k1 = seg == 1 ? ~0u : 0u, k2 = seg == 2 ? ~0u : 0u;
    const uint64_t q0 = seg == 0 ? ~0ull : 0ull, q1 = seg == 1 ? ~0ull : 0ull, q2 = seg == 2 ? ~0ull : 0ull;
    const uint32_t first_wave = (a.wave_end[0] & k1) | (a.wave_end[1] & k2);
    const uint8_t* const seg_blocks =
        (const uint8_t*)(((uintptr_t)a.blocks[0] & q0) | ((uintptr_t)a.blocks[1] & q1) | ((uintptr_t)a.blocks[2] & q2));
    void* const seg_y = (void*)(((uintptr_t)a.y[0] & q0) | ((uintptr_t)a.y[1] & q1) | ((uintptr_t)a.y[2] & q2));
    const uint32_t seg_n = (a.seg_rows[0] & k0) | (a.seg_rows[1] & k1) | (a.seg_rows[2] & k2);
    const uint32_t seg_ys = (a.y_stride[0] & k0) | (a.y_stride[1] & k1) | (a.y_stride[2] & k2);
    // the remaining arguments of the prologue, asked for here so that they arrive with the same batch of scalar loads
    asm volatile("" ::"s"(a.row_bytes), "s"(a.rows_per_wave), "s"(a.rows_per_span), "s"(a.blocks_per_row), "s"(a.m), "s"(a.x), "s"(a.x_stride));
    const uint64_t last_chunk = (uint64_t)seg_n * a.row_bytes - 16;    // last whole 16-byte chunk of the matrix
    const uint32_t row0 = gw < a.wave_end[kGemvMaxSegments - 1] ? (gw - first_wave) * a.rows_per_wave : seg_n;
    // Short rows share a span: RPS consecutive rows (contiguous in memory) fill the 64 lanes, lane l holding block
    // l % blocks_per_row of row l / blocks_per_row.
    const uint32_t RPS = a.rows_per_span;
    const uint32_t nsteps = a.rows_per_wave / RPS * NSP;

    // ---- 1. the first D spans go out before anything else ----------------------------------------
    uint32_t irow = 0, isp = 0;                              // next span to issue
    auto issue = [&](uint32_t slot) {
        uint32_t row = row0 + irow;
        row = row < seg_n ? row : seg_n - 1;                 // rows past the end of the matrix reload its last row
        const uint64_t base = (uint64_t)row * a.row_bytes + (uint64_t)isp * SPAN + (uint64_t)lane * 16;
#pragma unroll
        for (int i = 0; i < NDMA; i++) {
            uint64_t off = base + (uint64_t)i * 1024;
            off = off < last_chunk ? off : last_chunk;
            const uint8_t* g = seg_blocks + off;
            const uint32_t l = ring_lds + slot * SLOT + i * 1024;
            // the last instruction of a span covers only part of the wavefront: the other lanes are masked
            // off (never all of them, so the instruction is issued and counted every time)
            if ((i + 1) * 1024 <= SPAN || lane < (uint32_t)(SPAN - i * 1024) / 16)
                asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(l) : "memory");
        }
        if (++isp == NSP) { isp = 0; irow += RPS; }
    };
#pragma unroll
    for (int j = 0; j < D; j++)
        if ((uint32_t)j < nsteps) issue(j);

    // ---- 2. activations: loaded, permuted into pair order, summed per block, parked in LDS ---------
    const uint32_t ntasks = a.m * NSP;
    for (uint32_t t = wave; t < ntasks; t += WAVES) {
        const uint32_t m = t / NSP, sp = t - m * NSP;
        const uint32_t b = RPS > 1 ? lane % a.blocks_per_row : sp * 64 + lane;
        const bool valid = b < a.blocks_per_row;
        const u32x4* src = (const u32x4*)(a.x + (size_t)m * a.x_stride + (valid ? (size_t)b * GROUP : 0));
        uint32_t d[GROUP / 2];
#pragma unroll
        for (int i = 0; i < Q; i++) {
            const u32x4 v = src[i];
            d[4 * i + 0] = valid ? v.x : 0; d[4 * i + 1] = valid ? v.y : 0;
            d[4 * i + 2] = valid ? v.z : 0; d[4 * i + 3] = valid ? v.w : 0;
        }
        auto pairw = [&](auto I) -> uint32_t {
            constexpr int i = decltype(I)::value;
            constexpr int e0 = pair_elem<BITS>(i, 0), e1 = pair_elem<BITS>(i, 1);
            if constexpr (e1 == e0 + 1 && (e0 & 1) == 0) return d[e0 >> 1];
            else return __builtin_amdgcn_perm(d[e1 >> 1], d[e0 >> 1], (e0 & 1) ? 0x07060302u : 0x05040100u);
        };
        static_for<Q>([&](auto P) {
            constexpr int i = decltype(P)::value;
            u32x4 o;
            o.x = pairw(std::integral_constant<int, 4 * i + 0>{});
            o.y = pairw(std::integral_constant<int, 4 * i + 1>{});
            o.z = pairw(std::integral_constant<int, 4 * i + 2>{});
            o.w = pairw(std::integral_constant<int, 4 * i + 3>{});
            xs[((size_t)(m * NSP + sp) * Q + i) * 64 + lane] = o;
        });
        float sx = 0.0f;
#pragma unroll
        for (int j = 0; j < GROUP / 2; j++) sx = dot2_x<XA>(d[j], kOnes, sx);
        sxs[(size_t)(m * NSP + sp) * 64 + lane] = sx;
    }
    __syncthreads();

    u32x4 xr[XREG ? Q : 1];
    float sxr = 0.0f;
    if constexpr (XREG) {
#pragma unroll
        for (int p = 0; p < Q; p++) xr[p] = xs[(size_t)p * 64 + lane];
        sxr = sxs[lane];
    }

    uint32_t k_magic = XA == 1 ? 0x64006400u : 0x43004300u;  // f16 pair (1024.0, 1024.0) or bf16 pair (128.0, 128.0)
    uint32_t k_mask = BITS == 4 ? 0x000F000Fu : 0x00030003u;
    asm volatile("" : "+v"(k_magic));
    asm volatile("" : "+s"(k_mask));

    float acc[MT], res[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) acc[m] = res[m] = 0.0f;

    unsigned long long best = 0ull;  // ARGMAX, per lane: packed (ordered value, ~row); 0 = nothing seen
    auto flush = [&](uint32_t first_local, uint32_t count) {
        const uint32_t row = row0 + first_local + lane;
        if (lane < count && row < seg_n) {
#pragma unroll
            for (int m = 0; m < MT; m++) {
                if ((uint32_t)m < a.m) {
                    if (seg_y) {
                        const size_t o = (size_t)m * seg_ys + row;
                        if (a.y_dtype == MI355Q_F32) ((float*)seg_y)[o] = res[m];
                        else if (a.y_dtype == MI355Q_BF16) ((uint16_t*)seg_y)[o] = f32_to_bf16_rne(res[m]);
                        else ((uint16_t*)seg_y)[o] = f32_to_f16_rne(res[m]);
                    }
                    if (a.logits && m == 0) a.logits[row] = res[m];
                }
            }
            if constexpr (ARGMAX) {
                const float v = res[0];
                if (v > -INFINITY) {                         // NaN and -inf never contribute
                    const uint32_t u = __float_as_uint(v + 0.0f);   // -0 -> +0
                    const uint32_t key = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
                    const unsigned long long pk = ((unsigned long long)key << 32) | (unsigned long long)(0xFFFFFFFFu - row);
                    best = pk > best ? pk : best;
                }
            }
        }
    };

    // ---- 3. one span per step: wait for the oldest slot, unpack it, refill it ------------------------
    uint32_t lrow = 0, sp = 0;
    for (uint32_t step = 0; step < nsteps; step++) {
        const uint32_t slot = step % D;
        // spans issued after this one: D-1 in the steady state, fewer over the last steps
        const uint32_t younger = nsteps - 1 - step < (uint32_t)(D - 1) ? nsteps - 1 - step : (uint32_t)(D - 1);
        static_for<D>([&](auto Y) {
            constexpr int y = decltype(Y)::value;
            if (younger == (uint32_t)y) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NDMA * y) : "memory");
        });
        const uint32_t* blk = (const uint32_t*)(ring + (size_t)slot * SLOT) + lane * BW;
        const bool valid = RPS > 1 || sp * 64 + lane < a.blocks_per_row;
        uint32_t hdr = blk[0];
        uint32_t w[WPB];
#pragma unroll
        for (int i = 0; i < WPB; i++) w[i] = blk[1 + i];
        hdr = valid ? hdr : 0u;

        float dot[MT];
#pragma unroll
        for (int m = 0; m < MT; m++) dot[m] = 0.0f;
        static_for<Q>([&](auto P) {
            constexpr int p = decltype(P)::value;
            u32x4 xv[MT];
            if constexpr (XREG) {
                xv[0] = xr[p];
            } else {
#pragma unroll
                for (int m = 0; m < MT; m++) xv[m] = xs[((size_t)(m * NSP + sp) * Q + p) * 64 + lane];
            }
            if constexpr (DOT2) {
                uint32_t pr[4];
                if constexpr (BITS == 4) {
                    const uint32_t wv = w[p];
                    pr[0] = (wv & k_mask) | k_magic;
                    pr[1] = ((wv >> 4) & k_mask) | k_magic;
                    pr[2] = ((wv >> 8) & k_mask) | k_magic;
                    pr[3] = ((wv >> 12) & k_mask) | k_magic;
                } else if constexpr (BITS == 2) {
                    const uint32_t wv = w[p >> 1] >> (8 * (p & 1));
                    pr[0] = (wv & k_mask) | k_magic;
                    pr[1] = ((wv >> 2) & k_mask) | k_magic;
                    pr[2] = ((wv >> 4) & k_mask) | k_magic;
                    pr[3] = ((wv >> 6) & k_mask) | k_magic;
                } else {
                    static_for<4>([&](auto I) {
                        constexpr int i = decltype(I)::value;
                        const uint32_t qa = extract_code<(p * 8 + 2 * i) * BITS, BITS, WPB>(w);
                        const uint32_t qb = extract_code<(p * 8 + 2 * i + 1) * BITS, BITS, WPB>(w);
                        pr[i] = ((qb << 16) | qa) | k_magic;
                    });
                }
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    float dsum = dot[m];
                    dsum = dot2_x<XA>(pr[0], xv[m].x, dsum);
                    dsum = dot2_x<XA>(pr[1], xv[m].y, dsum);
                    dsum = dot2_x<XA>(pr[2], xv[m].z, dsum);
                    dsum = dot2_x<XA>(pr[3], xv[m].w, dsum);
                    dot[m] = dsum;
                }
            } else {
                float qf[8];
                static_for<8>([&](auto E) {
                    constexpr int e = decltype(E)::value;
                    qf[e] = (float)extract_code<(p * 8 + e) * BITS, BITS, WPB>(w);
                });
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    const uint32_t xw[4] = {xv[m].x, xv[m].y, xv[m].z, xv[m].w};
                    float dsum = dot[m];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        dsum = __builtin_fmaf(qf[2 * e], __uint_as_float(xw[e] << 16), dsum);
                        dsum = __builtin_fmaf(qf[2 * e + 1], __uint_as_float(xw[e] & 0xFFFF0000u), dsum);
                    }
                    dot[m] = dsum;
                }
            }
        });
        const float s = f16_to_f32((uint16_t)(hdr & 0xFFFFu)), z = f16_to_f32((uint16_t)(hdr >> 16));
        const float zc = DOT2 ? z - OFS * s : z;
#pragma unroll
        for (int m = 0; m < MT; m++) acc[m] += s * dot[m] + zc * (XREG ? sxr : sxs[(size_t)(m * NSP + sp) * 64 + lane]);

        // the slot's LDS reads have been consumed by the arithmetic above: it can be overwritten
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (step + D < nsteps) issue(slot);

        if (++sp == NSP) {                                   // row complete
            sp = 0;
#pragma unroll
            for (int m = 0; m < MT; m++) {
                float total;
                if (RPS == 1) {
                    total = wave_reduce_sum(acc[m]);
                    if (lane == (lrow & 63u)) res[m] = total;
                } else {
                    // sum inside each run of blocks_per_row lanes, then hand the RPS row totals to their parking lanes
                    total = acc[m];
                    for (uint32_t off = a.blocks_per_row >> 1; off > 0; off >>= 1) total += __shfl_xor(total, (int)off, 64);
                    const uint32_t park = (lane - lrow) & 63u;             // which row of this span parks here, if any
                    const float moved = __shfl(total, (int)((park & (RPS - 1)) * a.blocks_per_row), 64);
                    if (park < RPS) res[m] = moved;
                }
                acc[m] = 0.0f;
            }
            lrow += RPS;
            if ((lrow & 63u) == 0) flush(lrow - 64, 64);
        }
    }
    if (lrow & 63u) flush(lrow & ~63u, lrow & 63u);
    if constexpr (ARGMAX) {
        // wavefront maximum of the packed keys, workgroup maximum through LDS, one plain store per workgroup;
        // argmax_finish_kernel picks the token from the partial keys
        __shared__ unsigned long long s_best[WAVES];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const uint32_t hi = (uint32_t)__shfl_xor((int)(best >> 32), off, 64);
            const uint32_t lo = (uint32_t)__shfl_xor((int)(best & 0xFFFFFFFFull), off, 64);
            const unsigned long long o = ((unsigned long long)hi << 32) | lo;
            best = o > best ? o : best;
        }
        if (lane == 0) s_best[wave] = best;
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned long long m = s_best[0];
#pragma unroll
            for (int w2 = 1; w2 < WAVES; w2++) m = s_best[w2] > m ? s_best[w2] : m;
            a.scratch[blockIdx.x] = m;
        }
    }
}

constexpr int kWaves = 4;

// Ring depth and wavefronts per CU.
// Measured on MI355X (q4 g64, 14336x4096, M = 1): depth 2 with 8 wavefronts per CU 9.2 us, depth 4
// 11.1 us; 4 wavefronts per CU 11.6 us, 16 and more 9.6 us and up.
struct StafCfg { int depth; uint32_t per_cu; };
StafCfg staf_cfg() {
    return StafCfg{2, 8};
}

size_t staf_lds_bytes(uint32_t span_slot, uint32_t q, uint32_t nsp, int mt, int depth) {
    return (size_t)mt * nsp * (q * 1024 + 256) + (size_t)kWaves * depth * span_slot;
}

// When the staged activations leave room for a single workgroup per CU, its four wavefronts take the
// CU's whole share of rows (every extra workgroup would stage the activations again).
void staf_one_workgroup_per_cu(size_t lds, StafCfg& c) {
    if (lds > 80 * 1024) c.per_cu = kWaves;
}

// Rows that are a power-of-two fraction of a span (32, 16, 8 ... blocks) share one.
uint32_t staf_rows_per_span(uint32_t blocks_per_row) {
    if (blocks_per_row >= 64 || (blocks_per_row & (blocks_per_row - 1)) != 0) return 1;
    return 64 / blocks_per_row;
}

// Each wavefront owns a run of consecutive rows.
uint32_t staf_rows_per_wave(const mi355q_context* ctx, uint32_t n, const StafCfg& c) {
    const uint32_t target = (uint32_t)ctx->props.multiProcessorCount * c.per_cu;
    const uint32_t rpw = (n + target - 1) / target;
    return rpw ? rpw : 1;
}

// `total_rows`: rows of all matrices of the launch; `grid`: workgroups (the caller has dealt the wavefronts).
template <int BITS, int GROUP, int XA>
mi355q_status launch_for_format(hipStream_t s, const StafArgs& a, int mt, int depth, uint32_t grid, bool argmax) {
    using G = StafGeo<BITS, GROUP>;
    const size_t lds = staf_lds_bytes(G::SLOT, G::Q, a.nsp, mt, depth);
    const bool xreg = mt == 1 && a.nsp == 1;
    auto go = [&](auto kernel) -> mi355q_status {
        if (lds > 48 * 1024)
            if (mi355q_status st = raise_lds_limit((const void*)kernel, lds)) return st;
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(kWaves * 64), lds, s, a);
        MI355Q_HIP(hipGetLastError());
        return MI355Q_OK;
    };
    if (depth == 2) {
        if (argmax) return xreg ? go(gemv_staf_kernel<BITS, GROUP, 1, kWaves, 2, true, true, XA>)
                                : go(gemv_staf_kernel<BITS, GROUP, 1, kWaves, 2, true, false, XA>);
        switch (mt) {
        case 1: return xreg ? go(gemv_staf_kernel<BITS, GROUP, 1, kWaves, 2, false, true, XA>)
                            : go(gemv_staf_kernel<BITS, GROUP, 1, kWaves, 2, false, false, XA>);
        case 2: return go(gemv_staf_kernel<BITS, GROUP, 2, kWaves, 2, false, false, XA>);
        default: return go(gemv_staf_kernel<BITS, GROUP, 4, kWaves, 2, false, false, XA>);
        }
    }
    return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no block-layout GEMV with ring depth %d", depth);
}

mi355q_status launch_by_format(hipStream_t s, uint32_t bits, uint32_t group, const StafArgs& a, int mt, int depth,
                               uint32_t grid, bool argmax, int x_dtype) {
#define MI355Q_STAF_LAUNCH(B, GR) \
    case B * 1000 + GR: \
        return x_dtype == MI355Q_F16 ? launch_for_format<B, GR, 1>(s, a, mt, depth, grid, argmax) \
                                     : launch_for_format<B, GR, 0>(s, a, mt, depth, grid, argmax);
    switch (bits * 1000 + group) {
    MI355Q_STAF_LAUNCH(4, 64) MI355Q_STAF_LAUNCH(4, 128) MI355Q_STAF_LAUNCH(8, 32) MI355Q_STAF_LAUNCH(8, 64)
    MI355Q_STAF_LAUNCH(2, 64) MI355Q_STAF_LAUNCH(3, 64) MI355Q_STAF_LAUNCH(5, 64) MI355Q_STAF_LAUNCH(6, 64)
    MI355Q_STAF_LAUNCH(2, 16) MI355Q_STAF_LAUNCH(2, 32) MI355Q_STAF_LAUNCH(3, 32) MI355Q_STAF_LAUNCH(5, 32)
    MI355Q_STAF_LAUNCH(6, 16) MI355Q_STAF_LAUNCH(6, 32) MI355Q_STAF_LAUNCH(8, 128)
    default: break;
    }
#undef MI355Q_STAF_LAUNCH
    return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no block-layout GEMV for q%ug%u", bits, group);
}

struct StafShape { uint32_t slot, q; };
bool staf_shape(uint32_t bits, uint32_t group, StafShape& out) {
#define MI355Q_STAF_CASE(B, GR) \
    if (bits == B && group == GR) { out = {StafGeo<B, GR>::SLOT, StafGeo<B, GR>::Q}; return true; }
    MI355Q_STAF_CASE(4, 64) MI355Q_STAF_CASE(4, 128) MI355Q_STAF_CASE(8, 32) MI355Q_STAF_CASE(8, 64)
    MI355Q_STAF_CASE(2, 64) MI355Q_STAF_CASE(3, 64) MI355Q_STAF_CASE(5, 64) MI355Q_STAF_CASE(6, 64)
    MI355Q_STAF_CASE(2, 16) MI355Q_STAF_CASE(2, 32) MI355Q_STAF_CASE(3, 32) MI355Q_STAF_CASE(5, 32)
    MI355Q_STAF_CASE(6, 16) MI355Q_STAF_CASE(6, 32) MI355Q_STAF_CASE(8, 128)
#undef MI355Q_STAF_CASE
    return false;
}

constexpr size_t kStafLdsBudget = 144 * 1024;

int staf_max_mt(const WView& w, const StafShape& sh) {
    const uint32_t nsp = (w.blocks_per_row + 63) / 64;
    for (int mt = 4; mt >= 1; mt >>= 1)
        if (staf_lds_bytes(sh.slot, sh.q, nsp, mt, staf_cfg().depth) <= kStafLdsBudget) return mt;
    return 0;
}

}  // namespace

bool gemv_staf_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride) {
    if (w.layout != MI355Q_LAYOUT_STAF_BLOCKS || (x_dtype != MI355Q_BF16 && x_dtype != MI355Q_F16)) return false;
    if (m < 1 || m > 8 || !w.blocks) return false;
    StafShape sh;
    if (!staf_shape(w.bits, w.group, sh)) return false;
    if (w.k % w.group) return false;
    const uint64_t row_bytes = (uint64_t)w.blocks_per_row * w.bytes_per_block;
    if (row_bytes % 16 || (uintptr_t)w.blocks % 16) return false;   // 128-bit loads of every row
    if (x_stride % 8) return false;                                 // 128-bit activation loads
    if ((uint64_t)w.n * row_bytes < 16) return false;
    return staf_max_mt(w, sh) != 0;
}

GemvLaunchShape gemv_staf_shape(const mi355q_context* ctx, const WView& w, uint32_t m) {
    GemvLaunchShape g{};
    StafShape sh;
    if (!staf_shape(w.bits, w.group, sh)) return g;
    const int fit = staf_max_mt(w, sh);
    int mt = m >= 3 ? 4 : (int)m;
    if (mt > fit) mt = fit;
    StafCfg c = staf_cfg();
    g.lds_bytes = (uint32_t)staf_lds_bytes(sh.slot, sh.q, (w.blocks_per_row + 63) / 64, mt ? mt : 1, c.depth);
    staf_one_workgroup_per_cu(g.lds_bytes, c);
    const uint32_t rps = staf_rows_per_span(w.blocks_per_row);
    const uint32_t rows_per_wg = (staf_rows_per_wave(ctx, w.n, c) + rps - 1) / rps * rps * kWaves;
    g.grid = (w.n + rows_per_wg - 1) / rows_per_wg;
    g.block = kWaves * 64;
    g.rows_per_workgroup = rows_per_wg;
    g.kernel = "gemv_staf";
    return g;
}

// Up to three weights sharing K, format and activations in one launch; `w[0]` supplies the format, the caller has
// checked that the others match.  `token_out` selects the fused arg-max tail (one weight, M == 1).
mi355q_status launch_gemv_staf_multi(hipStream_t s, const mi355q_context* ctx, uint32_t count, const WView* w,
                                     const void* x, int x_dtype, void* const* y, const uint32_t* y_strides, int y_dtype,
                                     uint32_t m, uint32_t x_stride, float* logits_f32, int32_t* token_out,
                                     HeadKeys keys) {
    if (count < 1 || count > (uint32_t)kGemvMaxSegments)
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "1..%d weights per fused launch", kGemvMaxSegments);
    if ((uintptr_t)x % 16) return fail(MI355Q_ERR_INVALID_ARGUMENT, "activation pointer must be 16-byte aligned");
    const bool argmax = token_out != nullptr;
    if (argmax && (m != 1 || count != 1)) return fail(MI355Q_ERR_INVALID_ARGUMENT, "fused argmax needs M == 1");
    if (logits_f32 && count != 1) return fail(MI355Q_ERR_INVALID_ARGUMENT, "fp32 logits need a single weight");
    StafShape sh;
    if (!staf_shape(w[0].bits, w[0].group, sh))
        return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no block-layout GEMV for q%ug%u", w[0].bits, w[0].group);
    const int fit = staf_max_mt(w[0], sh);
    if (fit == 0) return fail(MI355Q_ERR_SHAPE, "K = %u is too long for the block-layout GEMV", w[0].k);
    uint64_t total = 0;
    for (uint32_t i = 0; i < count; i++) total += w[i].n;
    if (total > 0xFFFFFFFFull) return fail(MI355Q_ERR_SHAPE, "too many rows");
    const size_t ysz = y_dtype == MI355Q_F32 ? 4 : 2;
    StafArgs a{};
    a.row_bytes = (uint64_t)w[0].blocks_per_row * w[0].bytes_per_block;
    a.k = w[0].k;
    a.x_stride = x_stride;
    a.y_dtype = (uint32_t)y_dtype;
    a.blocks_per_row = w[0].blocks_per_row;
    a.nsp = (w[0].blocks_per_row + 63) / 64;
    a.rows_per_span = staf_rows_per_span(w[0].blocks_per_row);
    a.logits = logits_f32;
    a.scratch = keys.ptr;
    for (uint32_t m0 = 0; m0 < m;) {
        const uint32_t left = m - m0;
        int mt = left >= 3 ? 4 : (int)left;                  // 3 rows run as a 4-row launch with one row masked
        if (mt > fit) mt = fit;
        const uint32_t mm = left < (uint32_t)mt ? left : (uint32_t)mt;
        StafCfg c = staf_cfg();
        staf_one_workgroup_per_cu(staf_lds_bytes(sh.slot, sh.q, a.nsp, mt, c.depth), c);
        a.rows_per_wave = staf_rows_per_wave(ctx, (uint32_t)total, c);
        a.rows_per_wave = (a.rows_per_wave + a.rows_per_span - 1) / a.rows_per_span * a.rows_per_span;
        uint32_t waves = 0;
        for (uint32_t i = 0; i < (uint32_t)kGemvMaxSegments; i++) {
            const uint32_t j = i < count ? i : count - 1;
            if (i < count) waves += (w[i].n + a.rows_per_wave - 1) / a.rows_per_wave;
            a.blocks[i] = w[j].blocks;
            a.y[i] = y[j] ? (void*)((char*)y[j] + (size_t)m0 * y_strides[j] * ysz) : nullptr;
            a.y_stride[i] = y_strides[j];
            a.seg_rows[i] = w[j].n;
            a.wave_end[i] = waves;
        }
        const uint32_t grid = (waves + kWaves - 1) / kWaves;
        if (argmax && grid > keys.capacity) return fail(MI355Q_ERR_SHAPE, "too many workgroups for the fused argmax");
        a.x = (const uint16_t*)x + (size_t)m0 * x_stride;
        a.m = mm;
        if (mi355q_status st = launch_by_format(s, w[0].bits, w[0].group, a, mt, c.depth, grid, argmax, x_dtype)) return st;
        if (argmax) return launch_argmax_finish(s, keys.ptr, grid, token_out);
        m0 += mm;
    }
    return MI355Q_OK;
}

mi355q_status launch_gemv_staf(hipStream_t s, const mi355q_context* ctx, const WView& w, const void* x, int x_dtype,
                               void* y, int y_dtype, uint32_t m, uint32_t x_stride, uint32_t y_stride) {
    void* ys[1] = {y};
    const uint32_t strides[1] = {y_stride};
    return launch_gemv_staf_multi(s, ctx, 1, &w, x, x_dtype, ys, strides, y_dtype, m, x_stride, nullptr, nullptr, HeadKeys{});
}

}  // namespace mi355q
