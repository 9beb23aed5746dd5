// Decode / small-batch projection on the matrix cores over the TILE16 layout (4-bit codes, groups of
// 64), 1 <= M <= 16 activation rows per launch.
//
// Stands in for gemv_q4_g64 and, at small sequence lengths, gemm_q4_g64
// (Sources/MetalCompiler/Generator/MetalSourceGenerator+Quantized.swift:496-575 and :22-156):
//   y[m, n] = sum_g sum_{k in g} (s[n,g] * q[n,k] + z[n,g]) * x[m,k],  fp32 accumulation.
//
// TILE16 layout (built once at weight preparation, kernels_generic.hip::tile16_pack_kernel): rows are
// taken 16 at a time and K 128 codes (two groups) at a time; each (row tile, K-block) is one record
// of 1152 contiguous bytes:
//   bytes    0..1023  64 lanes x 16 bytes of codes in the order a wavefront loads them:
//                     lane = kq*16 + n (n = row in the tile, kq = 0..3); its word j (j = 0..3) holds
//                     the 8 codes at K-block offset (j/2)*64 + kq*16 + (j%2)*8 .. +8, nibbles stored
//                     as (c0,c2,c4,c6,c1,c3,c5,c7) so that (w >> 4i) & 0x000F000F is the code pair
//                     (c2i, c2i+1): the bf16 operand order of the MFMA, with no shuffle;
//   bytes 1024..1151  16 rows x 2 groups of packed (scale | bias << 16) words, [n][g].
// A wavefront reads a record with one 128-bit and one 64-bit load per lane and feeds four
// v_mfma_f32_16x16x32_bf16 per group pair: codes become bf16 (128 + q) with one and-or each, the
// activations are the A operand straight from LDS (natural order, no permutation), the matrix core
// does every multiply-add; sum(x) per group and activation row is computed once per workgroup while the
// activations are staged.  Per group the VALU applies the affine form once per kept output row:
//   acc += s * D + (z - 128 s) * SX        (D = sum (128+q) x,  SX = sum x).
// The accumulator of lane (kq, n) holds output rows m = 4 kq .. 4 kq + 3 of weight row n, so there is
// no cross-lane reduction at all; the WAVES wavefronts of a workgroup split K and add their partial
// tiles through LDS at the end.
//
// f16 activations (the reference's decode type): a row is staged as TWO bf16 rows, hi = the upper eight significant
// bits and lo = the remaining three (every f16 value, subnormals included, is their sum exactly and lies inside
// bf16's exponent range), at rows 2 m and 2 m + 1.  The matrix core then works on 2 M rows with exact products, and
// since a lane holds output rows 4 kq .. 4 kq + 3 the two partial results of a row are added in the lane that holds
// them before the store: M <= 8 rows of f16 per launch at the cost of 2 M rows of bf16.
#include "device_utils.h"

namespace mi355q {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float float2_t;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 t16_bf16x2_t;

__device__ __forceinline__ float t16_dot2(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(t16_bf16x2_t, a), __builtin_bit_cast(t16_bf16x2_t, b), acc, false);
}

struct T16Args {
    const uint32_t* tiles[kTile16MaxSegments];   // TILE16 buffers of up to three matrices sharing x
    void* y[kTile16MaxSegments];
    uint32_t tile_end[kTile16MaxSegments];       // cumulative row-tile counts; unused entries repeat the last
    uint32_t seg_rows[kTile16MaxSegments];       // N_i
    uint32_t y_stride[kTile16MaxSegments];
    const uint16_t* x;                           // bf16 or f16 [M, x_stride]
    uint32_t x_f16;                              // 1: f16 rows, staged as two bf16 rows each (ms = 2 m)
    uint32_t ms;                                 // staged rows: the M dimension the matrix core works on
    float* logits;                               // optional fp32 [N] copy (M == 1, one matrix)
    int32_t* token_out;                          // ARGMAX only
    unsigned long long* scratch;                 // ARGMAX only: one packed key per workgroup; 0 = no candidate
    uint32_t k, m, x_stride;
    uint32_t kblocks;                            // K / 128
    uint32_t blocks_per_wave;                    // K-blocks per wavefront (K split over the workgroup)
    uint32_t passes;                             // row tiles a wavefront walks, one after the other, on one staged copy of x
    uint32_t lds_row_bytes;                      // part_blocks*256 + 16: staged activation row pitch
    uint32_t y_dtype, sb_dtype;
    uint32_t parts;                              // K parts, each with workgroups of its own that stage only their columns
    uint32_t part_blocks;                        // K-blocks per part (kblocks / parts)
    float* partial;                              // K parts only: fp32 partial results [part][M][N] (one matrix)
};

constexpr int kT16RecordWords = 288;             // 1152 bytes

// MR: output rows kept per lane (1, 2 or 4): M <= MR uses lane group 0 only; M > 4 needs MR = 4.
// A workgroup of KSPLIT * TPW wavefronts covers TPW consecutive row tiles, each split over KSPLIT
// wavefronts along K; all of them share one staged copy of the activations.
template <int MR, int KSPLIT, int TPW, int D, bool ARGMAX>
__global__ __launch_bounds__(KSPLIT * TPW * 64) void gemv_tile16_kernel(T16Args a) {
    constexpr int WAVES = KSPLIT * TPW;
    extern __shared__ u32x4 smem_t16[];
    char* lds = (char*)smem_t16;
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t n_in = lane & 15, kq = lane >> 4;
    // K part of this workgroup: K-blocks [kb0, kb0 + part_blocks), activation columns [kb0 * 128, ...)
    // (the part is the grid's second dimension: nothing is loaded or divided before the first weight loads go out)
    const uint32_t part = blockIdx.y;
    const uint32_t wg = blockIdx.x;
    const uint32_t kb0 = part * a.part_blocks;
    const uint32_t kp = a.part_blocks * 128;                // activation elements this workgroup stages per row

    // ---- matrix and row tile of this wavefront in pass `pass` (scalar select chain) ---------------
    const uint32_t slice = wave % KSPLIT;                   // share of K
    struct Tile {
        const uint32_t* base;      // first record of the row tile
        void* y;
        uint32_t ys, rows, n0, nb, b_first, b_last;
        bool valid;
    };
    auto select_tile = [&](uint32_t pass) {
        Tile t;
        uint32_t gt = (wg * a.passes + pass) * TPW + wave / KSPLIT;
        t.valid = gt < a.tile_end[kTile16MaxSegments - 1];
        gt = t.valid ? gt : a.tile_end[kTile16MaxSegments - 1] - 1;      // idle wavefronts re-read the last tile
        const bool in1 = gt >= a.tile_end[0], in2 = gt >= a.tile_end[1];
        const uint32_t* const seg_tiles = in2 ? a.tiles[2] : in1 ? a.tiles[1] : a.tiles[0];
        t.y = in2 ? a.y[2] : in1 ? a.y[1] : a.y[0];
        t.ys = in2 ? a.y_stride[2] : in1 ? a.y_stride[1] : a.y_stride[0];
        t.rows = in2 ? a.seg_rows[2] : in1 ? a.seg_rows[1] : a.seg_rows[0];
        const uint32_t lt = gt - (in2 ? a.tile_end[1] : in1 ? a.tile_end[0] : 0u);
        t.n0 = lt * 16;
        const uint32_t kb_end = kb0 + a.part_blocks;
        t.b_first = kb0 + slice * a.blocks_per_wave;
        uint32_t nb = kb_end > t.b_first ? kb_end - t.b_first : 0;            // blocks this wavefront owns
        nb = nb < a.blocks_per_wave ? nb : a.blocks_per_wave;
        t.nb = t.valid ? nb : 0;
        t.b_last = t.nb ? t.b_first + t.nb - 1 : kb_end - 1;                 // clamp target (always valid)
        t.base = seg_tiles + (size_t)lt * a.kblocks * kT16RecordWords;
        return t;
    };
    Tile tile = select_tile(0);

    // ---- 1. activation loads first (vector loads return in issue order) -------------------------
    // Raw copy of the M rows into LDS, row pitch K*2 + 16 bytes (the pad spreads the 16 rows of an
    // A-fragment read over all banks).  Each thread moves up to XC 16-byte chunks per row pass.
    const uint32_t chunks = kp / 8;                         // 16-byte chunks per staged activation row
    constexpr int XC = 2;
    u32x4 xe[XC];
    auto x_row = [&](uint32_t i, uint32_t& m, uint32_t& c) {   // chunk index -> (row, chunk in row)
        if (a.m == 1) { m = 0; c = i; }                        // uniform: no division on the decode path
        else { m = i / chunks; c = i - m * chunks; }
    };
    auto x_src = [&](uint32_t idx) -> const u32x4* {        // idx over M * chunks, row-major
        const uint32_t total = a.m * chunks;
        uint32_t m, c;
        x_row(idx < total ? idx : 0, m, c);
        return (const u32x4*)(a.x + (size_t)m * a.x_stride + (size_t)kb0 * 128) + c;
    };
    auto x_dst = [&](uint32_t idx) -> u32x4* {
        uint32_t m, c;
        x_row(idx, m, c);
        return (u32x4*)(lds + (size_t)m * a.lds_row_bytes) + c;
    };
#pragma unroll
    for (int t = 0; t < XC; t++) xe[t] = *x_src(tid + t * WAVES * 64);

    // ---- 2. the first D K-blocks of this wavefront's share of the first row tile -----------------
    struct Rec { u32x4 w; u32x2 sz; };
    Rec ring[D];
    auto issue = [&](uint32_t b, Rec& r) {
        b = b < tile.b_last ? b : tile.b_last;              // unconditional, clamped
        const uint32_t* rec = tile.base + (size_t)b * kT16RecordWords;   // scalar
        r.w = *((const u32x4*)rec + lane);
        r.sz = *((const u32x2*)(rec + 256) + n_in);
    };
    static_for<D>([&](auto J) { issue(tile.b_first + decltype(J)::value, ring[decltype(J)::value]); });

    // ---- 3. stage the activations (waits only for the loads of step 1) --------------------------
    // With each 16-byte chunk goes its share of sum(x): eight consecutive lanes hold the eight chunks of one
    // 64-element group of one row, so three cross-lane adds give the group sum, kept as sxs[group][row].
    float* const sxs = (float*)(lds + (size_t)a.ms * a.lds_row_bytes);
    {
        const uint32_t total = a.m * chunks;
        auto group_sum = [&](const u32x4& v) {
            float p = t16_dot2(v.x, 0x3F803F80u, 0.0f);
            p = t16_dot2(v.y, 0x3F803F80u, p);
            p = t16_dot2(v.z, 0x3F803F80u, p);
            p = t16_dot2(v.w, 0x3F803F80u, p);
            p += dpp_f32<0xB1>(p);     // lane pairs (quad_perm [1,0,3,2]), quads ([2,3,0,1]), then the mirror image inside
            p += dpp_f32<0x4E>(p);     // eight lanes (every lane of a quad holds the quad's sum by then): no trip through
            p += dpp_f32<0x141>(p);    // LDS, an instruction each
            return p;
        };
        auto stage = [&](uint32_t idx, const u32x4& v) {
            if (a.x_f16) {                                   // wavefront-uniform
                u32x4 hi, lo;
                f16x8_to_bf16_hi_lo(v, hi, lo);
                const float ph = group_sum(hi), pl = group_sum(lo);
                if (idx < total) {
                    uint32_t m, c;
                    x_row(idx, m, c);
                    *((u32x4*)(lds + (size_t)(2 * m) * a.lds_row_bytes) + c) = hi;
                    *((u32x4*)(lds + (size_t)(2 * m + 1) * a.lds_row_bytes) + c) = lo;
                    if ((c & 7u) == 0) { sxs[(c >> 3) * 16 + 2 * m] = ph; sxs[(c >> 3) * 16 + 2 * m + 1] = pl; }
                }
                return;
            }
            const float p = group_sum(v);
            if (idx < total) {
                *x_dst(idx) = v;
                uint32_t m, c;
                x_row(idx, m, c);
                if ((c & 7u) == 0) sxs[(c >> 3) * 16 + m] = p;
            }
        };
#pragma unroll
        for (int t = 0; t < XC; t++) stage(tid + t * WAVES * 64, xe[t]);
        // whole wavefronts take part in the shuffles: the loop bound is rounded up to the workgroup size
        for (uint32_t base = XC * WAVES * 64; base < total; base += WAVES * 64) stage(base + tid, *x_src(base + tid));
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");

    // ---- 4. K loop --------------------------------------------------------------------------------
    uint32_t k_mask = 0x000F000Fu, k_magic = 0x43004300u;   // opaque: keeps (w & mask) | magic one v_and_or_b32
    asm volatile("" : "+s"(k_mask));
    asm volatile("" : "+v"(k_magic));
    floatx4_t zero4 = {0.f, 0.f, 0.f, 0.f};
    float acc[MR];
#pragma unroll
    for (int r = 0; r < MR; r++) acc[r] = 0.f;

    // A operand: lane (m = lane & 15, kq) reads 8 consecutive bf16 of activation row min(m, M-1)
    const uint32_t am = n_in < a.ms ? n_in : a.ms - 1;
    const char* const a_lane = lds + (size_t)am * a.lds_row_bytes + kq * 32;

    auto unpack = [&](uint32_t w) -> bf16x8_t {
        u32x4 p;
        p.x = (w & k_mask) | k_magic;
        p.y = ((w >> 4) & k_mask) | k_magic;
        p.z = ((w >> 8) & k_mask) | k_magic;
        p.w = ((w >> 12) & k_mask) | k_magic;
        return __builtin_bit_cast(bf16x8_t, p);
    };
    auto compute = [&](uint32_t b, const Rec& r) {
        const uint32_t bl = b - kb0;                         // block inside the staged columns
        const char* ab = a_lane + (size_t)bl * 256;          // 128 codes = 256 bytes of activations
        static_for<2>([&](auto G) {
            constexpr int g = decltype(G)::value;
            const bf16x8_t a0 = *(const bf16x8_t*)(ab + g * 128);
            const bf16x8_t a1 = *(const bf16x8_t*)(ab + g * 128 + 16);
            const bf16x8_t b0 = unpack(g == 0 ? r.w.x : r.w.z);
            const bf16x8_t b1 = unpack(g == 0 ? r.w.y : r.w.w);
            floatx4_t d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b0, zero4, 0, 0, 0);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b1, d, 0, 0, 0);
            // sum(x) of this group for output rows 4 kq .. 4 kq + MR - 1
            const float* const sxp = sxs + (size_t)(bl * 2 + g) * 16 + 4 * kq;
            float sx[MR];
            if constexpr (MR == 4) { const floatx4_t t = *(const floatx4_t*)sxp; sx[0] = t[0]; sx[1] = t[1]; sx[2] = t[2]; sx[3] = t[3]; }
            else if constexpr (MR == 2) { const float2_t t = *(const float2_t*)sxp; sx[0] = t[0]; sx[1] = t[1]; }
            else sx[0] = sxp[0];
            const uint32_t szw = g == 0 ? r.sz.x : r.sz.y;
            float s, z;
            if (a.sb_dtype == MI355Q_BF16) {                // wavefront-uniform
                asm volatile("" ::: "memory");
                s = __uint_as_float(szw << 16); z = __uint_as_float(szw & 0xFFFF0000u);
            } else {
                asm volatile("" ::: "memory");
                s = f16_to_f32((uint16_t)(szw & 0xFFFFu)); z = f16_to_f32((uint16_t)(szw >> 16));
            }
            const float zc = z - 128.0f * s;
#pragma unroll
            for (int q = 0; q < MR; q++) acc[q] += s * d[q] + zc * sx[q];
        });
    };

    const uint32_t rounds = (a.blocks_per_wave + D - 1) / D;            // same for every wavefront
    // Partial tiles of the WAVES wavefronts, [WAVES][MR][64]: a single pass writes them over the staged activations
    // once every wavefront is done reading those (the workgroup then needs no LDS beyond the activations, which
    // decides how many workgroups share a CU); several passes keep them behind the activations and their sums.
    const bool red_over_x = a.passes == 1;
    float* const red = (float*)(red_over_x ? lds : lds + (size_t)a.ms * a.lds_row_bytes + kp);
    unsigned long long best = 0ull;
    for (uint32_t pass = 0; pass < a.passes; pass++) {
        if (pass) {                                            // the first tile's loads were issued before staging
            tile = select_tile(pass);
            static_for<D>([&](auto J) { issue(tile.b_first + decltype(J)::value, ring[decltype(J)::value]); });
        }
        for (uint32_t it = 0; it < rounds; it++) {
            static_for<D>([&](auto J) {
                constexpr int j = decltype(J)::value;
                const uint32_t idx = it * D + j;            // block index inside this wavefront's share
                if (idx < tile.nb) compute(tile.b_first + idx, ring[j]);
                issue(tile.b_first + idx + D, ring[j]);
            });
        }

        // ---- 5. add the partial tiles of the wavefronts that share a row tile, store ----------------
        if (red_over_x) __syncthreads();
#pragma unroll
        for (int r = 0; r < MR; r++) { red[(wave * MR + r) * 64 + lane] = acc[r]; acc[r] = 0.f; }
        __syncthreads();
        if (slice == 0 && tile.valid) {                     // the first wavefront of each tile adds and stores
            const uint32_t row = tile.n0 + n_in;
            float vv[MR];
#pragma unroll
            for (int r = 0; r < MR; r++) {
                vv[r] = 0.f;
                for (uint32_t w2 = 0; w2 < (uint32_t)KSPLIT; w2++) vv[r] += red[((wave + w2) * MR + r) * 64 + lane];
            }
            // f16 rows: staged rows 2 m and 2 m + 1 are the two parts of activation row m (smaller part first)
            constexpr int OUT = MR >= 2 ? MR / 2 : 1;
            const bool fold = MR >= 2 && a.x_f16;
#pragma unroll
            for (int r = 0; r < MR; r++) {
                if (fold && r >= OUT) break;
                const float v = fold ? vv[(2 * r + 1) % MR] + vv[(2 * r) % MR] : vv[r];
                const uint32_t m = fold ? 2 * kq + r : 4 * kq + r;
                if (m < a.m && row < tile.rows) {
                    if (a.parts > 1) {                       // one matrix: the reduction launch converts and stores
                        a.partial[((size_t)part * a.m + m) * tile.rows + row] = v;
                        continue;
                    }
                    if (tile.y) {
                        const size_t o = (size_t)m * tile.ys + row;
                        if (a.y_dtype == MI355Q_F32) ((float*)tile.y)[o] = v;
                        else if (a.y_dtype == MI355Q_BF16) ((uint16_t*)tile.y)[o] = f32_to_bf16_rne(v);
                        else ((uint16_t*)tile.y)[o] = f32_to_f16_rne(v);
                    }
                    if (a.logits && m == 0) a.logits[row] = v;
                    if constexpr (ARGMAX) {
                        if (m == 0 && v > -INFINITY) {      // NaN and -inf never contribute
                            const uint32_t u = __float_as_uint(v + 0.0f);   // -0 -> +0
                            const uint32_t key = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
                            const unsigned long long pk = ((unsigned long long)key << 32) | (unsigned long long)(0xFFFFFFFFu - row);
                            best = pk > best ? pk : best;
                        }
                    }
                }
            }
        }
        if (pass + 1 < a.passes) __syncthreads();           // the partial tiles are read before the next pass overwrites them
    }
    if constexpr (ARGMAX) {
        // wavefront maximum of the packed (ordered value, ~row) key, workgroup maximum through LDS, one plain
        // store per workgroup; argmax_finish_kernel picks the token from the partial keys
        __shared__ unsigned long long s_best[WAVES];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const uint32_t hi = (uint32_t)__shfl_xor((int)(best >> 32), off, 64);
            const uint32_t lo = (uint32_t)__shfl_xor((int)(best & 0xFFFFFFFFull), off, 64);
            const unsigned long long o = ((unsigned long long)hi << 32) | lo;
            best = o > best ? o : best;
        }
        if (lane == 0) s_best[wave] = best;               // 0 for the wavefronts that hold no result rows
        __syncthreads();
        if (tid == 0) {
            unsigned long long m = s_best[0];
#pragma unroll
            for (int w2 = 1; w2 < WAVES; w2++) m = s_best[w2] > m ? s_best[w2] : m;
            a.scratch[blockIdx.x] = m;
        }
    }
}

// Sum of the K parts, in part order, then the conversion the single-launch form does in its epilogue.
__global__ __launch_bounds__(256) void tile16_sum_parts_kernel(const float* __restrict__ partial, uint32_t parts,
                                                               uint32_t m, uint32_t n, void* __restrict__ y,
                                                               uint32_t y_stride, uint32_t y_dtype,
                                                               float* __restrict__ logits) {
    // x over the columns of an activation row, y over the (at most 16) rows
    const uint32_t row = blockIdx.y;
    for (uint32_t col = blockIdx.x * 256 + threadIdx.x; col < n; col += gridDim.x * 256) {
        float v = 0.f;
        for (uint32_t p = 0; p < parts; p++) v += partial[((size_t)p * m + row) * n + col];
        if (y) {
            const size_t o = (size_t)row * y_stride + col;
            if (y_dtype == MI355Q_F32) ((float*)y)[o] = v;
            else if (y_dtype == MI355Q_BF16) ((uint16_t*)y)[o] = f32_to_bf16_rne(v);
            else ((uint16_t*)y)[o] = f32_to_f16_rne(v);
        }
        if (logits && row == 0) logits[col] = v;
    }
}

namespace {

constexpr size_t kT16LdsBudget = 144 * 1024;

// M staged activation rows of k elements and the sums per half block (a block: 64 bytes of a weight row, bc codes)
size_t t16_staged_bytes(uint32_t m, uint32_t k, uint32_t bc) { return (size_t)m * ((size_t)k * 2 + 16) + (size_t)(k / bc) * 128; }

// K parts of a launch: 1 when the staged activations of whole rows fit in LDS; else a power of two that divides the
// K-blocks and whose columns fit, 0 when none does.  Among those the smallest that leaves a workgroup either a small
// staged copy (two workgroups per CU) or, with one workgroup per CU, at least three row tiles to walk on it (measured,
// 14336 -> 4096: M = 8 in two parts 18.6 us, in four 14.2 us; M = 16 in four 16.4 us, in eight 17.6 us).
uint32_t t16_parts(uint32_t k, uint32_t m, uint32_t n_row_tiles, uint32_t cus, uint32_t bc = 128) {
    const uint32_t kblocks = k / bc;
    if (t16_staged_bytes(m, k, bc) <= kT16LdsBudget) return 1;
    uint32_t first_fit = 0;
    for (uint32_t p = 2; p <= 16 && kblocks % p == 0; p *= 2) {
        const size_t staged = t16_staged_bytes(m, k / p, bc);
        if (staged > kT16LdsBudget) continue;
        if (!first_fit) first_fit = p;
        if (staged <= 80 * 1024 || (uint64_t)n_row_tiles * p >= 3ull * cus) return p;
    }
    return first_fit;
}

template <int MR, int KSPLIT, int TPW, bool ARGMAX>
mi355q_status launch_t16(hipStream_t s, const T16Args& a, uint32_t grid, size_t lds) {   // grid: workgroups of one K part
    auto kern = gemv_tile16_kernel<MR, KSPLIT, TPW, 4, ARGMAX>;
    if (lds > 64 * 1024)
        if (mi355q_status st = raise_lds_limit((const void*)kern, lds)) return st;
    kern<<<dim3(grid, a.parts), dim3(KSPLIT * TPW * 64), lds, s>>>(a);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

template <int MR, bool ARGMAX>
mi355q_status launch_t16_shape(hipStream_t s, const T16Args& a, const Tile16LaunchShape& g) {
    const uint32_t ks = g.ksplit, tpw = g.tiles_per_wg;
    if (ks == 4 && tpw == 1) return launch_t16<MR, 4, 1, ARGMAX>(s, a, g.wgs_per_part, g.lds_bytes);
    if (ks == 4 && tpw == 2) return launch_t16<MR, 4, 2, ARGMAX>(s, a, g.wgs_per_part, g.lds_bytes);
    if (ks == 4 && tpw == 4) return launch_t16<MR, 4, 4, ARGMAX>(s, a, g.wgs_per_part, g.lds_bytes);
    if constexpr (!ARGMAX && MR == 4) {   // one round of workgroups with a CU's share of row tiles each (M >= 3)
        if (ks == 4 && tpw == 3) return launch_t16<MR, 4, 3, false>(s, a, g.wgs_per_part, g.lds_bytes);
        if (ks == 2 && tpw == 5) return launch_t16<MR, 2, 5, false>(s, a, g.wgs_per_part, g.lds_bytes);
        if (ks == 2 && tpw == 6) return launch_t16<MR, 2, 6, false>(s, a, g.wgs_per_part, g.lds_bytes);
        if (ks == 2 && tpw == 7) return launch_t16<MR, 2, 7, false>(s, a, g.wgs_per_part, g.lds_bytes);
        if (ks == 2 && tpw == 8) return launch_t16<MR, 2, 8, false>(s, a, g.wgs_per_part, g.lds_bytes);
    }
    if (ks == 8 && tpw == 1) return launch_t16<MR, 8, 1, ARGMAX>(s, a, g.wgs_per_part, g.lds_bytes);
    if (ks == 8 && tpw == 2) return launch_t16<MR, 8, 2, ARGMAX>(s, a, g.wgs_per_part, g.lds_bytes);
    if (ks == 16 && tpw == 1) return launch_t16<MR, 16, 1, ARGMAX>(s, a, g.wgs_per_part, g.lds_bytes);
    return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no TILE16 variant for K-split %u x %u tiles per workgroup", ks, tpw);
}

}  // namespace

bool gemv_tile16_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride) {
    if (w.layout != MI355Q_LAYOUT_TILE16 || !w.tiles || (x_dtype != MI355Q_BF16 && x_dtype != MI355Q_F16)) return false;
    const uint32_t ms = staged_rows(x_dtype, m);                      // f16 rows are staged as two bf16 rows each
    if (m < 1 || ms > 16) return false;
    if (w.bits != 4 || w.group != 64 || w.k % 128) return false;
    if (x_stride % 8) return false;                                   // 128-bit activation loads
    return t16_parts(w.k, ms, (w.n + 15) / 16, 256) != 0;             // staged activations and their group sums fit in LDS
}

uint32_t gemv_tile16_parts_for(uint32_t k, uint32_t m, uint32_t n_row_tiles, uint32_t cus, uint32_t block_codes) {
    return t16_parts(k, m, n_row_tiles, cus, block_codes);
}

uint32_t gemv_tile16_k_parts(const mi355q_context* ctx, const WView& w, uint32_t m) {
    return t16_parts(w.k, m, (w.n + 15) / 16, (uint32_t)ctx->props.multiProcessorCount);
}

Tile16LaunchShape gemv_tile16_shape(const mi355q_context* ctx, uint32_t n_row_tiles, uint32_t k_total, uint32_t m,
                                    uint32_t block_codes) {
    Tile16LaunchShape g{};
    // With K parts the launch is shaped as parts x as many row tiles of rows of K / parts codes: every workgroup
    // belongs to one part, and the workgroups of a part cover all row tiles.
    const uint32_t cus = (uint32_t)ctx->props.multiProcessorCount;
    uint32_t parts = t16_parts(k_total, m, n_row_tiles, cus, block_codes);
    if (!parts) parts = 1;
    const uint32_t k = k_total / parts;
    const uint32_t n_total_tiles = n_row_tiles * parts;
    g.parts = parts;
    const uint32_t kblocks = k / block_codes;
    // Measured on MI355X.  K split: the smallest of 4, 8, 16 that puts about eight wavefronts on
    // every CU (and leaves each wavefront at least two K-blocks).
    uint32_t ks = 4;
    while (ks < 16 && n_total_tiles * ks < cus * 8 && kblocks / (ks * 2) >= 2) ks *= 2;
    // long rows: at most 16 K-blocks per wavefront (28672 -> 8192 at M = 1: 48 us with a four-way split, 30 us
    // with sixteen; 14336 -> 4096: 13.2 / 9.4 us), which leaves the four-way split to rows of up to 8192 codes
    while (ks < 16 && kblocks / ks > 16) ks *= 2;
    // One row tile per workgroup at one activation row (two pay on 4096 -> 14336 alone, 8.99 -> 8.36 us, and cost the
    // fused gate+up launch as much: 15.0 -> 16.0 us), two up to four rows, four above, while that leaves a workgroup
    // per two CUs.  A matrix with at most one row tile per CU keeps one tile per workgroup and, when every wavefront
    // still gets two K-blocks (four up to M = 2), all sixteen wavefronts on it (14336 -> 4096 at M = 2: 12.3 -> 10.5 us;
    // 4096 -> 4096: M = 2 5.8 -> 5.1 us with eight, M = 4 6.5 -> 6.2 us, M = 8 7.6 -> 7.2 us with sixteen).
    const uint32_t want_tpw = m == 1 ? 1u : m <= 4 ? 2u : 4u;
    const uint32_t least_wgs = cus / 2;
    uint32_t tpw = 1;
    while (tpw < want_tpw && ks * tpw * 2 <= 16 && (n_total_tiles + tpw * 2 - 1) / (tpw * 2) >= least_wgs) tpw *= 2;
    if (n_total_tiles <= cus) {
        tpw = 1;
        if (kblocks / 16 >= (m >= 3 ? 2u : 4u)) ks = 16;
    }
    // The staged activations leave room for one workgroup per CU: sixteen wavefronts.  With at least three row tiles
    // per CU they take four row tiles at a time (each wavefront keeps a quarter of K: long enough a stream to fill
    // its prefetch ring) and walk further tiles in passes; with fewer, all sixteen share one row tile.
    const bool big_x = (size_t)m * ((size_t)k * 2 + 16) > 80 * 1024;
    // From three activation rows and three row tiles per CU on, exactly one round of workgroups: each takes its CU's
    // share of the row tiles at once when sixteen wavefronts can hold them two or four to a tile (28672 rows at M = 8,
    // seven tiles per CU: 21.4 us as 4 x 4 wavefronts walking two passes on 224 CUs, 17.4 us as 2 x 7 on all 256; M = 4:
    // 18.8 -> 16.3 us), else four tiles at a time in passes.
    const uint32_t tiles_per_cu = (n_total_tiles + cus - 1) / cus;
    const bool balanced = m >= 3 && n_total_tiles >= 3 * cus && tiles_per_cu <= 8;
    const bool one_wg_per_cu = balanced || (big_x && n_total_tiles >= 3 * cus);
    if (balanced) {
        tpw = tiles_per_cu;
        ks = tpw <= 4 ? 4 : 2;
    } else if (one_wg_per_cu) {
        ks = 4;
        tpw = 4;
    } else if (big_x) {
        // one workgroup per CU and fewer than three row tiles per CU: all sixteen wavefronts on one row tile, or on the
        // two or three a CU gets, so that the launch stays one round and the activations are staged once per CU
        // (q+k+v 4096 -> 6144 at M = 16, 1.5 tiles per CU: 16.8 us with one tile per workgroup, 9.9 us with two)
        tpw = tiles_per_cu < 3 || m < 3 ? (tiles_per_cu > 1 ? 2u : 1u) : 3u;
        const uint32_t most_ks = tpw == 1 ? 16u : tpw == 2 ? 8u : 4u;
        ks = tpw == 3 ? 4u : ks;
        while (ks < most_ks && kblocks / (ks * 2) >= 2) ks *= 2;
        if (ks > most_ks) ks = most_ks;
    }
    g.ksplit = ks;
    g.tiles_per_wg = tpw;
    g.waves = ks * tpw;
    g.blocks_per_wave = (kblocks + ks - 1) / ks;
    // A workgroup stages all M activation rows once.  When that is more than half of the weight bytes it streams
    // (large batches: 131 KB of activations against 37 KB of weights per row tile at M = 16, K = 4096), its
    // wavefronts walk several row tiles on the one staged copy -- as many as still leave a workgroup per CU.
    {
        const size_t staged = (size_t)m * ((size_t)k * 2 + 16);
        const size_t per_pass = (size_t)tpw * 16 * kblocks * 72 / 2;
        uint32_t want = (uint32_t)((staged + per_pass - 1) / per_pass);
        // not more than leaves one workgroup per CU; with one workgroup per CU, exactly one round of workgroups
        const uint32_t most = one_wg_per_cu ? (n_total_tiles + tpw * cus - 1) / (tpw * cus) : n_total_tiles / (tpw * cus);
        if (want > most || one_wg_per_cu) want = most;
        if (want > 16) want = 16;
        g.passes = want ? want : 1;
    }
    g.wgs_per_part = (n_row_tiles + tpw * g.passes - 1) / (tpw * g.passes);
    g.grid = g.wgs_per_part * parts;
    g.block = g.waves * 64;
    const size_t x_bytes = t16_staged_bytes(m, k, block_codes);      // rows, then sum(x) per half block: [2 kblocks][16] floats
    const size_t red_bytes = (size_t)g.waves * 4 * 64 * 4;     // partial tiles, behind the activations
    g.lds_bytes = (uint32_t)(g.passes > 1 ? x_bytes + red_bytes : (x_bytes > red_bytes ? x_bytes : red_bytes));
    return g;
}

mi355q_status launch_gemv_tile16_multi(hipStream_t s, mi355q_context* ctx, uint32_t count, const WView* w,
                                       const void* x, int x_dtype, void* const* y, const uint32_t* y_strides, int y_dtype,
                                       uint32_t m, uint32_t x_stride, float* logits_f32, int32_t* token_out,
                                       HeadKeys keys) {
    if (count < 1 || count > (uint32_t)kTile16MaxSegments)
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "1..%d weights per fused launch", kTile16MaxSegments);
    if ((uintptr_t)x % 16) return fail(MI355Q_ERR_INVALID_ARGUMENT, "activation pointer must be 16-byte aligned");
    const bool argmax = token_out != nullptr;
    if (argmax && (m != 1 || count != 1)) return fail(MI355Q_ERR_INVALID_ARGUMENT, "fused argmax needs M == 1");
    if (logits_f32 && count != 1) return fail(MI355Q_ERR_INVALID_ARGUMENT, "fp32 logits need a single weight");
    T16Args a{};
    uint32_t tiles = 0;
    for (uint32_t i = 0; i < (uint32_t)kTile16MaxSegments; i++) {
        const uint32_t j = i < count ? i : count - 1;
        if (i < count) tiles += (w[i].n + 15) / 16;
        a.tiles[i] = w[j].tiles;
        a.y[i] = y[j];
        a.y_stride[i] = y_strides[j];
        a.seg_rows[i] = w[j].n;
        a.tile_end[i] = tiles;
    }
    const uint32_t ms = staged_rows(x_dtype, m);
    if (argmax && x_dtype != MI355Q_BF16) return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "the fused head on TILE16 records reads bf16 activations");
    const Tile16LaunchShape g = gemv_tile16_shape(ctx, tiles, w[0].k, ms);
    a.x = (const uint16_t*)x;
    a.x_f16 = x_dtype == MI355Q_F16 ? 1u : 0u;
    a.ms = ms;
    a.logits = logits_f32; a.token_out = token_out; a.scratch = keys.ptr;
    a.k = w[0].k; a.m = m; a.x_stride = x_stride;
    a.kblocks = w[0].k / 128;
    a.parts = g.parts;
    a.part_blocks = a.kblocks / g.parts;
    a.blocks_per_wave = g.blocks_per_wave;
    a.passes = g.passes;
    a.lds_row_bytes = a.part_blocks * 256 + 16;
    if (g.parts > 1) {
        if (count != 1 || argmax)
            return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "rows of %u codes at M = %u are split over K parts: one matrix, no fused argmax",
                        w[0].k, m);
        if (mi355q_status st = ensure_workspace(ctx, (size_t)g.parts * m * w[0].n * sizeof(float))) return st;
        a.partial = (float*)ctx->workspace;
    }
    a.y_dtype = (uint32_t)y_dtype; a.sb_dtype = w[0].sb_dtype;
    const int mr = ms == 1 ? 1 : ms == 2 ? 2 : 4;
    if (argmax) {
        if (g.grid > keys.capacity)
            return fail(MI355Q_ERR_SHAPE, "the fused output head keeps one partial key per workgroup: %u workgroups exceed %u",
                        g.grid, keys.capacity);
        if (mi355q_status st = launch_t16_shape<1, true>(s, a, g)) return st;
        return launch_argmax_finish(s, keys.ptr, g.grid, token_out);
    }
    mi355q_status st = mr == 1 ? launch_t16_shape<1, false>(s, a, g)
                     : mr == 2 ? launch_t16_shape<2, false>(s, a, g) : launch_t16_shape<4, false>(s, a, g);
    if (st != MI355Q_OK || g.parts == 1) return st;
    uint32_t sum_wgs = (w[0].n + 255) / 256;
    if (sum_wgs > 65535u) sum_wgs = 65535u;
    tile16_sum_parts_kernel<<<dim3(sum_wgs, m), dim3(256), 0, s>>>(a.partial, g.parts, m, w[0].n, y[0],
                                                                            y_strides[0], (uint32_t)y_dtype, logits_f32);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

}  // namespace mi355q
