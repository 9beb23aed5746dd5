// Small-batch projection on the matrix cores straight from the split planes (4-bit codes in groups of 64 or 128,
// 8-bit codes in groups of 32, 64 or 128), 2 <= M <= 16 activation rows per launch: the layout that serves M = 1 best also
// serves a batch.
//
// Stands in for gemv_q4_g{64,128} / gemv_q8_g{32,64} widened to the sequence signature and, at small sequence lengths,
// for gemm_q4_g64 / gemm_q8_g32 (Sources/MetalCompiler/Generator/MetalSourceGenerator+Quantized.swift:496-575 and :22-156):
//   y[m, n] = sum_g sum_{k in g} (s[n,g] * q[n,k] + z[n,g]) * x[m,k],  fp32 accumulation.
//
// A wavefront owns 16 consecutive weight rows and a share of K, walked in blocks of 128 codes.  One load instruction
// takes 64 contiguous bytes of each of its 16 rows (four consecutive lanes per row); a cross-lane read per word then
// gives lane (n = lane % 16, kq = lane / 16) the 32 codes at offset 32 kq of the block of row n, the order the matrix
// core wants.  Four v_mfma_f32_16x16x32_bf16 consume such a load, one per 32-bit word: a
// word's nibbles become the bf16 pairs (c0,c4) (c1,c5) (c2,c6) (c3,c7), each 128 + q, with one and-or per pair; the
// activations are staged once per workgroup in LDS with every run of eight in that same order
// (x0,x4,x1,x5,x2,x6,x3,x7), so they are the A operand as they lie.
// The matrix core sums over all four kq, which for groups of 64 are two quantisation groups (kq 0,1 and kq 2,3).  They
// are kept apart in the M dimension, which a batch of at most eight rows leaves half empty: A rows 0..7 carry the
// activations only where kq < 2 (zeros elsewhere), rows 8..15 only where kq >= 2.  D rows 0..7 are then the first
// group's sums, rows 8..15 the second's, and the accumulator of lane (n, kq), which holds D rows 4 kq .. 4 kq + 3, holds
// sums of the very group whose codes and (scale, bias) word it loaded: the affine form
//   acc += s * D + (z - 128 s) * SX        (D = sum (128 + q) x,  SX = sum x, computed while staging)
// is applied lane by lane, once per block, and lanes kq and kq + 2 add their halves at the end.  The KSPLIT wavefronts
// that share a row tile add their partial tiles through LDS.  (With groups of 128 both halves belong to one group and
// the same code runs unchanged.)
//
// 8-bit codes: a block is the same 64 bytes of a row, now 64 codes, and a lane's 16 bytes are 16 codes.  A code is
// split into its nibbles, q = 16 h + l: the masks that pair up a 4-bit word's nibbles give, on an 8-bit word, the pairs
// (l0,l2) (h0,h2) (l1,l3) (h1,h3), so two words make the B operand of one product over the low nibbles and one over the
// high nibbles of eight codes, against the same A operand (activations staged as (x0,x2,x1,x3,x4,x6,x5,x7)):
//   sum q x = D_l + 16 D_h - (128 + 16 * 128) SX.
// Instructions per byte of weights are those of the 4-bit form; groups of 32 take the place of groups of 64.
#include "device_utils.h"

namespace mi355q {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 pm_bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float pm_floatx4_t;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 pm_bf16x2_t;

__device__ __forceinline__ float pm_dot2(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(pm_bf16x2_t, a), __builtin_bit_cast(pm_bf16x2_t, b), acc, false);
}

constexpr int kPmMaxSegments = 3;

struct PmArgs {
    const uint32_t* rows[kPmMaxSegments];      // code words of row 0 of up to three matrices sharing x
    void* y[kPmMaxSegments];
    uint32_t tile_end[kPmMaxSegments];         // cumulative 16-row tile counts; unused entries repeat the last
    uint32_t seg_rows[kPmMaxSegments];         // N_i
    uint32_t y_stride[kPmMaxSegments];
    const uint16_t* x;                         // bf16 or f16 [M, x_stride]
    uint32_t x_f16;                            // 1: f16 rows, staged as two bf16 rows each (upper eight bits, the rest)
    uint32_t ms;                               // staged rows (2 M for f16): the M dimension the matrix core works on
    uint32_t k, m, x_stride;
    uint32_t row_words;                        // 32-bit words from one row to the next (codes, then the row's sz words)
    uint32_t sz_offset;                        // words from a row's first code word to its first (scale, bias) word
    uint32_t blocks_per_wave;                  // blocks (64 bytes of a row) per wavefront (K split over the workgroup)
    uint32_t passes;                           // row tiles a wavefront walks, one after the other, on one staged copy of x
    uint32_t lds_row_bytes;                    // part_blocks * (activation bytes per block) + 16: staged row pitch
    uint32_t y_dtype, sb_dtype;
    uint32_t parts;                            // K parts, each with workgroups of its own that stage only their columns
    uint32_t part_blocks;                      // blocks per part
    float* partial;                            // K parts only: fp32 partial results [part][M][N] (one matrix)
#ifdef MI355Q_GEMV_TIMELINE
    unsigned long long* timeline;              // measurement build only: 100 MHz time stamps per workgroup
#endif
};

#ifdef MI355Q_GEMV_TIMELINE
extern unsigned long long* g_gemv_timeline;
#endif

// BITS, GROUP: 4 with 64 or 128, 8 with 32, 64 or 128 (a group of two blocks: both blocks apply the group's word).  A workgroup of KSPLIT * TPW wavefronts covers TPW consecutive row tiles, each split over KSPLIT
// wavefronts along K; all of them share one staged copy of the activations.
// WIDE: nine to sixteen activation rows.  The M dimension then has no empty half, so the two groups of a block are
// kept apart with two products per word instead: one whose A operand carries the activations only where kq < 2, one
// only where kq >= 2 (groups of 128 need neither: one product with the whole A operand).  Every lane then holds rows
// 4 kq .. 4 kq + 3 of both groups' sums and applies both (scale, bias) words.
template <int BITS, int GROUP, int KSPLIT, int TPW, bool SBBF16, bool WIDE>
__global__ __launch_bounds__(KSPLIT * TPW * 64) void gemv_mfma_planes_kernel(PmArgs a) {
    constexpr uint32_t BC = 512 / BITS;                     // codes per block: 64 bytes of a row
    constexpr uint32_t XBYTES = BC * 2;                     // bytes of one activation row per block
    constexpr uint32_t HALF = BC / 2;                       // codes of half a block: the run the staged sums cover
    constexpr bool TWO = GROUP * 2 == (int)BC;              // a block holds two quantisation groups (else one)
    constexpr bool PAIR = GROUP == 2 * (int)BC;             // a quantisation group spans two blocks (8 bits, groups of 128)
    static_assert((BITS == 4 || BITS == 8) && (TWO || PAIR || GROUP == (int)BC), "4 bits: groups of 64 / 128; 8 bits: 32 / 64 / 128");
    constexpr uint32_t SXR = WIDE ? 16 : 8;                 // activation rows per run of 64 in the staged sums
    constexpr int WAVES = KSPLIT * TPW;
    constexpr int D = 4;                                    // blocks in flight per wavefront
    constexpr int MR = 4;
    extern __shared__ u32x4 smem_pm[];
    char* lds = (char*)smem_pm;
#ifdef MI355Q_GEMV_TIMELINE
    const unsigned long long tl_entry = __builtin_amdgcn_s_memrealtime();
    unsigned long long tl_staged = 0, tl_first = 0, tl_loop = 0;
#endif
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t n_in = lane & 15, kq = lane >> 4;
    const uint32_t part = blockIdx.y, wg = blockIdx.x;
    const uint32_t b0 = part * a.part_blocks;               // first block of this workgroup's K part
    const uint32_t kp = a.part_blocks * BC;                 // activation elements staged per row

    const uint32_t slice = wave % KSPLIT;
    struct Tile {
        const uint32_t* lane_row;  // this lane's row: first code word
        void* y;
        uint32_t ys, rows, n0, nb, b_first, b_last;
        bool valid;
    };
    auto select_tile = [&](uint32_t pass) {
        Tile t;
        const uint32_t last = a.tile_end[kPmMaxSegments - 1];
        uint32_t gt = (wg * a.passes + pass) * TPW + wave / KSPLIT;
        t.valid = gt < last;
        gt = t.valid ? gt : last - 1;                                     // idle wavefronts re-read the last tile
        const bool in1 = gt >= a.tile_end[0], in2 = gt >= a.tile_end[1];
        const uint32_t* const seg = in2 ? a.rows[2] : in1 ? a.rows[1] : a.rows[0];
        t.y = in2 ? a.y[2] : in1 ? a.y[1] : a.y[0];
        t.ys = in2 ? a.y_stride[2] : in1 ? a.y_stride[1] : a.y_stride[0];
        t.rows = in2 ? a.seg_rows[2] : in1 ? a.seg_rows[1] : a.seg_rows[0];
        const uint32_t lt = gt - (in2 ? a.tile_end[1] : in1 ? a.tile_end[0] : 0u);
        t.n0 = lt * 16;
        uint32_t row = t.n0 + (lane >> 2);                                // the row this lane LOADS (see `issue`)
        row = row < t.rows ? row : t.rows - 1;                            // rows past the end re-read the last one
        t.lane_row = seg + (size_t)row * a.row_words;
        const uint32_t b_end = b0 + a.part_blocks;
        t.b_first = b0 + slice * a.blocks_per_wave;
        uint32_t nb = b_end > t.b_first ? b_end - t.b_first : 0;
        nb = nb < a.blocks_per_wave ? nb : a.blocks_per_wave;
        t.nb = t.valid ? nb : 0;
        t.b_last = t.nb ? t.b_first + t.nb - 1 : b_end - 1;              // clamp target (always valid)
        return t;
    };
    Tile tile = select_tile(0);

    // ---- 1. activation loads first (vector loads return in issue order) -------------------------------------------
    // The M x chunks 16-byte chunks of the staged columns are dealt to the threads in order, XB a thread at a time: a
    // batch's loads all go out before its first chunk is staged, and the first batch goes out before the weight
    // loads.  Behind the staged rows lie 256 bytes of zeros (the masked half of A).
    const uint32_t chunks = kp / 8;                         // 16-byte chunks per staged activation row
    constexpr uint32_t NT = WAVES * 64;
    constexpr int XB = 8;
    const uint32_t total = a.m * chunks;
    const float inv_chunks = 1.0f / (float)chunks;
    auto x_at = [&](uint32_t idx, uint32_t& m, uint32_t& c) -> bool {     // false: past the end
        const bool has = idx < total;
        idx = has ? idx : 0;
        m = (uint32_t)(((float)idx + 0.5f) * inv_chunks);     // exact: idx < 2^20, chunks <= 2^13
        c = idx - m * chunks;
        return has;
    };
    auto x_load = [&](uint32_t idx) -> u32x4 {
        uint32_t m, c;
        x_at(idx, m, c);
        return *((const u32x4*)(a.x + (size_t)m * a.x_stride + (size_t)b0 * BC) + c);
    };
    u32x4 xe[XB];
#pragma unroll
    for (int t = 0; t < XB; t++)
        if ((uint32_t)t * NT < total) xe[t] = x_load(tid + (uint32_t)t * NT);     // wavefront-uniform: no load past the end
    __builtin_amdgcn_sched_barrier(0);

    // ---- 2. the first D blocks of this wavefront's share of the first row tile ---------------------------------------
    // Loads are issued with four consecutive lanes on one row (lane L: row L / 4, 16-byte piece L % 4), so that a
    // load instruction is sixteen coalesced 64-byte requests; the matrix core wants lane kq * 16 + n to hold piece kq
    // of row n, which `compute` arranges with one cross-lane read per 32-bit word.
    const uint32_t piece = lane & 3u;
    struct Rec { u32x4 w; };
    Rec ring[D];
    auto issue = [&](uint32_t b, Rec& r) {
        b = b < tile.b_last ? b : tile.b_last;              // unconditional, clamped
        r.w = __builtin_nontemporal_load((const u32x4*)(tile.lane_row + (size_t)b * 16 + piece * 4));
    };
    // (scale, bias) words, sixteen blocks of the wavefront's share at a time: this lane keeps those of blocks
    // first + piece * 4 .. + 3 of the row it loads (one word per group: two per block where a block holds two groups)
    constexpr int SZW = TWO ? 2 : 1;
    uint32_t szr[4][SZW];
    auto issue_sz = [&](uint32_t first) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t b = first + piece * 4 + i;
            b = b < tile.b_last ? b : tile.b_last;
            const uint32_t* q = tile.lane_row + a.sz_offset + (size_t)(PAIR ? b >> 1 : b) * SZW;
            if constexpr (SZW == 2) { const u32x2 t = *(const u32x2*)q; szr[i][0] = t.x; szr[i][1] = t.y; }
            else szr[i][0] = *q;
        }
    };
    static_for<D>([&](auto J) { issue(tile.b_first + decltype(J)::value, ring[decltype(J)::value]); });
    issue_sz(tile.b_first);

    // ---- 3. stage the activations: every run of eight as (x0,x4,x1,x5,x2,x6,x3,x7) (8 bits: (x0,x2,x1,x3,x4,x6,x5,x7)),
    //         and sum(x) per half block and row ----------------------------------------------------------------------
    constexpr uint32_t CH = HALF / 8;                       // 16-byte chunks per half block
    // behind the staged rows: 256 bytes of zeros (the masked half of A reads them at every block), then the sums
    char* const zero_block = lds + (size_t)a.ms * a.lds_row_bytes;
    float* const sxs = (float*)(zero_block + 256);                            // [half block in part][SXR]
    {
        auto run_sum = [&](const u32x4& v) {
            float p = pm_dot2(v.x, 0x3F803F80u, 0.0f);
            p = pm_dot2(v.y, 0x3F803F80u, p);
            p = pm_dot2(v.z, 0x3F803F80u, p);
            p = pm_dot2(v.w, 0x3F803F80u, p);
            // over the CH consecutive lanes of a half block, inside the vector unit (lane pairs, quads, then the mirror
            // image inside eight lanes: every lane of a quad holds the quad's sum by then)
            p += dpp_f32<0xB1>(p);                           // quad_perm [1,0,3,2]
            p += dpp_f32<0x4E>(p);                           // quad_perm [2,3,0,1]
            if constexpr (CH == 8) p += dpp_f32<0x141>(p);   // row_half_mirror
            return p;
        };
        // one chunk of a staged row: every run of eight in the operand order of the unpacked codes, and its share of sum(x)
        auto stage_row = [&](uint32_t m, uint32_t c, bool has, const u32x4& v) {
            const float p = run_sum(v);
            if (has) {
                u32x4 o;
                if constexpr (BITS == 4) {
                    o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);    // (x0, x4)
                    o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);    // (x1, x5)
                    o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);    // (x2, x6)
                    o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);    // (x3, x7)
                } else {
                    o.x = __builtin_amdgcn_perm(v.y, v.x, 0x05040100u);    // (x0, x2)
                    o.y = __builtin_amdgcn_perm(v.y, v.x, 0x07060302u);    // (x1, x3)
                    o.z = __builtin_amdgcn_perm(v.w, v.z, 0x05040100u);    // (x4, x6)
                    o.w = __builtin_amdgcn_perm(v.w, v.z, 0x07060302u);    // (x5, x7)
                }
                *((u32x4*)(lds + (size_t)m * a.lds_row_bytes) + c) = o;
                if ((c & (CH - 1)) == 0) sxs[(c / CH) * SXR + m] = p;  // CH chunks: one half block
            }
        };
        auto stage = [&](uint32_t idx, const u32x4& v) {
            uint32_t m, c;
            const bool has = x_at(idx, m, c);
            if (a.x_f16) {                                  // wavefront-uniform: an f16 row becomes staged rows 2 m, 2 m + 1
                u32x4 hi, lo;
                f16x8_to_bf16_hi_lo(v, hi, lo);
                stage_row(2 * m, c, has, hi);
                stage_row(2 * m + 1, c, has, lo);
            } else {
                stage_row(m, c, has, v);
            }
        };
        // whole wavefronts take part in the shuffles of every step: the walk is rounded up to whole batches
#pragma unroll
        for (int t = 0; t < XB; t++)
            if ((uint32_t)t * NT < total) stage(tid + (uint32_t)t * NT, xe[t]);
        for (uint32_t base = XB * NT; base < total; base += XB * NT) {
#pragma unroll
            for (int t = 0; t < XB; t++)
                if (base + (uint32_t)t * NT < total) xe[t] = x_load(base + tid + (uint32_t)t * NT);
#pragma unroll
            for (int t = 0; t < XB; t++)
                if (base + (uint32_t)t * NT < total) stage(base + tid + (uint32_t)t * NT, xe[t]);
        }
        const u32x4 zero = {0u, 0u, 0u, 0u};
        if (tid < 16) *((u32x4*)zero_block + tid) = zero;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
#ifdef MI355Q_GEMV_TIMELINE
    tl_staged = __builtin_amdgcn_s_memrealtime();
    {   // when the first weight words of this wavefront are there
        uint32_t first_word = ring[0].w.x;
        asm volatile("s_waitcnt vmcnt(0)" : "+v"(first_word));
        ring[0].w.x = first_word;
        tl_first = __builtin_amdgcn_s_memrealtime();
    }
#endif

    // ---- 4. K loop --------------------------------------------------------------------------------------------------
    uint32_t k_mask = 0x000F000Fu, k_magic = 0x43004300u;   // opaque: keeps (w & mask) | magic one v_and_or_b32
    asm volatile("" : "+s"(k_mask));
    asm volatile("" : "+v"(k_magic));
    const pm_floatx4_t zero4 = {0.f, 0.f, 0.f, 0.f};
    float acc[MR];
#pragma unroll
    for (int r = 0; r < MR; r++) acc[r] = 0.f;

    // A operand: lane (i = lane % 16, kq) stands for A row i.  Rows 0..7 are activation rows 0..7 where kq < 2, rows
    // 8..15 are the same activation rows where kq >= 2; elsewhere zeros, read from the same 64 bytes at every block (the
    // lane's offset from block to block is masked away).  Rows past M read row M-1 (their results are never stored).
    const uint32_t xi = WIDE ? n_in : (n_in & 7u);
    const uint32_t xr = xi < a.ms ? xi : a.ms - 1;
    const bool live = WIDE ? (kq < 2) : (n_in >> 3) == (kq >> 1);
    const bool reads_x = live || (WIDE && !TWO);
    const char* const a_lane = (reads_x ? lds + (size_t)xr * a.lds_row_bytes : zero_block) + kq * (XBYTES / 4);
    const uint32_t a_mask = reads_x ? ~0u : 0u;            // (an and per block: a per-lane multiply is a slow instruction)
    // WIDE, two groups per block: the second product's operand, live where the first one's is not
    const char* const a_lane_hi = (live ? zero_block : lds + (size_t)xr * a.lds_row_bytes) + kq * (XBYTES / 4);
    const uint32_t a_mask_hi = live ? 0u : ~0u;

    auto unpack = [&](uint32_t w) -> pm_bf16x8_t {
        u32x4 p;
        p.x = (w & k_mask) | k_magic;
        p.y = ((w >> 4) & k_mask) | k_magic;
        p.z = ((w >> 8) & k_mask) | k_magic;
        p.w = ((w >> 12) & k_mask) | k_magic;
        return __builtin_bit_cast(pm_bf16x8_t, p);
    };
    // 8 bits: the low (SH = 0) or high (SH = 4) nibbles of the eight codes of two words, in the order c0,c2,c1,c3 of each
    auto unpack8 = [&](uint32_t wa, uint32_t wb, auto SH) -> pm_bf16x8_t {
        constexpr int sh = decltype(SH)::value;
        u32x4 p;
        p.x = ((wa >> sh) & k_mask) | k_magic;
        p.y = ((wa >> (8 + sh)) & k_mask) | k_magic;
        p.z = ((wb >> sh) & k_mask) | k_magic;
        p.w = ((wb >> (8 + sh)) & k_mask) | k_magic;
        return __builtin_bit_cast(pm_bf16x8_t, p);
    };
    using Lo = std::integral_constant<int, 0>;
    using Hi = std::integral_constant<int, 4>;
    // sum (128 + q) x for 4 bits; for 8 bits sum (128 + l) x + 16 sum (128 + h) x: the offset the affine form takes back
    constexpr float kOffset = BITS == 4 ? 128.0f : 128.0f * 17.0f;
    // this lane's D rows 4 kq .. 4 kq + 3 are activation rows 4 (kq & 1) .. + 3
    const uint32_t sx_lane = WIDE ? 4 * kq : (kq >> 1) * 8 + 4 * (kq & 1);
    const int from_lane = (int)((4u * n_in + kq) * 4u);     // byte address of the lane that loaded (row n, piece kq)
    auto compute = [&](uint32_t b, const Rec& r, const uint32_t (&sz_pair)[SZW], uint32_t sz_piece) {
        const uint32_t bl = b - b0;                          // block inside the staged columns
        const char* ab = a_lane + ((bl * XBYTES) & a_mask);  // this block's activations
        // every LDS operation of the block goes out first: the cross-lane reads, the A operands, sum(x) over this lane
        // half's run of 64 (runs 2 bl and 2 bl + 1 of the part): a group of 64, or half of a group of 128 whose other
        // half the other lanes add
        const uint32_t w0 = (uint32_t)__builtin_amdgcn_ds_bpermute(from_lane, (int)r.w.x);
        const uint32_t w1 = (uint32_t)__builtin_amdgcn_ds_bpermute(from_lane, (int)r.w.y);
        const uint32_t w2 = (uint32_t)__builtin_amdgcn_ds_bpermute(from_lane, (int)r.w.z);
        const uint32_t w3 = (uint32_t)__builtin_amdgcn_ds_bpermute(from_lane, (int)r.w.w);
        // the block's (scale, bias) words sit with the lane that loaded piece `sz_piece` of this row
        const int sz_from = (int)((4u * n_in + sz_piece) * 4u);
        uint32_t szw = (uint32_t)__builtin_amdgcn_ds_bpermute(sz_from, (int)sz_pair[0]);
        uint32_t szw_hi = szw;
        if constexpr (SZW == 2) {
            szw_hi = (uint32_t)__builtin_amdgcn_ds_bpermute(sz_from, (int)sz_pair[1]);
            if constexpr (!WIDE) szw = kq >> 1 ? szw_hi : szw;
        }
        const pm_bf16x8_t a0 = *(const pm_bf16x8_t*)(ab), a1 = *(const pm_bf16x8_t*)(ab + 16);
        pm_bf16x8_t a2 = a0, a3 = a1;                       // (8 bits: a lane's share of a block is two operands)
        if constexpr (BITS == 4) { a2 = *(const pm_bf16x8_t*)(ab + 32); a3 = *(const pm_bf16x8_t*)(ab + 48); }
        const pm_floatx4_t sx = *(const pm_floatx4_t*)(sxs + (size_t)bl * 2 * SXR + sx_lane);
        auto scale_zero = [&](uint32_t word, float& sc, float& zc) {
            float zr;
            if constexpr (SBBF16) { sc = __uint_as_float(word << 16); zr = __uint_as_float(word & 0xFFFF0000u); }
            else { sc = f16_to_f32((uint16_t)(word & 0xFFFFu)); zr = f16_to_f32((uint16_t)(word >> 16)); }
            zc = zr - kOffset * sc;
        };
        if constexpr (BITS == 8) {
            // products over the low and the high nibbles share the A operands; WIDE with two groups per block: each
            // against both masked operands
            const pm_bf16x8_t l0 = unpack8(w0, w1, Lo{}), l1 = unpack8(w2, w3, Lo{});
            const pm_bf16x8_t h0 = unpack8(w0, w1, Hi{}), h1 = unpack8(w2, w3, Hi{});
            if constexpr (!(WIDE && TWO)) {
                pm_floatx4_t sxv = sx;
                if constexpr (WIDE) {
                    const pm_floatx4_t sx_hi = *(const pm_floatx4_t*)(sxs + (size_t)(bl * 2 + 1) * SXR + sx_lane);
                    sxv += sx_hi;
                }
                __builtin_amdgcn_sched_barrier(0);
                pm_floatx4_t dl = zero4, dh = zero4;
                dl = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, l0, dl, 0, 0, 0);
                dh = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, h0, dh, 0, 0, 0);
                dl = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, l1, dl, 0, 0, 0);
                dh = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, h1, dh, 0, 0, 0);
                float sc, zc;
                scale_zero(szw, sc, zc);
#pragma unroll
                for (int q = 0; q < MR; q++) acc[q] += sc * __builtin_fmaf(16.0f, dh[q], dl[q]) + zc * sxv[q];
            } else {
                const pm_floatx4_t sx_hi = *(const pm_floatx4_t*)(sxs + (size_t)(bl * 2 + 1) * SXR + sx_lane);
                const char* ah = a_lane_hi + ((bl * XBYTES) & a_mask_hi);
                const pm_bf16x8_t g0 = *(const pm_bf16x8_t*)(ah), g1 = *(const pm_bf16x8_t*)(ah + 16);
                __builtin_amdgcn_sched_barrier(0);
                pm_floatx4_t dl = zero4, dh = zero4, el = zero4, eh = zero4;
                dl = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, l0, dl, 0, 0, 0);
                dh = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, h0, dh, 0, 0, 0);
                el = __builtin_amdgcn_mfma_f32_16x16x32_bf16(g0, l0, el, 0, 0, 0);
                eh = __builtin_amdgcn_mfma_f32_16x16x32_bf16(g0, h0, eh, 0, 0, 0);
                dl = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, l1, dl, 0, 0, 0);
                dh = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, h1, dh, 0, 0, 0);
                el = __builtin_amdgcn_mfma_f32_16x16x32_bf16(g1, l1, el, 0, 0, 0);
                eh = __builtin_amdgcn_mfma_f32_16x16x32_bf16(g1, h1, eh, 0, 0, 0);
                float s0, z0, s1, z1;
                scale_zero(szw, s0, z0);
                scale_zero(szw_hi, s1, z1);
#pragma unroll
                for (int q = 0; q < MR; q++)
                    acc[q] += (s0 * __builtin_fmaf(16.0f, dh[q], dl[q]) + z0 * sx[q]) +
                              (s1 * __builtin_fmaf(16.0f, eh[q], el[q]) + z1 * sx_hi[q]);
            }
        } else if constexpr (!WIDE) {
            __builtin_amdgcn_sched_barrier(0);
            pm_floatx4_t d = zero4;
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, unpack(w0), d, 0, 0, 0);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, unpack(w1), d, 0, 0, 0);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2, unpack(w2), d, 0, 0, 0);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a3, unpack(w3), d, 0, 0, 0);
            float sc, zc;
            scale_zero(szw, sc, zc);
#pragma unroll
            for (int q = 0; q < MR; q++) acc[q] += sc * d[q] + zc * sx[q];
        } else {
            const pm_floatx4_t sx_hi = *(const pm_floatx4_t*)(sxs + (size_t)(bl * 2 + 1) * SXR + sx_lane);
            const pm_bf16x8_t b0 = unpack(w0), b1 = unpack(w1), b2 = unpack(w2), b3 = unpack(w3);
            if constexpr (!TWO) {
                __builtin_amdgcn_sched_barrier(0);
                pm_floatx4_t d = zero4;
                d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b0, d, 0, 0, 0);
                d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b1, d, 0, 0, 0);
                d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2, b2, d, 0, 0, 0);
                d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a3, b3, d, 0, 0, 0);
                float sc, zc;
                scale_zero(szw, sc, zc);
#pragma unroll
                for (int q = 0; q < MR; q++) acc[q] += sc * d[q] + zc * (sx[q] + sx_hi[q]);
            } else {
                const char* ah = a_lane_hi + ((bl * XBYTES) & a_mask_hi);
                const pm_bf16x8_t h0 = *(const pm_bf16x8_t*)(ah), h1 = *(const pm_bf16x8_t*)(ah + 16);
                const pm_bf16x8_t h2 = *(const pm_bf16x8_t*)(ah + 32), h3 = *(const pm_bf16x8_t*)(ah + 48);
                __builtin_amdgcn_sched_barrier(0);
                pm_floatx4_t d = zero4, e = zero4;
                d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b0, d, 0, 0, 0);
                e = __builtin_amdgcn_mfma_f32_16x16x32_bf16(h0, b0, e, 0, 0, 0);
                d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b1, d, 0, 0, 0);
                e = __builtin_amdgcn_mfma_f32_16x16x32_bf16(h1, b1, e, 0, 0, 0);
                d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2, b2, d, 0, 0, 0);
                e = __builtin_amdgcn_mfma_f32_16x16x32_bf16(h2, b2, e, 0, 0, 0);
                d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a3, b3, d, 0, 0, 0);
                e = __builtin_amdgcn_mfma_f32_16x16x32_bf16(h3, b3, e, 0, 0, 0);
                float s0, z0, s1, z1;
                scale_zero(szw, s0, z0);
                scale_zero(szw_hi, s1, z1);
#pragma unroll
                for (int q = 0; q < MR; q++) acc[q] += (s0 * d[q] + z0 * sx[q]) + (s1 * e[q] + z1 * sx_hi[q]);
            }
        }
    };

    const uint32_t rounds = (a.blocks_per_wave + D - 1) / D;              // same for every wavefront
    // Partial tiles of the WAVES wavefronts, [WAVES][MR][64]: a single pass writes them over the staged activations
    // once every wavefront is done reading those; several passes keep them behind the activations and their sums.
    const bool red_over_x = a.passes == 1;
    float* const red = (float*)(red_over_x ? lds : (char*)sxs + (size_t)(kp / HALF) * SXR * 4);
    for (uint32_t pass = 0; pass < a.passes; pass++) {
        if (pass) {                                            // the first tile's loads were issued before staging
            tile = select_tile(pass);
            static_for<D>([&](auto J) { issue(tile.b_first + decltype(J)::value, ring[decltype(J)::value]); });
            issue_sz(tile.b_first);
        }
        for (uint32_t it = 0; it < rounds; it++) {
            if (it && (it & 3u) == 0) issue_sz(tile.b_first + it * D);       // the next sixteen blocks' words
            static_for<D>([&](auto J) {
                constexpr int j = decltype(J)::value;
                const uint32_t idx = it * D + j;
                if (idx < tile.nb) compute(tile.b_first + idx, ring[j], szr[j], it & 3u);
                issue(tile.b_first + idx + D, ring[j]);
            });
        }

#ifdef MI355Q_GEMV_TIMELINE
        if (pass + 1 == a.passes) tl_loop = __builtin_amdgcn_s_memrealtime();
#endif
        // ---- 5. add the partial tiles of the wavefronts that share a row tile, store ---------------------------------
        if (red_over_x) __syncthreads();
#pragma unroll
        for (int r = 0; r < MR; r++) { red[(wave * MR + r) * 64 + lane] = acc[r]; acc[r] = 0.f; }
        __syncthreads();
        if (slice == 0 && tile.valid && (WIDE || kq < 2)) { // the first wavefront of each tile adds and stores
            const uint32_t row = tile.n0 + n_in;
            float vv[MR];
#pragma unroll
            for (int r = 0; r < MR; r++) {
                vv[r] = 0.f;
                for (uint32_t w2 = 0; w2 < (uint32_t)KSPLIT; w2++) {     // (not WIDE: both halves of K of every block)
                    vv[r] += red[((wave + w2) * MR + r) * 64 + lane];
                    if constexpr (!WIDE) vv[r] += red[((wave + w2) * MR + r) * 64 + lane + 32];
                }
            }
            // f16 rows: staged rows 2 m and 2 m + 1, both in this lane, are the two parts of activation row m
            const bool fold = a.x_f16;
#pragma unroll
            for (int r = 0; r < MR; r++) {
                if (fold && r >= MR / 2) break;
                const float v = fold ? vv[(2 * r + 1) % MR] + vv[(2 * r) % MR] : vv[r];
                const uint32_t m = fold ? 2 * kq + r : 4 * kq + r;
                if (m < a.m && row < tile.rows) {
                    if (a.parts > 1) {                       // one matrix: the reduction launch converts and stores
                        a.partial[((size_t)part * a.m + m) * tile.rows + row] = v;
                        continue;
                    }
                    const size_t o = (size_t)m * tile.ys + row;
                    if (a.y_dtype == MI355Q_F32) ((float*)tile.y)[o] = v;
                    else if (a.y_dtype == MI355Q_BF16) ((uint16_t*)tile.y)[o] = f32_to_bf16_rne(v);
                    else ((uint16_t*)tile.y)[o] = f32_to_f16_rne(v);
                }
            }
        }
        if (pass + 1 < a.passes) __syncthreads();           // the partial tiles are read before the next pass overwrites them
    }
#ifdef MI355Q_GEMV_TIMELINE
    if (a.timeline && wave == 0 && lane == 0) {
        unsigned long long* const t = a.timeline + ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 6;
        uint32_t hw_id;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw_id));
        t[0] = tl_entry; t[1] = tl_staged; t[2] = tl_first; t[3] = __builtin_amdgcn_s_memrealtime();
        t[4] = hw_id; t[5] = tl_loop;
    }
#endif
}

// Sum of the K parts, in part order, then the conversion the single-launch form does in its epilogue.
__global__ __launch_bounds__(256) void pm_sum_parts_kernel(const float* __restrict__ partial, uint32_t parts, uint32_t m,
                                                           uint32_t n, void* __restrict__ y, uint32_t y_stride,
                                                           uint32_t y_dtype) {
    const uint32_t row = blockIdx.y;
    for (uint32_t col = blockIdx.x * 256 + threadIdx.x; col < n; col += gridDim.x * 256) {
        float v = 0.f;
        for (uint32_t p = 0; p < parts; p++) v += partial[((size_t)p * m + row) * n + col];
        const size_t o = (size_t)row * y_stride + col;
        if (y_dtype == MI355Q_F32) ((float*)y)[o] = v;
        else if (y_dtype == MI355Q_BF16) ((uint16_t*)y)[o] = f32_to_bf16_rne(v);
        else ((uint16_t*)y)[o] = f32_to_f16_rne(v);
    }
}

namespace {

template <int BITS, int GROUP, int KSPLIT, int TPW>
mi355q_status launch_pm(hipStream_t s, const PmArgs& a, uint32_t grid, size_t lds) {
    auto kern = a.ms > 8 ? (a.sb_dtype == MI355Q_BF16 ? gemv_mfma_planes_kernel<BITS, GROUP, KSPLIT, TPW, true, true>
                                                     : gemv_mfma_planes_kernel<BITS, GROUP, KSPLIT, TPW, false, true>)
                        : (a.sb_dtype == MI355Q_BF16 ? gemv_mfma_planes_kernel<BITS, GROUP, KSPLIT, TPW, true, false>
                                                     : gemv_mfma_planes_kernel<BITS, GROUP, KSPLIT, TPW, false, false>);
    if (lds > 64 * 1024)
        if (mi355q_status st = raise_lds_limit((const void*)kern, lds)) return st;
    kern<<<dim3(grid, a.parts), dim3(KSPLIT * TPW * 64), lds, s>>>(a);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

template <int BITS, int GROUP>
mi355q_status launch_pm_shape(hipStream_t s, const PmArgs& a, const Tile16LaunchShape& g) {
    const uint32_t ks = g.ksplit, tpw = g.tiles_per_wg;
    if (ks == 4 && tpw == 1) return launch_pm<BITS, GROUP, 4, 1>(s, a, g.wgs_per_part, g.lds_bytes);
    if (ks == 4 && tpw == 2) return launch_pm<BITS, GROUP, 4, 2>(s, a, g.wgs_per_part, g.lds_bytes);
    if (ks == 4 && tpw == 3) return launch_pm<BITS, GROUP, 4, 3>(s, a, g.wgs_per_part, g.lds_bytes);
    if (ks == 4 && tpw == 4) return launch_pm<BITS, GROUP, 4, 4>(s, a, g.wgs_per_part, g.lds_bytes);
    if (ks == 2 && tpw == 5) return launch_pm<BITS, GROUP, 2, 5>(s, a, g.wgs_per_part, g.lds_bytes);
    if (ks == 2 && tpw == 6) return launch_pm<BITS, GROUP, 2, 6>(s, a, g.wgs_per_part, g.lds_bytes);
    if (ks == 2 && tpw == 7) return launch_pm<BITS, GROUP, 2, 7>(s, a, g.wgs_per_part, g.lds_bytes);
    if (ks == 2 && tpw == 8) return launch_pm<BITS, GROUP, 2, 8>(s, a, g.wgs_per_part, g.lds_bytes);
    if (ks == 8 && tpw == 1) return launch_pm<BITS, GROUP, 8, 1>(s, a, g.wgs_per_part, g.lds_bytes);
    if (ks == 8 && tpw == 2) return launch_pm<BITS, GROUP, 8, 2>(s, a, g.wgs_per_part, g.lds_bytes);
    if (ks == 16 && tpw == 1) return launch_pm<BITS, GROUP, 16, 1>(s, a, g.wgs_per_part, g.lds_bytes);
    return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "no matrix-core planes variant for K-split %u x %u tiles per workgroup", ks, tpw);
}

}  // namespace

// The workgroups are shaped like those of the TILE16 kernel (16-row tiles walked in blocks of 128 codes, the same split
// of K over wavefronts, tiles per workgroup, passes and K parts), plus 256 bytes of zeros behind the staged rows.  That
// kernel's LDS sizes bound this one's (M rows and K / 2 bytes of sums against M rows and K bytes).
bool gemv_mfma_planes_eligible(const WView& w, int x_dtype, uint32_t m, uint32_t x_stride) {
    if (w.layout != MI355Q_LAYOUT_PLANES || !w.sz || (x_dtype != MI355Q_BF16 && x_dtype != MI355Q_F16)) return false;
    const uint32_t ms = staged_rows(x_dtype, m);                           // f16 rows are staged as two bf16 rows each
    if (ms < 2 || ms > 16) return false;
    if (w.bits != 4 && w.bits != 8) return false;
    const uint32_t bc = 512 / w.bits;                                     // codes per block
    if ((w.group != bc && w.group * 2 != bc && !(w.bits == 8 && w.group == 2 * bc)) || w.k % w.group || w.k % bc) return false;
    if (x_stride % 8) return false;                                       // 128-bit activation loads
    // a row is one stream: its sz words follow its code words at the same pitch; code words 16-byte aligned
    if (w.sz_stride != w.code_stride || w.code_stride % 4 || (uintptr_t)w.codes % 16) return false;
    if (w.sz < w.codes || (size_t)(w.sz - w.codes) >= w.code_stride || (w.sz - w.codes) % 2) return false;
    return gemv_tile16_parts_for(w.k, ms, (w.n + 15) / 16, 256, bc) != 0;
}

uint32_t gemv_mfma_planes_k_parts(const mi355q_context* ctx, const WView& w, uint32_t m) {
    return gemv_tile16_parts_for(w.k, m, (w.n + 15) / 16, (uint32_t)ctx->props.multiProcessorCount, 512 / w.bits);
}

Tile16LaunchShape gemv_mfma_planes_shape(const mi355q_context* ctx, uint32_t n_row_tiles, uint32_t k_total, uint32_t bits,
                                         uint32_t m) {
    Tile16LaunchShape g = gemv_tile16_shape(ctx, n_row_tiles, k_total, m, 512 / bits);
    g.lds_bytes += 256;                                                    // the block of zeros behind the staged rows
    return g;
}

mi355q_status launch_gemv_mfma_planes_multi(hipStream_t s, mi355q_context* ctx, uint32_t count, const WView* w,
                                            const void* x, int x_dtype, void* const* y, const uint32_t* y_strides, int y_dtype,
                                            uint32_t m, uint32_t x_stride) {
    if (count < 1 || count > (uint32_t)kPmMaxSegments)
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "1..%d weights per fused launch", kPmMaxSegments);
    if ((uintptr_t)x % 16) return fail(MI355Q_ERR_INVALID_ARGUMENT, "activation pointer must be 16-byte aligned");
    PmArgs a{};
    uint32_t tiles = 0;
    for (uint32_t i = 0; i < (uint32_t)kPmMaxSegments; i++) {
        const uint32_t j = i < count ? i : count - 1;
        if (i < count) tiles += (w[i].n + 15) / 16;
        a.rows[i] = w[j].codes;
        a.y[i] = y[j];
        a.y_stride[i] = y_strides[j];
        a.seg_rows[i] = w[j].n;
        a.tile_end[i] = tiles;
        if (w[j].code_stride != w[0].code_stride || (w[j].sz - w[j].codes) != (w[0].sz - w[0].codes) ||
            w[j].k != w[0].k || w[j].bits != w[0].bits || w[j].group != w[0].group || w[j].sb_dtype != w[0].sb_dtype)
            return fail(MI355Q_ERR_SHAPE, "fused projections must share K, format, row pitch and scale type");
    }
    const uint32_t ms = staged_rows(x_dtype, m);
    const Tile16LaunchShape g = gemv_mfma_planes_shape(ctx, tiles, w[0].k, w[0].bits, ms);
    const uint32_t bc = 512 / w[0].bits;
    a.x = (const uint16_t*)x;
    a.k = w[0].k; a.m = m; a.x_stride = x_stride;
    a.x_f16 = x_dtype == MI355Q_F16 ? 1u : 0u;
    a.ms = ms;
    a.row_words = w[0].code_stride;
    a.sz_offset = (uint32_t)(w[0].sz - w[0].codes);
    a.parts = g.parts;
    a.part_blocks = w[0].k / bc / g.parts;
    a.blocks_per_wave = g.blocks_per_wave;
    a.passes = g.passes;
    a.lds_row_bytes = a.part_blocks * bc * 2 + 16;
    if (g.parts > 1) {
        if (count != 1)
            return fail(MI355Q_ERR_KERNEL_NOT_FOUND, "rows of %u codes at M = %u are split over K parts: one matrix per launch",
                        w[0].k, m);
        if (mi355q_status st = ensure_workspace(ctx, (size_t)g.parts * m * w[0].n * sizeof(float))) return st;
        a.partial = (float*)ctx->workspace;
    }
    a.y_dtype = (uint32_t)y_dtype; a.sb_dtype = w[0].sb_dtype;
#ifdef MI355Q_GEMV_TIMELINE
    a.timeline = g_gemv_timeline;
#endif
    const mi355q_status st = w[0].bits == 4 ? (w[0].group == 64 ? launch_pm_shape<4, 64>(s, a, g) : launch_pm_shape<4, 128>(s, a, g))
                                            : (w[0].group == 32 ? launch_pm_shape<8, 32>(s, a, g)
                                               : w[0].group == 64 ? launch_pm_shape<8, 64>(s, a, g) : launch_pm_shape<8, 128>(s, a, g));
    if (st != MI355Q_OK || g.parts == 1) return st;
    uint32_t sum_wgs = (w[0].n + 255) / 256;
    if (sum_wgs > 65535u) sum_wgs = 65535u;
    pm_sum_parts_kernel<<<dim3(sum_wgs, m), dim3(256), 0, s>>>(a.partial, g.parts, m, w[0].n, y[0], y_strides[0],
                                                                       (uint32_t)y_dtype);
    MI355Q_HIP(hipGetLastError());
    return MI355Q_OK;
}

}  // namespace mi355q
