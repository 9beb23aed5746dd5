/*
 * CPU oracle for the group-affine quantized-linear path -- TEST INFRASTRUCTURE ONLY.
 * See qlin_oracle.h for the role of this file and the parity-pinning status of each function.
 * Build with -ffp-contract=off: the reference's CPU loop (Swift) does not fuse multiply-add.
 */
#include "qlin_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ formats */

/* Registry rows: scheme ids from MC/STAF/STAFFormat.swift:175-217; the (bits, group) pairs
 * from MC/STAF/QuantizationFormat.swift:1315-1335.  0x22 (q6g64) and 0x62 (q2g64) are not in
 * the reference; they take the next free id of their family (ids are append-only). */
static const orc_format k_formats[] = {
    {0x60, 2, 16, 4 + 16 * 2 / 8, 1},  {0x61, 2, 32, 4 + 32 * 2 / 8, 1},
    {0x62, 2, 64, 4 + 64 * 2 / 8, 0},  {0x50, 3, 16, 4 + 16 * 3 / 8, 1},
    {0x51, 3, 32, 4 + 32 * 3 / 8, 1},  {0x52, 3, 64, 4 + 64 * 3 / 8, 1},
    {0x40, 4, 64, 4 + 64 * 4 / 8, 1},  {0x41, 4, 128, 4 + 128 * 4 / 8, 1},
    {0x30, 5, 32, 4 + 32 * 5 / 8, 1},  {0x31, 5, 64, 4 + 64 * 5 / 8, 1},
    {0x20, 6, 16, 4 + 16 * 6 / 8, 1},  {0x21, 6, 32, 4 + 32 * 6 / 8, 1},
    {0x22, 6, 64, 4 + 64 * 6 / 8, 0},  {0x10, 8, 32, 4 + 32, 1},
    {0x11, 8, 64, 4 + 64, 1},          {0x12, 8, 128, 4 + 128, 1},
};
#define N_FORMATS (sizeof(k_formats) / sizeof(k_formats[0]))

int orc_format_for_mlx(int bits, int group, orc_format* out) {
    for (size_t i = 0; i < N_FORMATS; i++) {
        if (k_formats[i].bits == bits && k_formats[i].group == group) {
            if (out) *out = k_formats[i];
            return 0;
        }
    }
    return -1;
}

int orc_format_for_scheme(int scheme, orc_format* out) {
    /* 0x42 (q4Group128ScaleF16Zero) aliases q4g128: QuantizationFormat.swift:1298-1301 */
    if (scheme == 0x42) scheme = 0x41;
    for (size_t i = 0; i < N_FORMATS; i++) {
        if (k_formats[i].scheme == scheme) {
            if (out) *out = k_formats[i];
            return 0;
        }
    }
    return -1;
}

/* ------------------------------------------------------------- float formats */

static uint32_t f32_bits(float v) {
    uint32_t b;
    memcpy(&b, &v, 4);
    return b;
}
static float bits_f32(uint32_t b) {
    float v;
    memcpy(&v, &b, 4);
    return v;
}

/* MC/BFloat16.swift:25-32: bits + 0x7FFF + lsb, then >> 16 (no NaN special case, wrapping add) */
uint16_t orc_bf16_from_f32(float v) {
    uint32_t bits = f32_bits(v);
    uint32_t lsb = (bits >> 16) & 1u;
    uint32_t rounded = bits + 0x7FFFu + lsb;
    return (uint16_t)(rounded >> 16);
}
float orc_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* IEEE binary16 <- binary32, round-to-nearest-even, with subnormals, inf and NaN. */
uint16_t orc_f16_from_f32(float v) {
    uint32_t x = f32_bits(v);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xFFu;
    uint32_t man = x & 0x7FFFFFu;
    if (exp == 0xFF) { /* inf / nan */
        if (man) return (uint16_t)(sign | 0x7E00u | (man >> 13));
        return (uint16_t)(sign | 0x7C00u);
    }
    int32_t e = (int32_t)exp - 127 + 15;
    if (e >= 0x1F) return (uint16_t)(sign | 0x7C00u); /* overflow -> inf */
    if (e <= 0) {                                      /* subnormal or zero */
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e); /* 14..24 */
        uint32_t half = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half & 1u))) half++;
        return (uint16_t)(sign | half);
    }
    uint32_t half = ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++; /* may carry into exp/inf */
    return (uint16_t)(sign | half);
}

float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float f = (float)man * (1.0f / 16777216.0f);
        return sign ? -f : f;
    }
    if (exp == 0x1F) return bits_f32(sign | 0x7F800000u | (man << 13));
    return bits_f32(sign | ((exp - 15 + 127) << 23) | (man << 13));
}

static float load_sb(const void* p, size_t i, int dtype) {
    switch (dtype) {
    case ORC_F16: return orc_f16_to_f32(((const uint16_t*)p)[i]);
    case ORC_BF16: return orc_bf16_to_f32(((const uint16_t*)p)[i]);
    default: return ((const float*)p)[i];
    }
}

/* -------------------------------------------------------------------- unpack */

/* One code from a block's `qs` bytes, written per bit width exactly as the reference's
 * per-weight expressions (QuantizationFormat.swift):
 *   2-bit :1060-1062   byte k>>2, shift (k&3)*2
 *   4-bit :1087-1089   byte k>>1, low nibble for even k
 *   3-bit :1121-1139   8 codes per 3 bytes, slot table
 *   5-bit :1172-1192   8 codes per 5 bytes, slot table
 *   6-bit :1221-1235   4 codes per 3 bytes, slot table
 *   8-bit :1254-1256   byte k                                                          */
uint32_t orc_unpack_code(const uint8_t* qs, int k, int bits) {
    switch (bits) {
    case 2: return (uint32_t)(qs[k >> 2] >> ((k & 3) * 2)) & 0x3u;
    case 4: return (uint32_t)(qs[k >> 1] >> ((k & 1) * 4)) & 0xFu;
    case 8: return qs[k];
    case 3: {
        const uint8_t* b = qs + (k >> 3) * 3;
        uint32_t b0 = b[0], b1 = b[1], b2 = b[2];
        switch (k & 7) {
        case 0: return b0 & 0x07u;
        case 1: return (b0 >> 3) & 0x07u;
        case 2: return ((b0 >> 6) & 0x03u) | ((b1 & 0x01u) << 2);
        case 3: return (b1 >> 1) & 0x07u;
        case 4: return (b1 >> 4) & 0x07u;
        case 5: return ((b1 >> 7) & 0x01u) | ((b2 & 0x03u) << 1);
        case 6: return (b2 >> 2) & 0x07u;
        default: return (b2 >> 5) & 0x07u;
        }
    }
    case 5: {
        const uint8_t* b = qs + (k >> 3) * 5;
        uint32_t b0 = b[0], b1 = b[1], b2 = b[2], b3 = b[3], b4 = b[4];
        switch (k & 7) {
        case 0: return b0 & 0x1Fu;
        case 1: return ((b0 >> 5) & 0x07u) | ((b1 & 0x03u) << 3);
        case 2: return (b1 >> 2) & 0x1Fu;
        case 3: return ((b1 >> 7) & 0x01u) | ((b2 & 0x0Fu) << 1);
        case 4: return ((b2 >> 4) & 0x0Fu) | ((b3 & 0x01u) << 4);
        case 5: return (b3 >> 1) & 0x1Fu;
        case 6: return ((b3 >> 6) & 0x03u) | ((b4 & 0x07u) << 2);
        default: return (b4 >> 3) & 0x1Fu;
        }
    }
    case 6: {
        const uint8_t* b = qs + (k >> 2) * 3;
        uint32_t b0 = b[0], b1 = b[1], b2 = b[2];
        switch (k & 3) {
        case 0: return b0 & 0x3Fu;
        case 1: return ((b0 >> 6) & 0x03u) | ((b1 & 0x0Fu) << 2);
        case 2: return ((b1 >> 4) & 0x0Fu) | ((b2 & 0x03u) << 4);
        default: return b2 >> 2;
        }
    }
    default: return 0xFFFFFFFFu;
    }
}

uint32_t orc_unpack_code_stream(const uint8_t* qs, size_t k, int bits) {
    size_t bit = k * (size_t)bits;
    size_t byte = bit >> 3;
    unsigned sh = (unsigned)(bit & 7);
    uint32_t v = qs[byte];
    if (sh + (unsigned)bits > 8) v |= (uint32_t)qs[byte + 1] << 8;
    return (v >> sh) & ((1u << bits) - 1u);
}

void orc_pack_stream(const uint8_t* codes, size_t n, int bits, uint8_t* out) {
    size_t nbytes = (n * (size_t)bits + 7) / 8;
    memset(out, 0, nbytes);
    uint32_t mask = (1u << bits) - 1u;
    for (size_t k = 0; k < n; k++) {
        size_t bit = k * (size_t)bits;
        size_t byte = bit >> 3;
        unsigned sh = (unsigned)(bit & 7);
        uint32_t v = ((uint32_t)codes[k] & mask) << sh;
        out[byte] |= (uint8_t)(v & 0xFFu);
        if (sh + (unsigned)bits > 8) out[byte + 1] |= (uint8_t)(v >> 8);
    }
}

/* -------------------------------------------------------------------- repack */

/* MC/STAF/STAFPayloadConverter.swift:209-282.  K is derived from the packed width as the
 * reference does (:230-236): bytesPerRow = packed*4, K = bytesPerRow*8/bits. */
int orc_repack_mlx_to_staf(int bits, int group, size_t n_rows, size_t packed_words_per_row,
                           const uint32_t* codes, const void* scales, const void* biases,
                           int sb_dtype, uint8_t* out_blocks) {
    orc_format f;
    if (orc_format_for_mlx(bits, group, &f)) return -1;
    size_t bytes_per_row = packed_words_per_row * 4;
    size_t k = bytes_per_row * 8 / (size_t)bits;
    size_t blocks_per_row = k / (size_t)group;
    size_t bytes_per_group = (size_t)group * (size_t)bits / 8;
    if (bytes_per_group * 8 != (size_t)group * (size_t)bits) return -2;
    const uint8_t* wbytes = (const uint8_t*)codes; /* little-endian word plane as bytes */
    for (size_t row = 0; row < n_rows; row++) {
        for (size_t b = 0; b < blocks_per_row; b++) {
            uint8_t* dst = out_blocks + (row * blocks_per_row + b) * (size_t)f.bytes_per_block;
            /* scales/biases normalised to f16 first (:223-224, :326-368) */
            uint16_t s = sb_dtype == ORC_F16
                             ? ((const uint16_t*)scales)[row * blocks_per_row + b]
                             : orc_f16_from_f32(load_sb(scales, row * blocks_per_row + b, sb_dtype));
            uint16_t z = sb_dtype == ORC_F16
                             ? ((const uint16_t*)biases)[row * blocks_per_row + b]
                             : orc_f16_from_f32(load_sb(biases, row * blocks_per_row + b, sb_dtype));
            memcpy(dst, &s, 2);
            memcpy(dst + 2, &z, 2);
            memcpy(dst + 4, wbytes + row * bytes_per_row + b * bytes_per_group, bytes_per_group);
        }
    }
    return 0;
}

int orc_staf_to_planes(int bits, int group, size_t n_rows, size_t k, const uint8_t* blocks,
                       uint32_t* codes, uint16_t* scales_f16, uint16_t* biases_f16) {
    orc_format f;
    if (orc_format_for_mlx(bits, group, &f)) return -1;
    if (k % (size_t)group) return -2;
    if ((k * (size_t)bits) % 32) return -3;
    size_t blocks_per_row = k / (size_t)group;
    size_t bytes_per_group = (size_t)group * (size_t)bits / 8;
    size_t bytes_per_row = k * (size_t)bits / 8;
    uint8_t* wbytes = (uint8_t*)codes;
    for (size_t row = 0; row < n_rows; row++) {
        for (size_t b = 0; b < blocks_per_row; b++) {
            const uint8_t* src = blocks + (row * blocks_per_row + b) * (size_t)f.bytes_per_block;
            memcpy(&scales_f16[row * blocks_per_row + b], src, 2);
            memcpy(&biases_f16[row * blocks_per_row + b], src + 2, 2);
            memcpy(wbytes + row * bytes_per_row + b * bytes_per_group, src + 4, bytes_per_group);
        }
    }
    return 0;
}

int orc_unpack_staf_codes(int bits, int group, size_t n_rows, size_t k, const uint8_t* blocks,
                          uint8_t* out_codes) {
    orc_format f;
    if (orc_format_for_mlx(bits, group, &f)) return -1;
    if (k % (size_t)group) return -2;
    size_t blocks_per_row = k / (size_t)group;
    for (size_t row = 0; row < n_rows; row++)
        for (size_t b = 0; b < blocks_per_row; b++) {
            const uint8_t* qs = blocks + (row * blocks_per_row + b) * (size_t)f.bytes_per_block + 4;
            for (int e = 0; e < group; e++)
                out_codes[row * k + b * (size_t)group + (size_t)e] =
                    (uint8_t)orc_unpack_code(qs, e, bits);
        }
    return 0;
}

int orc_unpack_plane_codes(int bits, size_t n_rows, size_t k, const uint32_t* codes,
                           uint8_t* out_codes) {
    if (bits < 2 || bits > 8 || bits == 7) return -1;
    if ((k * (size_t)bits) % 32) return -3;
    size_t bytes_per_row = k * (size_t)bits / 8;
    const uint8_t* wbytes = (const uint8_t*)codes;
    for (size_t row = 0; row < n_rows; row++)
        for (size_t c = 0; c < k; c++)
            out_codes[row * k + c] =
                (uint8_t)orc_unpack_code_stream(wbytes + row * bytes_per_row, c, bits);
    return 0;
}

/* ------------------------------------------------------------------- dequant */

int orc_dequant_staf_f32(int bits, int group, size_t n_rows, size_t k, const uint8_t* blocks,
                         float* out) {
    orc_format f;
    if (orc_format_for_mlx(bits, group, &f)) return -1;
    if (k % (size_t)group) return -2;
    size_t blocks_per_row = k / (size_t)group;
    for (size_t row = 0; row < n_rows; row++)
        for (size_t b = 0; b < blocks_per_row; b++) {
            const uint8_t* blk = blocks + (row * blocks_per_row + b) * (size_t)f.bytes_per_block;
            uint16_t sb, zb;
            memcpy(&sb, blk, 2);
            memcpy(&zb, blk + 2, 2);
            float scale = orc_f16_to_f32(sb), zero = orc_f16_to_f32(zb);
            for (int e = 0; e < group; e++) {
                float q = (float)orc_unpack_code(blk + 4, e, bits);
                float prod = scale * q; /* CPUWeightStore.swift:170: scale*Float(q) + zero */
                out[row * k + b * (size_t)group + (size_t)e] = prod + zero;
            }
        }
    return 0;
}

int orc_dequant_planes_f32(int bits, int group, size_t n_rows, size_t k, const uint32_t* codes,
                           const void* scales, const void* biases, int sb_dtype, float* out) {
    orc_format f;
    if (orc_format_for_mlx(bits, group, &f)) return -1;
    if (k % (size_t)group) return -2;
    if ((k * (size_t)bits) % 32) return -3;
    size_t blocks_per_row = k / (size_t)group;
    size_t bytes_per_row = k * (size_t)bits / 8;
    const uint8_t* wbytes = (const uint8_t*)codes;
    for (size_t row = 0; row < n_rows; row++)
        for (size_t b = 0; b < blocks_per_row; b++) {
            float scale = load_sb(scales, row * blocks_per_row + b, sb_dtype);
            float zero = load_sb(biases, row * blocks_per_row + b, sb_dtype);
            for (int e = 0; e < group; e++) {
                size_t c = b * (size_t)group + (size_t)e;
                float q = (float)orc_unpack_code_stream(wbytes + row * bytes_per_row, c, bits);
                float prod = scale * q;
                out[row * k + c] = prod + zero;
            }
        }
    return 0;
}

int orc_dequant_staf_bf16(int bits, int group, size_t n_rows, size_t k, const uint8_t* blocks,
                          uint16_t* out) {
    float* tmp = (float*)malloc(n_rows * k * sizeof(float));
    if (!tmp) return -9;
    int rc = orc_dequant_staf_f32(bits, group, n_rows, k, blocks, tmp);
    if (!rc)
        for (size_t i = 0; i < n_rows * k; i++) out[i] = orc_bf16_from_f32(tmp[i]);
    free(tmp);
    return rc;
}

/* ------------------------------------------------------------------ embedding */

int orc_embedding_lookup_staf_f32(int bits, int group, size_t vocab, size_t dim, const uint8_t* table,
                                  const int32_t* token_ids, size_t sequence_length, int has_scale,
                                  float embedding_scale, float* out) {
    orc_format f;
    if (orc_format_for_mlx(bits, group, &f)) return -1;
    if (dim % (size_t)group) return -2;
    size_t blocks_per_row = dim / (size_t)group;
    for (size_t pos = 0; pos < sequence_length; pos++) {
        int32_t tok = token_ids[pos];
        if (tok < 0 || (size_t)tok >= vocab) return -3; /* the reference reads out of bounds here */
        const uint8_t* row = table + (size_t)tok * blocks_per_row * (size_t)f.bytes_per_block;
        for (size_t d = 0; d < dim; d++) {
            const uint8_t* blk = row + (d / (size_t)group) * (size_t)f.bytes_per_block;
            uint16_t sb, zb;
            memcpy(&sb, blk, 2);
            memcpy(&zb, blk + 2, 2);
            float q = (float)orc_unpack_code(blk + 4, (int)(d % (size_t)group), bits);
            float prod = q * orc_f16_to_f32(sb); /* quantized * blockScale + blockZero */
            float value = prod + orc_f16_to_f32(zb);
            if (has_scale) value = value * embedding_scale;
            out[pos * dim + d] = value;
        }
    }
    return 0;
}

/* ---------------------------------------------------------------------- gemm */

void orc_gemm_f64(const float* w, const float* x, size_t m, size_t n, size_t k, size_t x_stride,
                  double* y) {
    for (size_t mi = 0; mi < m; mi++)
        for (size_t row = 0; row < n; row++) {
            double acc = 0.0;
            const float* wr = w + row * k;
            const float* xr = x + mi * x_stride;
            for (size_t c = 0; c < k; c++) acc += (double)wr[c] * (double)xr[c];
            y[mi * n + row] = acc;
        }
}

typedef struct {
    int bits, group, bytes_per_block, sb_dtype, planes;
    const uint8_t* blocks;
    const uint8_t* wbytes;
    const void* scales;
    const void* biases;
    const float* x;
    size_t m, n, k, x_stride, row_lo, row_hi;
    float* y;
} ref_job;

/* Loop nest of the reference kernels: m (grid.y) -> row -> block -> k, one fp32 accumulator. */
static void* ref_worker(void* arg) {
    ref_job* j = (ref_job*)arg;
    size_t blocks_per_row = j->k / (size_t)j->group;
    size_t bytes_per_row = j->k * (size_t)j->bits / 8;
    for (size_t mi = 0; mi < j->m; mi++) {
        const float* xr = j->x + mi * j->x_stride;
        for (size_t row = j->row_lo; row < j->row_hi; row++) {
            float sum = 0.0f;
            for (size_t b = 0; b < blocks_per_row; b++) {
                float scale, zero;
                const uint8_t* qs;
                if (j->planes) {
                    scale = load_sb(j->scales, row * blocks_per_row + b, j->sb_dtype);
                    zero = load_sb(j->biases, row * blocks_per_row + b, j->sb_dtype);
                    qs = j->wbytes + row * bytes_per_row + b * ((size_t)j->group * (size_t)j->bits / 8);
                } else {
                    const uint8_t* blk =
                        j->blocks + (row * blocks_per_row + b) * (size_t)j->bytes_per_block;
                    uint16_t sb, zb;
                    memcpy(&sb, blk, 2);
                    memcpy(&zb, blk + 2, 2);
                    scale = orc_f16_to_f32(sb);
                    zero = orc_f16_to_f32(zb);
                    qs = blk + 4;
                }
                const float* xb = xr + b * (size_t)j->group;
                for (int e = 0; e < j->group; e++) {
                    float wq = scale * (float)orc_unpack_code(qs, e, j->bits);
                    float w = wq + zero;
                    float p = w * xb[e];
                    sum = sum + p;
                }
            }
            j->y[mi * j->n + row] = sum;
        }
    }
    return NULL;
}

static int run_ref(ref_job base, int threads) {
    if (threads < 1) threads = 1;
    if ((size_t)threads > base.n) threads = (int)(base.n ? base.n : 1);
    pthread_t* tids = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)threads);
    ref_job* jobs = (ref_job*)malloc(sizeof(ref_job) * (size_t)threads);
    char* spawned = (char*)calloc((size_t)threads, 1);
    if (!tids || !jobs || !spawned) { free(tids); free(jobs); free(spawned); return -9; }
    size_t per = (base.n + (size_t)threads - 1) / (size_t)threads;
    for (int t = 0; t < threads; t++) {
        jobs[t] = base;
        jobs[t].row_lo = (size_t)t * per;
        jobs[t].row_hi = jobs[t].row_lo + per > base.n ? base.n : jobs[t].row_lo + per;
        if (jobs[t].row_lo >= base.n) break;
        if (threads > 1 && pthread_create(&tids[t], NULL, ref_worker, &jobs[t]) == 0)
            spawned[t] = 1;
        else
            ref_worker(&jobs[t]);
    }
    for (int t = 0; t < threads; t++)
        if (spawned[t]) pthread_join(tids[t], NULL);
    free(tids);
    free(jobs);
    free(spawned);
    return 0;
}

int orc_qgemm_staf_ref_f32(int bits, int group, const uint8_t* blocks, const float* x, size_t m,
                           size_t n, size_t k, size_t x_stride, float* y, int threads) {
    orc_format f;
    if (orc_format_for_mlx(bits, group, &f)) return -1;
    if (k % (size_t)group) return -2;
    ref_job j;
    memset(&j, 0, sizeof j);
    j.bits = bits; j.group = group; j.bytes_per_block = f.bytes_per_block; j.planes = 0;
    j.blocks = blocks; j.x = x; j.m = m; j.n = n; j.k = k; j.x_stride = x_stride; j.y = y;
    return run_ref(j, threads);
}

int orc_qgemm_planes_ref_f32(int bits, int group, const uint32_t* codes, const void* scales,
                             const void* biases, int sb_dtype, const float* x, size_t m, size_t n,
                             size_t k, size_t x_stride, float* y, int threads) {
    orc_format f;
    if (orc_format_for_mlx(bits, group, &f)) return -1;
    if (k % (size_t)group) return -2;
    if ((k * (size_t)bits) % 32) return -3;
    ref_job j;
    memset(&j, 0, sizeof j);
    j.bits = bits; j.group = group; j.bytes_per_block = f.bytes_per_block; j.planes = 1;
    j.sb_dtype = sb_dtype; j.wbytes = (const uint8_t*)codes; j.scales = scales; j.biases = biases;
    j.x = x; j.m = m; j.n = n; j.k = k; j.x_stride = x_stride; j.y = y;
    return run_ref(j, threads);
}

/* ---------------------------------------------------------- gated activation */

static float round_to(float v, int dtype) {
    if (dtype == ORC_BF16) return orc_bf16_to_f32(orc_bf16_from_f32(v));
    if (dtype == ORC_F16) return orc_f16_to_f32(orc_f16_from_f32(v));
    return v;
}

/* generateGatedActivation (MC/Generator/MetalSourceGenerator+NormAndElementwise.swift:196-249) */
void orc_gated_activation_f32(const float* gate, const float* up, size_t n, int kind, int dtype, float* out) {
    for (size_t i = 0; i < n; i++) {
        const float g = round_to(gate[i], dtype), u = round_to(up[i], dtype);
        float activated;
        if (kind == 1) {
            const float inner = 0.7978845608f * (g + 0.044715f * g * g * g);
            activated = 0.5f * g * (1.0f + tanhf(inner));
        } else {
            activated = g * (1.0f / (1.0f + expf(-g)));
        }
        out[i] = round_to(activated * u, dtype);
    }
}

/* -------------------------------------------------------------------- argmax */

int32_t orc_argmax_lowest(const float* v, size_t n) {
    float best = -INFINITY;
    int32_t idx = 0;
    for (size_t i = 0; i < n; i++)
        if (v[i] > best) { best = v[i]; idx = (int32_t)i; }
    return idx;
}

/* ----------------------------------------------------------------- quantizer */

static void store_sb(void* p, size_t i, int dtype, float v) {
    switch (dtype) {
    case ORC_F16: ((uint16_t*)p)[i] = orc_f16_from_f32(v); break;
    case ORC_BF16: ((uint16_t*)p)[i] = orc_bf16_from_f32(v); break;
    default: ((float*)p)[i] = v; break;
    }
}

int orc_quantize_affine(const float* w, size_t n_rows, size_t k, int bits, int group, int sb_dtype,
                        uint32_t* codes, void* scales, void* biases) {
    if (bits < 2 || bits > 8 || bits == 7) return -1;
    if (k % (size_t)group) return -2;
    if ((k * (size_t)bits) % 32) return -3;
    size_t blocks_per_row = k / (size_t)group;
    size_t bytes_per_row = k * (size_t)bits / 8;
    int qmax = (1 << bits) - 1;
    uint8_t* tmp = (uint8_t*)malloc(k);
    if (!tmp) return -9;
    for (size_t row = 0; row < n_rows; row++) {
        for (size_t b = 0; b < blocks_per_row; b++) {
            const float* g = w + row * k + b * (size_t)group;
            float mn = INFINITY, mx = -INFINITY;
            for (int e = 0; e < group; e++) { mn = fminf(mn, g[e]); mx = fmaxf(mx, g[e]); }
            float scale = (mx - mn) / (float)qmax;
            if (scale < 1e-10f) scale = 1e-10f;
            size_t gi = row * blocks_per_row + b;
            store_sb(scales, gi, sb_dtype, scale);
            store_sb(biases, gi, sb_dtype, mn);
            float sr = load_sb(scales, gi, sb_dtype), zr = load_sb(biases, gi, sb_dtype);
            for (int e = 0; e < group; e++) {
                float t = (g[e] - zr) / sr;
                int q = (int)roundf(t); /* half away from zero, as MSL round() */
                if (q < 0) q = 0;
                if (q > qmax) q = qmax;
                tmp[b * (size_t)group + (size_t)e] = (uint8_t)q;
            }
        }
        orc_pack_stream(tmp, k, bits, (uint8_t*)codes + row * bytes_per_row);
    }
    free(tmp);
    return 0;
}


/* ---- quantized KV cache ---------------------------------------------------------------------------- */
/* MC/Generator/MetalSourceGenerator+Attention.swift:1894-1921 */
int orc_kv_quant_bits(int scheme) {
    if (scheme == 0x10 || scheme == 0x11 || scheme == 0x12) return 8;
    if (scheme == 0x40 || scheme == 0x41 || scheme == 0x42) return 4;
    return 0;
}
int orc_kv_quant_group(int scheme) {
    switch (scheme) {
    case 0x10: return 32;
    case 0x11: return 64;
    case 0x12: return 128;
    case 0x40: return 64;
    case 0x41: case 0x42: return 128;
    default: return 0;
    }
}

/* MC/Buffer/MetalGraphAllocator.swift:60-114 */
size_t orc_kv_bytes_per_head_slot(int scheme, size_t head_dim) {
    size_t weights_per_block, bytes_per_block, alignment;
    if (scheme == 0x00 || scheme == 0x01 || scheme == 0xFF) { weights_per_block = 1; bytes_per_block = 2; alignment = 256; }
    else if (scheme == 0x02) { weights_per_block = 1; bytes_per_block = 4; alignment = 256; }
    else {
        orc_format f;
        if (scheme == 0x70) scheme = 0x10;           /* rotor schemes size as their base scheme */
        if (scheme == 0x71) scheme = 0x40;
        if (orc_format_for_scheme(scheme, &f) != 0 || !f.in_reference) return 0;
        weights_per_block = (size_t)f.group; bytes_per_block = (size_t)f.bytes_per_block; alignment = 64;
    }
    const size_t raw = (head_dim + weights_per_block - 1) / weights_per_block * bytes_per_block;
    return (raw + alignment - 1) / alignment * alignment;
}

size_t orc_kv_slot_offset(int layout_mode, size_t head, size_t position, size_t kv_heads, size_t max_positions,
                          size_t head_slot_bytes) {
    return layout_mode == 0 ? head * max_positions * head_slot_bytes + position * head_slot_bytes
                            : position * kv_heads * head_slot_bytes + head * head_slot_bytes;
}

/* MC/Generator/MetalSourceGenerator+Attention.swift:2057-2157 (packed), :1958-1971 (dense) */
int orc_kv_write_slot(int scheme, const float* src, size_t head_dim, uint8_t* slot) {
    if (scheme == 0x00) { for (size_t d = 0; d < head_dim; d++) ((uint16_t*)slot)[d] = orc_f16_from_f32(src[d]); return 0; }
    if (scheme == 0x01) { for (size_t d = 0; d < head_dim; d++) ((uint16_t*)slot)[d] = orc_bf16_from_f32(src[d]); return 0; }
    if (scheme == 0x02) { memcpy(slot, src, head_dim * 4); return 0; }
    const int bits = orc_kv_quant_bits(scheme);
    const size_t group = (size_t)orc_kv_quant_group(scheme);
    if (!bits) return -1;
    const size_t bytes_per_block = 4 + group * (size_t)bits / 8;
    const float levels = bits == 8 ? 255.0f : 15.0f;
    const int top = bits == 8 ? 255 : 15;
    for (size_t g = 0; g * group < head_dim; g++) {
        const size_t start = g * group;
        float lo = HUGE_VALF, hi = -HUGE_VALF;
        for (size_t i = 0; i < group && start + i < head_dim; i++) {
            lo = fminf(lo, src[start + i]);
            hi = fmaxf(hi, src[start + i]);
        }
        float scale = (hi - lo) / levels;
        if (scale < 1e-10f) scale = 1e-10f;
        uint8_t* block = slot + g * bytes_per_block;
        const uint16_t hs = orc_f16_from_f32(scale), hz = orc_f16_from_f32(lo);
        memcpy(block, &hs, 2);
        memcpy(block + 2, &hz, 2);
        if (bits == 8) {
            for (size_t i = 0; i < group && start + i < head_dim; i++) {
                int q = (int)roundf((src[start + i] - lo) / scale);
                block[4 + i] = (uint8_t)(q < 0 ? 0 : q > top ? top : q);
            }
        } else {
            for (size_t i = 0; i < group / 2 && start + 2 * i < head_dim; i++) {
                const float v0 = src[start + 2 * i];
                const float v1 = start + 2 * i + 1 < head_dim ? src[start + 2 * i + 1] : 0.0f;
                int q0 = (int)roundf((v0 - lo) / scale), q1 = (int)roundf((v1 - lo) / scale);
                q0 = q0 < 0 ? 0 : q0 > top ? top : q0;
                q1 = q1 < 0 ? 0 : q1 > top ? top : q1;
                block[4 + i] = (uint8_t)(q0 | (q1 << 4));
            }
        }
    }
    return 0;
}

/* MC/Generator/MetalSourceGenerator+Attention.swift:1923-1956 */
int orc_kv_read_slot(int scheme, const uint8_t* slot, size_t head_dim, float* out) {
    if (scheme == 0x00) { for (size_t d = 0; d < head_dim; d++) out[d] = orc_f16_to_f32(((const uint16_t*)slot)[d]); return 0; }
    if (scheme == 0x01) { for (size_t d = 0; d < head_dim; d++) out[d] = orc_bf16_to_f32(((const uint16_t*)slot)[d]); return 0; }
    if (scheme == 0x02) { memcpy(out, slot, head_dim * 4); return 0; }
    const int bits = orc_kv_quant_bits(scheme);
    const size_t group = (size_t)orc_kv_quant_group(scheme);
    if (!bits) return -1;
    const size_t bytes_per_block = 4 + group * (size_t)bits / 8;
    for (size_t d = 0; d < head_dim; d++) {
        const uint8_t* block = slot + d / group * bytes_per_block;
        const size_t i = d % group;
        uint16_t hs, hz;
        memcpy(&hs, block, 2);
        memcpy(&hz, block + 2, 2);
        const float scale = orc_f16_to_f32(hs), zero = orc_f16_to_f32(hz);
        const unsigned q = bits == 8 ? block[4 + i] : (i % 2 == 0 ? (block[4 + i / 2] & 0x0Fu) : (block[4 + i / 2] >> 4));
        out[d] = scale * (float)q + zero;
    }
    return 0;
}
