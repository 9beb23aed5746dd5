/*
 * CPU oracle for the group-affine quantized-linear path -- TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of the reference's (1amageek/swift-mlx-lm) packing,
 * dequantization, GEMV/GEMM and argmax semantics.  It exists so that the HIP kernels can be
 * checked against it.  Nothing in the shipped library links, loads or calls it; only the test
 * suite, the smoke check and the benchmark's CPU-baseline leg may.
 *
 * Every function names the reference file:line it follows (paths relative to the reference
 * checkout; MC/ = Sources/MetalCompiler/).
 *
 * Parity pinning status (what fixes each function besides its own formula):
 *   orc_unpack_code            pinned: reference slot formulas + literal byte vectors + brute force
 *   orc_pack_stream            pinned: literal byte vectors (0x76543210 -> 10 32 54 76), Q6 byte formulas
 *   orc_repack_mlx_to_staf     pinned: byte-exact layout vectors from the reference's round-trip tests
 *   orc_dequant_*              pinned: closed-form KATs with power-of-two scales (exact in fp32)
 *   orc_gemm_f64 / *_ref_f32   pinned: closed-form KATs (192.0 / 320.0, integer dot products)
 *   orc_bf16_from_f32          pinned: RNE rule + known bit patterns
 *   orc_f16_from_f32           pinned: exhaustive round trip over all 65536 half patterns vs numpy
 *   orc_embedding_lookup_*     pinned: the reference's two embedding vectors + row gather of the pinned dequant
 *   orc_kv_*                   pinned: head-slot sizes, the q8 round-trip vector and the unsigned-byte read
 *                              vector of the reference's tests; exact rational arithmetic for the codes
 *   orc_gated_activation_f32   the reference holds no value test of its swiglu / gelu_gated kernels (only pipeline
 *                              existence and benchmark tests): pinned by closed forms (g = 0, u = 0, large |g|,
 *                              silu(1), gelu_tanh(1) to 1e-7 from their definitions) and by an fp64 evaluation
 *   orc_argmax_lowest          PARITY UNPINNED against the reference (it holds no argmax value
 *                              test); pinned only by brute force against numpy on tiny vectors
 *   orc_quantize_affine        PARITY UNPINNED (the reference has no weight quantizer; this is an
 *                              input generator, not part of the path under test)
 */
#ifndef QLIN_ORACLE_H
#define QLIN_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype tags for scale/bias planes and activations */
enum { ORC_F16 = 0, ORC_BF16 = 1, ORC_F32 = 2 };

typedef struct {
    int32_t scheme;          /* STAF scheme identifier (MC/STAF/STAFFormat.swift:175-217) */
    int32_t bits;
    int32_t group;           /* weights per block == group size */
    int32_t bytes_per_block; /* 4 + group*bits/8 */
    int32_t in_reference;    /* 1 if registered by the reference, 0 for q6g64 / q2g64 */
} orc_format;

/* MC/STAF/QuantizationFormat.swift:1315-1335 (formatForMLXQuantization) + q6g64/q2g64. */
int orc_format_for_mlx(int bits, int group, orc_format* out);
/* MC/STAF/QuantizationFormat.swift:1284-1312 (format(for:)). */
int orc_format_for_scheme(int scheme, orc_format* out);

/* MC/BFloat16.swift:25-32, MC/STAF/STAFPayloadConverter.swift:116-121. */
uint16_t orc_bf16_from_f32(float v);
float orc_bf16_to_f32(uint16_t h);
/* Swift Float16(Float): IEEE binary16 round-to-nearest-even. */
uint16_t orc_f16_from_f32(float v);
float orc_f16_to_f32(uint16_t h);

/* MC/STAF/QuantizationFormat.swift:1060-1062,1087-1089,1121-1139,1172-1192,1221-1235,1254-1256 */
uint32_t orc_unpack_code(const uint8_t* qs, int k, int bits);
/* Closed form q_k = (stream >> k*bits) & mask over the LSB-first byte stream. */
uint32_t orc_unpack_code_stream(const uint8_t* qs, size_t k, int bits);
/* LSB-first bit-stream packer (Tests/MetalCompilerTests/Core/UnifiedGEMVBitLevelTests.swift:303-321). */
void orc_pack_stream(const uint8_t* codes, size_t n, int bits, uint8_t* out);

/* MC/STAF/STAFPayloadConverter.swift:209-282 (+ :326-368 scale normalisation). */
int orc_repack_mlx_to_staf(int bits, int group, size_t n_rows, size_t packed_words_per_row,
                           const uint32_t* codes, const void* scales, const void* biases,
                           int sb_dtype, uint8_t* out_blocks);
/* Inverse view: STAF blocks -> MLX planes (codes words, f16 scales, f16 biases). */
int orc_staf_to_planes(int bits, int group, size_t n_rows, size_t k, const uint8_t* blocks,
                       uint32_t* codes, uint16_t* scales_f16, uint16_t* biases_f16);

/* Codes only (uint8 per weight), from either layout. */
int orc_unpack_staf_codes(int bits, int group, size_t n_rows, size_t k, const uint8_t* blocks,
                          uint8_t* out_codes);
int orc_unpack_plane_codes(int bits, size_t n_rows, size_t k, const uint32_t* codes,
                           uint8_t* out_codes);

/* Quantized embedding gather (Sources/MetalCompiler/Generator/MetalSourceGenerator+Embedding.swift:79-153
 * for q4, :229-322 for every format): out[pos, d] = (float(q) * scale + zero) [* embeddingScale] of row
 * token_ids[pos], fp32, unfused.  Pinned by the reference's own vectors
 * (Tests/MetalCompilerTests/Core/QuantizedEmbeddingKernelTests.swift:48-150, 229-270).  Returns -3 for a
 * token id outside the table (the reference has no check). */
int orc_embedding_lookup_staf_f32(int bits, int group, size_t vocab, size_t dim, const uint8_t* table,
                                  const int32_t* token_ids, size_t sequence_length, int has_scale,
                                  float embedding_scale, float* out);

/* Sources/SwiftLM/CPUWeightStore.swift:141-172: w = scale*float(q) + zero, fp32, unfused. */
int orc_dequant_staf_f32(int bits, int group, size_t n_rows, size_t k, const uint8_t* blocks,
                         float* out);
int orc_dequant_planes_f32(int bits, int group, size_t n_rows, size_t k, const uint32_t* codes,
                           const void* scales, const void* biases, int sb_dtype, float* out);
/* MC/Generator/MetalSourceGenerator+Quantized.swift:403-413: bfloat(scale*q+zero). */
int orc_dequant_staf_bf16(int bits, int group, size_t n_rows, size_t k, const uint8_t* blocks,
                          uint16_t* out);

/* fp64 accumulation of given fp32 weights [N,K] against activations x [M, x_stride]. */
void orc_gemm_f64(const float* w, const float* x, size_t m, size_t n, size_t k, size_t x_stride,
                  double* y);

/* Reference loop nest, fp32 accumulate (MC/Generator/MetalSourceGenerator+Quantized.swift:116-153,
 * :539-573): for m, for row, for block, for k: sum += (scale*q+zero)*x.  Rows are split over
 * `threads` pthreads.  Output y[m*N + row]. */
int orc_qgemm_staf_ref_f32(int bits, int group, const uint8_t* blocks, const float* x, size_t m,
                           size_t n, size_t k, size_t x_stride, float* y, int threads);
int orc_qgemm_planes_ref_f32(int bits, int group, const uint32_t* codes, const void* scales,
                             const void* biases, int sb_dtype, const float* x, size_t m, size_t n,
                             size_t k, size_t x_stride, float* y, int threads);

/* The gated MLP's elementwise step (generateGatedActivation,
 * MC/Generator/MetalSourceGenerator+NormAndElementwise.swift:196-249): with T the buffer type `dtype`,
 *   g = float(T(gate[i])), u = float(T(up[i])), activated = silu: g * (1 / (1 + exp(-g)))
 *                                                           gelu: 0.5 g (1 + tanh(0.7978845608 (g + 0.044715 g g g)))
 *   out[i] = float(T(activated * u)), all arithmetic in fp32.  kind 0 = silu (swiglu), 1 = gelu tanh (gelu_gated). */
void orc_gated_activation_f32(const float* gate, const float* up, size_t n, int kind, int dtype, float* out);

/* Strict '>' scan from index 0 (MC/Generator/MetalSourceGenerator+Sampling.swift:80-90):
 * NaN never wins, ties keep the lowest index, empty / all-NaN input yields 0. */
int32_t orc_argmax_lowest(const float* v, size_t n);

/* Input generator: per-group affine quantizer (MC/STAF/README.md:102-103; rounding, clamp and
 * 1e-10 floor as MC/Generator/MetalSourceGenerator+Quantized.swift:427-433). */
int orc_quantize_affine(const float* w, size_t n_rows, size_t k, int bits, int group, int sb_dtype,
                        uint32_t* codes, void* scales, void* biases);

/* ---- quantized KV cache (MC/Generator/MetalSourceGenerator+Attention.swift) ------------------------- */
/* kv_quant_bits / kv_quant_group_size / kv_quant_bytes_per_block (:1894-1921): 8-bit g32/64/128, 4-bit g64/128/128z;
 * 0 for every other scheme.  Dense 0x00 / 0x01 / 0x02 are handled by the read / write functions. */
int orc_kv_quant_bits(int scheme);
int orc_kv_quant_group(int scheme);
/* KVCacheSpecification.bytesPerHeadSlot (MC/Buffer/MetalGraphAllocator.swift:60-114): ceil(headDim / weightsPerBlock)
 * blocks, rounded up to 64 bytes for packed formats and 256 for dense ones; every registered format is sizable.
 * 0 for a scheme without a registered format. */
size_t orc_kv_bytes_per_head_slot(int scheme, size_t head_dim);
/* write_kv_quantized_q8 / _q4 (:2057-2157) and write_kv_element_dense (:1958-1971) for one head vector:
 * per group min/max, scale = (max - min) / levels clamped to 1e-10, header = f16(scale), f16(min),
 * q = clamp(round((v - min) / scale), 0, levels) with the unrounded fp32 scale.  Bytes of the slot that the
 * reference does not write are left as they are.  Returns 0, or -1 for a scheme the kernels do not write. */
int orc_kv_write_slot(int scheme, const float* src, size_t head_dim, uint8_t* slot);
/* read_kv_element (:1923-1956) for elements [0, head_dim) of one slot. */
int orc_kv_read_slot(int scheme, const uint8_t* slot, size_t head_dim, float* out);
/* Byte offset of the slot of (head, position): layoutMode 0 = [head][position], 1 = [position][head] (:762-769). */
size_t orc_kv_slot_offset(int layout_mode, size_t head, size_t position, size_t kv_heads, size_t max_positions,
                          size_t head_slot_bytes);

#ifdef __cplusplus
}
#endif
#endif
