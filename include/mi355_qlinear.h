/*
 * mi355_qlinear.h -- C ABI of the MI355X (gfx950) group-affine quantized-linear library.
 *
 * One shared library (libmi355_qlinear.so) replaces the quantized-linear hot path that
 * swift-lm's MetalCompiler emits as generated Metal kernels over STAF-packed weights:
 * decode GEMV, prefill GEMM, dequant-to-bf16, LM head + argmax.  The reference has no FFI;
 * its "plugin API" is the Swift value-type contract between planner and encoder.  Each entry
 * point below names the reference interface it stands in for (paths relative to the reference
 * checkout, MC/ = Sources/MetalCompiler/).
 *
 * Conventions
 *   - Every call returns mi355q_status (0 = ok, negative = error).  No exception or unwinding
 *     crosses this boundary.  mi355q_last_error() returns the message of the last failing call
 *     on the calling thread.
 *   - Pointers named *_dev are device pointers (HBM) valid on the context's GPU; *_host are host
 *     pointers.  Device pointers may come from mi355q_buffer_alloc or from any other HIP
 *     allocator in the same process (a torch tensor's data_ptr, hipMalloc, ...).
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).  Launch calls are
 *     asynchronous: they validate, enqueue and return.
 *   - A context is thread-compatible, not thread-safe: callers serialise calls per context, as
 *     the reference serialises per MetalSubmissionContext
 *     (MC/Execution/MetalSubmissionContext.swift:56-120).
 *   - PRECONDITION: one stream per context at a time.  A context owns device scratch that its
 *     launches share (split-K partial sums of mi355q_qgemm, per-workgroup argmax keys of
 *     mi355q_argmax / mi355q_lmhead_argmax, part sums of the matrix-core decode kernels, the dequantised
 *     matrix of the two-dispatch prefill route, the bf16 rows that fp32 activations are split into, the
 *     clock probe).  Work enqueued through one context must therefore be ordered: on a single stream, or
 *     on streams the caller has ordered with events.  Launches of one context that overlap in time
 *     on different streams race on that scratch and return wrong results without an error; a
 *     caller that wants concurrent streams creates one context per stream (contexts are cheap:
 *     a few MB of scratch, grown on demand).
 *   - Shapes follow the reference: a weight is [N = outputDimension, K = inputDimension];
 *     K % groupSize == 0 is required (MC/Generator/MetalSourceGenerator+Quantized.swift:547);
 *     activations are [M = sequenceLength, x_row_stride >= K] in elements; outputs are [M, N].
 *   - There is no CPU fallback anywhere.  If no GPU is usable the context cannot be created and
 *     every compute entry point fails with MI355Q_ERR_DEVICE.
 */
#ifndef MI355_QLINEAR_H
#define MI355_QLINEAR_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355Q_API __attribute__((visibility("default")))
#define MI355Q_ABI_VERSION 1

typedef int32_t mi355q_status;
enum {
    MI355Q_OK = 0,
    MI355Q_ERR_INVALID_ARGUMENT = -1,   /* precondition / fatalError in the reference */
    MI355Q_ERR_UNSUPPORTED_FORMAT = -2, /* STAFConversionError.unsupportedQuantization
                                           (MC/STAF/STAFConversionPlanner.swift:179-187) */
    MI355Q_ERR_SHAPE = -3,              /* STAFConversionError.inconsistentQuantizationShape
                                           (MC/STAF/STAFPayloadConverter.swift:238-243) */
    MI355Q_ERR_NULL_HANDLE = -4,
    MI355Q_ERR_DEVICE = -5,             /* MetalCompilerError.deviceSetupFailed */
    MI355Q_ERR_OUT_OF_MEMORY = -6,
    MI355Q_ERR_KERNEL_NOT_FOUND = -7,   /* MetalCompilerError.kernelNotFound */
    MI355Q_ERR_SIZE_MISMATCH = -8,      /* payload size != rows*blocksPerRow*bytesPerBlock
                                           (Sources/SwiftLM/CPUWeightStore.swift:133-138) */
    MI355Q_ERR_INVALID_FILE = -9,       /* STAFLoadError.invalidFile (MC/STAF/STAFLoader.swift:318-330) */
    MI355Q_ERR_IO = -10,                /* STAFLoadError.mmapFailed, file system errors */
    MI355Q_ERR_NOT_FOUND = -11          /* entries[name] == nil */
};

/* BufferPrecision (MC/MetalDispatchTypes.swift:13-37) */
typedef enum { MI355Q_F16 = 0, MI355Q_BF16 = 1, MI355Q_F32 = 2 } mi355q_dtype;

/* STAFWeightLayout (MC/STAF/STAFWeightAccessRequest.swift:3-7): the canonical row-major STAF
 * interleaved blocks, or this library's specialized layout (split planes: uint32 code words
 * [N, K*bits/32] + scales [N, K/g] + biases [N, K/g], i.e. the MLX source planes). */
typedef enum {
    MI355Q_LAYOUT_STAF_BLOCKS = 0,
    MI355Q_LAYOUT_PLANES = 1,
    /* Matrix-core decode layout (4-bit, group 64, K % 128 == 0): records of 16 rows x 128 codes in
     * the order a wavefront loads them, each followed by its (scale, bias) words.  Serves
     * 1 <= M <= 16 per launch at nearly the cost of M = 1; the prefill GEMM on the matrix cores
     * reads the same records. */
    MI355Q_LAYOUT_TILE16 = 2
} mi355q_layout;

/* Launch flags */
enum {
    MI355Q_FLAG_NONE = 0,
    MI355Q_FLAG_FORCE_GENERIC = 1, /* run the reference-shaped per-code kernel (A/B and tests) */
    MI355Q_FLAG_FORCE_SMALL_M = 2, /* qgemm: use the small-M GEMV-style kernel whatever M is */
    MI355Q_FLAG_FORCE_MFMA = 4,    /* qgemm: use the fused MFMA kernel whatever M is */
    /* bit 3 (value 8) is taken by the measurement flag of mi355_qlinear_probe.h */
    MI355Q_FLAG_FORCE_TWO_STEP = 16, /* qgemm: dequantise to bf16 scratch, then the dense library GEMM, whatever M is */
    MI355Q_FLAG_FORCE_STREAM = 32  /* qgemm: the streamed-weight matrix-core kernel (4- / 8-bit planes or blocks, bf16 or f16 rows, M <= 96) */
};

/* ElementwiseFragment.ElementwiseKind of the gated MLP (MC/Compilable/MLPFragment.swift:16-27) and the activation its
 * kernel applies to the gate (GatedActivation, MC/Generator/MetalSourceGenerator+NormAndElementwise.swift:175-207) */
typedef enum {
    MI355Q_GATED_SILU = 0,      /* .swiglu:    g / (1 + exp(-g)) * up */
    MI355Q_GATED_GELU_TANH = 1  /* .geluGated: 0.5 g (1 + tanh(0.7978845608 (g + 0.044715 g^3))) * up */
} mi355q_gated_activation;

/* ------------------------------------------------------------------------------------------
 * Format descriptor: QuantizationFormat protocol (MC/STAF/QuantizationFormat.swift:25-153)
 * ---------------------------------------------------------------------------------------- */
typedef struct {
    uint8_t scheme_identifier;   /* QuantizationSchemeIdentifier (MC/STAF/STAFFormat.swift:175-217) */
    uint8_t bits;
    uint8_t is_quantized;
    uint8_t is_aligned;          /* bits in {2,4,8,16,32} (QuantizationFormat.swift:161-166) */
    uint32_t group_size;
    uint32_t weights_per_block;
    uint32_t bytes_per_block;    /* 4 + group*bits/8 */
    uint8_t has_direct_gemm;     /* directGEMMKernel() != nil (q4g64,q4g128,q8g32,q8g64) */
    uint8_t batched_gemm_counts; /* bit c set <=> batchedGEMMKernel(count: c) != nil */
    uint8_t in_reference_registry; /* 0 for q6g64 / q2g64 (new scheme ids 0x22 / 0x62) */
    uint8_t reserved0;
    uint32_t direct_gemm_threadgroup_memory_length; /* max(2g,256)*4 (QuantizationFormat.swift:364-367) */
    char block_struct_name[32];
    char gemv_kernel_name[32];          /* "gemv_q4_g64" */
    char gemm_kernel_name_f32s[32];     /* gemmKernelName(.float32) */
    char gemm_kernel_name[32];          /* gemmKernelName(decode precision) */
    char dequant_to_bfloat_kernel_name[32]; /* "dequant_q4_g64_bf16" */
    char embedding_lookup_token[16];    /* "q4_g64" */
} mi355q_format;

/* QuantizationFormatRegistry.formatForMLXQuantization(bits:groupSize:)
 * (QuantizationFormat.swift:1315-1335).  Unknown pair -> MI355Q_ERR_UNSUPPORTED_FORMAT; there
 * is no silent default (MC/Generator/MetalKernelSourceCatalog.swift:14). */
MI355Q_API mi355q_status mi355q_format_for_mlx_quantization(int bits, int group_size,
                                                            mi355q_format* out);
/* QuantizationFormatRegistry.format(for:) (QuantizationFormat.swift:1284-1312); 0x42 aliases
 * q4g128.  Dense and rotor schemes are outside this path -> MI355Q_ERR_UNSUPPORTED_FORMAT. */
MI355Q_API mi355q_status mi355q_format_for_scheme(uint8_t scheme_identifier, mi355q_format* out);
/* Enumerate the registry (CaseIterable analogue) for contract tests. */
MI355Q_API int32_t mi355q_format_count(void);
MI355Q_API mi355q_status mi355q_format_at(int32_t index, mi355q_format* out);

/* bf16 round-to-nearest-even of the host type (MC/BFloat16.swift:25-32). */
MI355Q_API uint16_t mi355q_bf16_from_f32(float value);

/* STAFPayloadConverter.repackMLXQuantized (MC/STAF/STAFPayloadConverter.swift:209-282) on host
 * memory: MLX planes -> STAF interleaved blocks, scales/biases normalised to f16 (:326-368).
 * out_capacity must be >= n_rows * (K/group) * bytes_per_block. */
MI355Q_API mi355q_status mi355q_repack_mlx_to_staf(uint8_t scheme_identifier, size_t n_rows,
                                                   size_t packed_words_per_row,
                                                   const uint32_t* codes_host,
                                                   const void* scales_host,
                                                   const void* biases_host, mi355q_dtype sb_dtype,
                                                   uint8_t* out_blocks_host, size_t out_capacity);

/* ------------------------------------------------------------------------------------------
 * Context, memory, streams, events  (MTLDevice / MTLBuffer / MTLCommandQueue stand-ins)
 * ---------------------------------------------------------------------------------------- */
typedef struct mi355q_context mi355q_context;
typedef struct mi355q_weight mi355q_weight;

typedef struct {
    char name[64];
    char arch[32];              /* "gfx950..." */
    int32_t compute_units;
    int32_t wavefront_size;
    int32_t lds_bytes_per_workgroup;
    int32_t reserved0;
    uint64_t hbm_bytes;
    double hbm_peak_gbps;       /* published: 8000 */
    double mfma_bf16_peak_tflops; /* published dense: 2500 */
} mi355q_device_info;

MI355Q_API const char* mi355q_last_error(void);
MI355Q_API int32_t mi355q_abi_version(void);
/* MTLCreateSystemDefaultDevice analogue.  Fails with MI355Q_ERR_DEVICE when there is no GPU. */
MI355Q_API mi355q_status mi355q_context_create(int device_index, mi355q_context** out);
MI355Q_API mi355q_status mi355q_context_destroy(mi355q_context* ctx);
MI355Q_API mi355q_status mi355q_device_query(mi355q_context* ctx, mi355q_device_info* out);
/* Whether launches through this context may hand a dense product to the platform's GEMM library (hipBLASLt, opened
 * with dlopen on first use): the second half of the two-dispatch prefill route, as the reference's dense product is
 * the platform's matmul2d (MC/Generator/MetalSourceGenerator+Linear.swift:18-81).  On by default; with 0 every
 * launch stays on this library's own kernels (the fused, streamed-weight and decode kernels serve every shape, more
 * slowly where the route was the quicker one), and the library is never opened. */
MI355Q_API mi355q_status mi355q_context_set_library_use(mi355q_context* ctx, int enabled);

MI355Q_API mi355q_status mi355q_buffer_alloc(mi355q_context* ctx, size_t bytes, void** out_dev);
MI355Q_API mi355q_status mi355q_buffer_free(mi355q_context* ctx, void* dev);
MI355Q_API mi355q_status mi355q_buffer_upload(mi355q_context* ctx, void* dst_dev,
                                              const void* src_host, size_t bytes);
MI355Q_API mi355q_status mi355q_buffer_download(mi355q_context* ctx, void* dst_host,
                                                const void* src_dev, size_t bytes);
MI355Q_API mi355q_status mi355q_buffer_fill(mi355q_context* ctx, void* stream, void* dst_dev,
                                            uint32_t word, size_t n_words);

MI355Q_API mi355q_status mi355q_stream_create(mi355q_context* ctx, void** out_stream);
MI355Q_API mi355q_status mi355q_stream_destroy(mi355q_context* ctx, void* stream);
MI355Q_API mi355q_status mi355q_stream_synchronize(mi355q_context* ctx, void* stream);
MI355Q_API mi355q_status mi355q_event_create(mi355q_context* ctx, void** out_event);
MI355Q_API mi355q_status mi355q_event_destroy(mi355q_context* ctx, void* event);
MI355Q_API mi355q_status mi355q_event_record(mi355q_context* ctx, void* event, void* stream);
MI355Q_API mi355q_status mi355q_event_synchronize(mi355q_context* ctx, void* event);
MI355Q_API mi355q_status mi355q_event_elapsed_ms(mi355q_context* ctx, void* start, void* stop,
                                                 float* out_ms);

/* ------------------------------------------------------------------------------------------
 * Packed weights: STAFWeightStore.resolvedBufferAccess / registeringSpecializedBufferAccess
 * (MC/STAF/STAFLoader.swift:213-299) and STAFSpecializedWeightStoreBuilder.prepare
 * (MC/STAF/STAFSpecializedWeightStoreBuilder.swift:15-31).  A handle is immutable after
 * creation.  "prepare" handles own their device memory; "wrap" handles borrow it.
 * ---------------------------------------------------------------------------------------- */
typedef struct {
    uint8_t scheme_identifier;
    uint8_t bits;
    uint8_t layout;             /* mi355q_layout */
    uint8_t sb_dtype;           /* dtype of scale/bias: F16 for STAF blocks, F16/BF16 for planes */
    uint32_t group_size;
    uint64_t n_rows;            /* N */
    uint64_t k;                 /* K */
    uint64_t weight_bytes;      /* algorithmic: N*(K/g)*bytes_per_block
                                   (MC/Compiler/MetalCompilerDiagnostics.swift:192-203) */
    const void* blocks_dev;     /* STAF layout */
    const void* codes_dev;      /* planes layout */
    const void* scales_dev;
    const void* biases_dev;
    uint8_t owns_memory;
    uint8_t reserved[7];
} mi355q_weight_info;

/* From MLX source planes in host memory (uint32 [N, K*bits/32]; scales/biases [N, K/g] in
 * sb_dtype).  Whatever the layout, every scale and bias takes the value the converter's
 * normalizeScaleToFloat16 gives it (MC/STAF/STAFConverter.swift:326-368): F32 and BF16 values are
 * rounded to F16, round to nearest even, so values under the F16 normal range (6.1e-5) lose bits
 * or flush and values over 65504 become infinite, exactly as in a model.staf the reference wrote.
 * F32 planes are stored as F16; BF16 planes stay BF16 on the PLANES and TILE16 layouts, holding
 * those rounded values (each has an exact BF16 spelling), and the block layout stores the F16
 * header: one MLX tensor therefore decodes to the same weights on all three layouts.  `layout`
 * picks the device layout; STAF_BLOCKS repacks on the host first (the reference's load path). */
MI355Q_API mi355q_status mi355q_weight_prepare_mlx(mi355q_context* ctx, uint8_t scheme_identifier,
                                                   uint64_t n_rows, uint64_t k,
                                                   const uint32_t* codes_host,
                                                   const void* scales_host,
                                                   const void* biases_host, mi355q_dtype sb_dtype,
                                                   mi355q_layout layout, mi355q_weight** out);
/* From STAF interleaved blocks in host memory (a mapped model.staf payload).  payload_bytes
 * must equal N*(K/g)*bytes_per_block.  layout = PLANES de-interleaves once, at load time. */
MI355Q_API mi355q_status mi355q_weight_prepare_staf(mi355q_context* ctx, uint8_t scheme_identifier,
                                                    uint64_t n_rows, uint64_t k,
                                                    const uint8_t* blocks_host,
                                                    size_t payload_bytes, mi355q_layout layout,
                                                    mi355q_weight** out);
/* Zero-copy: borrow device memory that already holds the payload -- the (buffer, offset) pair
 * of STAFWeightBufferAccess.  The caller keeps the memory alive and unchanged. */
MI355Q_API mi355q_status mi355q_weight_wrap_staf(mi355q_context* ctx, uint8_t scheme_identifier,
                                                 uint64_t n_rows, uint64_t k,
                                                 const void* blocks_dev, size_t payload_bytes,
                                                 mi355q_weight** out);
MI355Q_API mi355q_status mi355q_weight_wrap_planes(mi355q_context* ctx, uint8_t scheme_identifier,
                                                   uint64_t n_rows, uint64_t k,
                                                   const void* codes_dev, const void* scales_dev,
                                                   const void* biases_dev, mi355q_dtype sb_dtype,
                                                   mi355q_weight** out);
MI355Q_API mi355q_status mi355q_weight_query(const mi355q_weight* w, mi355q_weight_info* out);
MI355Q_API mi355q_status mi355q_weight_destroy(mi355q_weight* w);

/* ------------------------------------------------------------------------------------------
 * Launches
 * ---------------------------------------------------------------------------------------- */

/* Decode projection: gemv_q{b}_g{g} (generateUnifiedQuantizedGEMV,
 * MC/Generator/MetalSourceGenerator+Quantized.swift:496-575; bindings 0=input 1=weight
 * 2=output 3=inputDimension 4=outputDimension, MC/Compiler/MetalDispatchStepBuilder.swift:679-688)
 * widened to the sequence signature for small M (5=sequenceLength 6=inputRowStride,
 * :116-153).  y[m*y_row_stride + n] = sum_k (scale*q + zero) * x[m*x_row_stride + k], fp32
 * accumulation, result rounded once to y_dtype.  1 <= M <= 8.  y_row_stride 0 means N.
 * Activation types: bf16 and f16 rows are read by the decode kernels directly.  fp32 rows are split on the
 * device into three bf16 rows each whose sum is the fp32 row exactly (8 + 8 + 8 significant bits); the bf16
 * kernel of the layout runs on the 3 M rows (the matrix is still read once, every product is exact) and a small
 * launch adds the three partial results of a row (the split rows and partial results live in a scratch buffer
 * of the context, grown on first use).  The matrix-core kernels (TILE16 records; 4- and 8-bit planes from three
 * rows) split f16 rows into two bf16 rows each (8 + 3 bits) while staging them, and add the two results of a
 * row before the store: eight f16 rows a launch. */
MI355Q_API mi355q_status mi355q_qgemv(mi355q_context* ctx, void* stream, const mi355q_weight* w,
                                      const void* x_dev, mi355q_dtype x_dtype, void* y_dev,
                                      mi355q_dtype y_dtype, uint32_t m, uint32_t x_row_stride,
                                      uint32_t y_row_stride, uint32_t flags);

/* Prefill projection: gemm_q4_g64_f32s / gemm_q8_g32_f32s (:22-156) and the two-step
 * dequant_q*_bf16 + gemm_bf16_f32s path (:361-416, MC/Generator/MetalSourceGenerator+Linear.swift:18-81).
 * Any M >= 1; M is a run-time value (the reference rebinds sequenceLength per call,
 * MC/Compiler/MetalPrefillStepBuilder.swift:728-732).  Four routes, all with fp32 accumulation, chosen by
 * measured cost unless flags say otherwise (mi355q_plan_prefill_steps reports the choice); the first keeps
 * the dequantised weights unrounded (the decode kernels' arithmetic), the others round them once to bf16
 * (the numerics of the reference's dequant -> bf16 -> GEMM route):
 *   - small M (up to 8 rows; 16 on TILE16 records and on q4 / q8 planes; up to 32 in two launches where the
 *     next route does not read the weight): the GEMV-style decode kernels;
 *   - 17 to 96 bf16 rows, or 9 to 96 f16 rows, on 4-bit planes (groups of 64 or 128) and 8-bit planes (groups
 *     of 32, 64 or 128), on the same formats left in STAF blocks from 3, 5 or 9 rows by the size of the
 *     matrix, and on 2-, 3-, 5- and 6-bit codes in groups of 64 (planes and blocks) from 5 rows (mi355q_qgemv included): the streamed-weight kernel -- weights dequantised in registers
 *     straight into the matrix cores' operand, the activations alone staged in LDS.  Up to 32 rows (groups of
 *     64 or 128) it keeps the weights unrounded like the decode kernels; beyond, and with groups of 32, it
 *     rounds them once to the activations' type.  Through mi355q_batched_qgemm two or three matrices share one
 *     launch (whose split of K follows the launch's size: its fp32 sums may be ordered differently from those of
 *     separate calls); fp32 rows split into three bf16 rows each ride on it up to 32 fp32 rows;
 *   - ONE fused kernel: code tiles are dequantised to bf16 in LDS and contracted on MFMA (the planes
 *     and TILE16 layouts, formats q4 g64/g128, q8 g32/g64, q6/q3/q2 g64, bf16 activations);
 *   - two dispatches, as the reference's second route: the whole matrix is dequantised to bf16 in a
 *     scratch matrix of the context (N*K*2 bytes, plus 64 MiB of library workspace) and multiplied by
 *     the platform's dense GEMM library (hipBLASLt, opened with dlopen on first use; the reference
 *     calls matmul2d there).  Serves every registered format on every layout: from 16 rows where the
 *     fused kernel does not read the weight; beside it from 512 rows (768 when N >= 8192, 2048 when K > N).  bf16
 *     activations, fp32 or bf16 output, K and the row stride multiples of 8, 16-byte aligned x; f16
 *     activations likewise in f16; fp32 activations into an fp32 result as two bf16 products (bf16
 *     weights as in gemm_bf16_f32s, the activations split into bf16 high and low halves).  The
 *     first eager call of a shape times the library's candidate algorithms once (a few milliseconds)
 *     and keeps the quickest.  When the library is absent or has no algorithm, the other routes serve.
 *     Batches of 2 to 15 rows whose layout or activation type no decode kernel reads (rows of the
 *     block layout that are not whole 16-byte units, fp32 rows beyond those the bf16 split of
 *     mi355q_qgemv serves: sixteen on TILE16 records and 4- / 8-bit planes, two elsewhere) take it too, there with UNROUNDED fp32 weights (N*K*4 bytes of scratch),
 *     the activations widened to fp32, the library's fp32 product and the result narrowed to y_dtype:
 *     the result keeps the decode kernels' accuracy, at a cost that does not grow with M.
 * Launches that split K over workgroups (few output
 * tiles at short M; on the TILE16 layout, rows too long for M staged activation rows) keep fp32
 * partial results in a scratch buffer of the context, grown on first use: two such launches of one
 * context must not overlap on different streams, and the first one of a size allocates (run a plan
 * once before capturing it, as mi355q_plan_graph_build does). */
MI355Q_API mi355q_status mi355q_qgemm(mi355q_context* ctx, void* stream, const mi355q_weight* w,
                                      const void* x_dev, mi355q_dtype x_dtype, void* y_dev,
                                      mi355q_dtype y_dtype, uint32_t m, uint32_t x_row_stride,
                                      uint32_t y_row_stride, uint32_t flags);

/* The elementwise step of the gated MLP, swiglu / gelu_gated (generateGatedActivation,
 * MC/Generator/MetalSourceGenerator+NormAndElementwise.swift:196-249; ElementwiseFragment of
 * MC/Compilable/MLPFragment.swift:7-14): out[s, i] = T(activation(float(gate[s, i])) * float(up[s, i])) for
 * i < dimension, s < sequence_length, all three buffers of type T with rows `row_stride` elements apart
 * (0 = dimension).  gate, up and out may alias. */
MI355Q_API mi355q_status mi355q_gated_activation_apply(mi355q_context* ctx, void* stream, const void* gate_dev,
                                                       const void* up_dev, void* out_dev, mi355q_dtype dtype,
                                                       uint32_t dimension, uint32_t sequence_length,
                                                       uint32_t row_stride, mi355q_gated_activation activation);

/* MLPFragment's first two steps as one call (MC/Compilable/MLPFragment.swift:7-14): the batched gate_proj + up_proj
 * projection of x and the gated activation, out[s, :] = activation(x[s] Wgate^T) * (x[s] Wup^T), one [M, N] result
 * instead of two and no elementwise dispatch.  Both weights share N, K, scheme and layout.  The gate and up sums are
 * rounded to y_dtype before the activation, as the reference's elementwise kernel reads them from buffers of that
 * type, so the result is that of mi355q_batched_qgemm followed by mi355q_gated_activation_apply up to the order of
 * the fp32 sums.  One activation row on split planes runs as ONE launch (a wavefront owns a gate row and the up row
 * of the same index), and so do 17 to 96 rows on the streamed-weight kernel (a workgroup's two row blocks are the same
 * rows of the two matrices) and, on 4-bit matrices, prompts from 97 rows on the wide-tile kernel (a wavefront's two
 * column fragments are), the activation in their epilogues; other shapes run the projections into the context's
 * scratch and then the elementwise kernel. */
MI355Q_API mi355q_status mi355q_gated_qgemm(mi355q_context* ctx, void* stream, const mi355q_weight* w_gate,
                                            const mi355q_weight* w_up, const void* x_dev, mi355q_dtype x_dtype,
                                            void* y_dev, mi355q_dtype y_dtype, uint32_t m, uint32_t x_row_stride,
                                            uint32_t y_row_stride, mi355q_gated_activation activation,
                                            uint32_t flags);

/* batched_gemm_q4_g64_{2,3} (:166-338; bindings MC/Compiler/MetalPrefillStepBuilder.swift:928-955):
 * 2 or 3 projections sharing one input (gate+up, q+k+v) in one launch: at decode and small batches on the decode
 * kernels, at 17 to 96 rows on the streamed-weight kernel, from 97 rows (4-bit matrices whose widths but the last
 * are multiples of 256) on the wide-tile prefill kernel; a launch per projection elsewhere.  All weights must share
 * K, scheme and layout.  Outputs are separate [M, N_i] buffers with row stride N_i. */
MI355Q_API mi355q_status mi355q_batched_qgemm(mi355q_context* ctx, void* stream, uint32_t count,
                                              const mi355q_weight* const* weights,
                                              const void* x_dev, mi355q_dtype x_dtype,
                                              void* const* y_devs, mi355q_dtype y_dtype,
                                              uint32_t m, uint32_t x_row_stride, uint32_t flags);

/* dequant_q{b}_g{g}_bf16 (generateUnifiedDequantToBFloat, :361-416): whole matrix to row-major
 * bf16 [N, K], each weight bf16_rne(scale*q + zero). */
MI355Q_API mi355q_status mi355q_dequant_bf16(mi355q_context* ctx, void* stream,
                                             const mi355q_weight* w, void* out_bf16_dev);

/* CPUWeightStore.decodeQuantized (Sources/SwiftLM/CPUWeightStore.swift:109-174): the whole matrix as row-major fp32
 * [N, K], each weight scale * float(q) + zero evaluated as the reference's host code does (:170): the product rounded
 * to fp32, then the sum rounded to fp32, no fused multiply-add.  Any registered format and any layout (the reference
 * decodes 4- and 8-bit blocks only, :156-166). */
MI355Q_API mi355q_status mi355q_dequant_f32(mi355q_context* ctx, void* stream,
                                            const mi355q_weight* w, float* out_f32_dev);

/* gemm_bf16_f32s (generateMPPGEMM, MC/Generator/MetalSourceGenerator+Linear.swift:18-81):
 * C[M,N] = A[M, a_row_stride>=K] * B[N,K]^T with B dense bf16 (the dequant scratch), MFMA,
 * fp32 accumulation.  From 128 rows the product goes to the platform's dense GEMM library, as the
 * reference's goes to matmul2d (bf16 A, fp32 or bf16 C, aligned operands); else, and when the
 * library cannot serve, this library's own matrix-core kernel runs. */
MI355Q_API mi355q_status mi355q_gemm_bf16(mi355q_context* ctx, void* stream, const void* a_dev,
                                          mi355q_dtype a_dtype, const void* b_bf16_dev,
                                          void* c_dev, mi355q_dtype c_dtype, uint32_t m,
                                          uint32_t n, uint32_t k, uint32_t a_row_stride,
                                          uint32_t c_row_stride);

/* Quantized embedding gather: embedding_lookup[_seq]_q{b}_g{g}
 * (MC/Generator/MetalSourceGenerator+Embedding.swift:79-153 for q4, :229-322 for every format; bindings
 * 0=tokenIDs 1=table 2=output 3=embeddingDim 4=sequenceLength 5=embeddingScale).  `table` is a packed
 * weight of shape [vocabularySize, embeddingDim] in any layout (a tied LM head can be passed as is);
 * token ids are int32 in device memory; out[pos*out_row_stride + d] = (float(q)*scale + zero)
 * [* embedding_scale], rounded once to out_dtype.  sequence_length 1 is the decode variant.  A token
 * id outside the table gives a row of zeros (the reference reads out of bounds). */
MI355Q_API mi355q_status mi355q_embedding_lookup(mi355q_context* ctx, void* stream,
                                                 const mi355q_weight* table,
                                                 const int32_t* token_ids_dev,
                                                 uint32_t sequence_length, void* out_dev,
                                                 mi355q_dtype out_dtype, uint32_t out_row_stride,
                                                 int has_embedding_scale, float embedding_scale);

/* Debug / parity: every code of the matrix as one byte, row-major [N, K]. */
MI355Q_API mi355q_status mi355q_unpack_codes(mi355q_context* ctx, void* stream,
                                             const mi355q_weight* w, uint8_t* out_codes_dev);

/* argmax / argmax_f32 (generateArgmax, MC/Generator/MetalSourceGenerator+Sampling.swift:62-107;
 * bindings 0=logits 1=int* result 2=vocabularySize).  Strict '>' from -inf with index 0 as
 * the start value: NaN never wins; ties resolve to the LOWEST index (a rule this library adds:
 * the reference's reduction order does not define ties).  Vocabulary-sized vectors run as two
 * launches through a small scratch of the context, as the fused head below does: calls on one
 * context that overlap in time (different streams) race on it; give each stream its own context. */
MI355Q_API mi355q_status mi355q_argmax(mi355q_context* ctx, void* stream, const void* logits_dev,
                                       mi355q_dtype dtype, uint32_t vocabulary_size,
                                       int32_t* token_out_dev);

/* OutputHeadFragment = LinearFragment + ArgmaxFragment (MC/Compilable/OutputHeadFragment.swift:5-8)
 * fused into one launch: fp32 logits [N] (optional, may be NULL) and the greedy token index.
 * M = 1 (the reference runs the head in lastToken mode, MC/Compiler/MetalPrefillStepBuilder.swift:493-507).
 * The fused kernels read bf16 activations on every layout and f16 ones on planes and blocks; fp32 activations
 * (the prefill's last token) and f16 ones on TILE16 records run the projection on its own fast route into the
 * logits buffer, which is then required, and an arg-max launch picks the token. */
MI355Q_API mi355q_status mi355q_lmhead_argmax(mi355q_context* ctx, void* stream,
                                              const mi355q_weight* w, const void* x_dev,
                                              mi355q_dtype x_dtype, float* logits_f32_dev,
                                              int32_t* token_out_dev, uint32_t flags);

/* mi355q_lmhead_argmax for callers that must not allocate.  No counterpart in the reference: it is for code that
 * runs under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc.  Same arguments, kernels
 * and results as mi355q_lmhead_argmax; the one partial key per workgroup that the head launch leaves for its
 * finishing launch lives in a device array of the library image (258 KiB per GPU, held until the process ends)
 * instead of the context's allocation, and the call makes no hipMalloc, hipFree or other allocating call: where
 * mi355q_lmhead_argmax would run the projection on a route that keeps scratch in the context (fp32 activations as
 * three bf16 rows; f16 activations on TILE16 records), this entry point runs the per-code projection kernel and the
 * arg-max launch instead (slower, same token up to ties between logits that differ in their last bits; a logits
 * buffer is required there, as for every head that is not fused).
 * Limit: a head launch of more than mi355q_lmhead_argmax_static_capacity() = 32768 workgroups (524288 rows of up to
 * 2048 4-bit codes, 262144 rows of up to 4096) is refused with MI355Q_ERR_SHAPE.  Every call on a GPU shares that
 * GPU's array and overwrites the keys it uses (nothing has to be cleared between calls: a call reads back only the
 * keys its own launch wrote): calls that overlap in time on one GPU race, whatever their contexts and streams. */
MI355Q_API mi355q_status mi355q_lmhead_argmax_static(mi355q_context* ctx, void* stream,
                                                     const mi355q_weight* w, const void* x_dev,
                                                     mi355q_dtype x_dtype, float* logits_f32_dev,
                                                     int32_t* token_out_dev, uint32_t flags);
MI355Q_API uint32_t mi355q_lmhead_argmax_static_capacity(void);

/* ------------------------------------------------------------------------------------------
 * Planner mirror: launch shapes, kernel selection and the quantization-plan record
 * ---------------------------------------------------------------------------------------- */

/* DecodeProjectionShapeFamily (MC/Compiler/MetalCompileContext.swift:5-90) */
typedef enum {
    MI355Q_FAMILY_GENERIC = 0,
    MI355Q_FAMILY_LARGE_DENSE = 1,
    MI355Q_FAMILY_INPUT2048_SQUARE = 2,
    MI355Q_FAMILY_INPUT2048_6144 = 3,
    MI355Q_FAMILY_INPUT2048_8192 = 4,
    MI355Q_FAMILY_INPUT2048_EXPANDED = 5,
    MI355Q_FAMILY_INPUT8192_TILED = 6,
    MI355Q_FAMILY_VOCAB_DENSE = 7
} mi355q_shape_family;

/* MetalQuantizationExecutionPath / FallbackReason (MC/Compiler/MetalQuantizationPlan.swift:22-27,290-298) */
typedef enum {
    MI355Q_PATH_PREFILL_PROJECTION = 0,
    MI355Q_PATH_DECODE_PROJECTION = 1
} mi355q_execution_path;
typedef enum {
    MI355Q_FALLBACK_NONE = 0,
    MI355Q_FALLBACK_INPUT_STRIDE_MISMATCH = 1,
    MI355Q_FALLBACK_LAST_TOKEN_USES_DECODE_KERNEL = 2,
    MI355Q_FALLBACK_DISABLED_BY_ENVIRONMENT = 3,
    MI355Q_FALLBACK_UNAVAILABLE_ACCELERATION = 4
} mi355q_fallback_reason;

/* One planned dispatch: MetalDispatchStep / MetalPrefillStep reduced to what a HIP launch
 * needs (MC/Execution/MetalDecodePlan.swift:6-97, MC/Execution/MetalPrefillPlan.swift:6-140)
 * together with its MetalQuantizationPlanEntry (MC/Compiler/MetalQuantizationPlan.swift:304-318). */
typedef struct {
    char kernel_name[48];        /* reference-compatible name, e.g. "gemv_q4_g64" */
    char device_kernel[48];      /* the HIP kernel variant that will run */
    char kernel_family[32];      /* MetalQuantizationKernelFamily.description */
    uint32_t grid[3];            /* workgroups */
    uint32_t block[3];           /* threads per workgroup */
    uint32_t lds_bytes;
    uint32_t rows_per_workgroup;
    uint32_t reference_simdgroups;   /* DecodeProjectionShapeFamily.preferredSimdgroups */
    uint32_t reference_tile_elements;
    int32_t shape_family;        /* mi355q_shape_family */
    int32_t path;                /* mi355q_execution_path */
    uint8_t scheme_identifier;
    uint8_t layout;
    uint8_t used_fallback;
    uint8_t fallback_reason;     /* mi355q_fallback_reason */
    uint32_t input_dimension;    /* binding 3 */
    uint32_t output_dimension;   /* binding 4 */
    uint32_t sequence_length;    /* binding 5 (planned maximum) */
    uint32_t input_row_stride;   /* binding 6 */
    uint64_t weight_bytes;       /* blocks * bytesPerBlock */
    uint64_t flops;              /* 2*M*K*N */
} mi355q_step;

MI355Q_API mi355q_status mi355q_shape_family_resolve(uint32_t output_dimension,
                                                     uint32_t input_dimension,
                                                     int32_t* out_family,
                                                     uint32_t* out_simdgroups,
                                                     uint32_t* out_tile_elements,
                                                     char* out_kernel_base_name, size_t name_cap);
/* MetalDispatchStepBuilder (decode) for one LinearFragment. */
MI355Q_API mi355q_status mi355q_plan_decode_step(const mi355q_weight* w, uint32_t m,
                                                 mi355q_dtype x_dtype, uint32_t flags,
                                                 mi355q_step* out);
/* MetalPrefillStepBuilder.buildSteps(LinearFragment): writes 1 or 2 steps (dequant + GEMM when
 * the two-step path is selected).  `is_last_token` mirrors mode = .lastToken. */
MI355Q_API mi355q_status mi355q_plan_prefill_steps(const mi355q_weight* w,
                                                   uint32_t maximum_sequence_length,
                                                   uint32_t input_row_stride, mi355q_dtype x_dtype,
                                                   int is_last_token, uint32_t flags,
                                                   mi355q_step* out_steps, uint32_t* out_count);

/* ------------------------------------------------------------------------------------------
 * Dispatch plan: MetalDispatchPlan (MC/Execution/MetalDecodePlan.swift:6-140) built once at load
 * time and replayed for every token by MetalDecodeEncoder.encodeSteps
 * (MC/Execution/MetalDecodeEncoder.swift:18-36).  Steps run in order on one stream, which
 * satisfies the read/write ordering the reference enforces with barriers
 * (MC/Compiler/MetalDispatchStepBuilder.swift:276-350).  A plan borrows its weights and
 * buffers: they must outlive it.
 * ---------------------------------------------------------------------------------------- */
typedef struct mi355q_plan mi355q_plan;

MI355Q_API mi355q_status mi355q_plan_create(mi355q_context* ctx, mi355q_plan** out);
MI355Q_API mi355q_status mi355q_plan_destroy(mi355q_plan* plan);
/* One LinearFragment step (bindings as mi355q_qgemm).  layer_index and tensor_name are the
 * step metadata (MetalDispatchStepMetadata); tensor_name may be NULL. */
MI355Q_API mi355q_status mi355q_plan_add_linear(mi355q_plan* plan, const mi355q_weight* w,
                                                const void* x_dev, mi355q_dtype x_dtype,
                                                void* y_dev, mi355q_dtype y_dtype, uint32_t m,
                                                uint32_t x_row_stride, uint32_t y_row_stride,
                                                uint32_t flags, int32_t layer_index,
                                                const char* tensor_name);
/* One step for 2 or 3 projections that share their input (bindings as mi355q_batched_qgemm):
 * the decode-time counterpart of the reference's batched prefill kernels
 * (MC/Generator/MetalSourceGenerator+Quantized.swift:166-338; the entry collector that groups
 * q/k/v and gate/up is MC/Compiler/MetalEntryCollector.swift:55-95).  For M <= 8 on the
 * split-plane layout the projections run as one launch. */
MI355Q_API mi355q_status mi355q_plan_add_batched_linear(mi355q_plan* plan, uint32_t count,
                                                        const mi355q_weight* const* weights,
                                                        const void* x_dev, mi355q_dtype x_dtype,
                                                        void* const* y_devs, mi355q_dtype y_dtype,
                                                        uint32_t m, uint32_t x_row_stride,
                                                        uint32_t flags, int32_t layer_index,
                                                        const char* tensor_name);
/* One step for MLPFragment's gate_proj + up_proj + elementwise activation (bindings as mi355q_gated_qgemm;
 * MC/Compilable/MLPFragment.swift:7-14).  The step record's kernel family is gatedFused... when the activation is the
 * projection launch's epilogue, gatedBatched2... when the elementwise kernel follows the batched projection. */
MI355Q_API mi355q_status mi355q_plan_add_gated_mlp(mi355q_plan* plan, const mi355q_weight* w_gate,
                                                   const mi355q_weight* w_up, const void* x_dev,
                                                   mi355q_dtype x_dtype, void* y_dev, mi355q_dtype y_dtype,
                                                   uint32_t m, uint32_t x_row_stride, uint32_t y_row_stride,
                                                   mi355q_gated_activation activation, uint32_t flags,
                                                   int32_t layer_index, const char* tensor_name);
/* One OutputHeadFragment step (bindings as mi355q_lmhead_argmax). */
MI355Q_API mi355q_status mi355q_plan_add_output_head(mi355q_plan* plan, const mi355q_weight* w,
                                                     const void* x_dev, mi355q_dtype x_dtype,
                                                     float* logits_f32_dev, int32_t* token_out_dev,
                                                     uint32_t flags, const char* tensor_name);
MI355Q_API int32_t mi355q_plan_step_count(const mi355q_plan* plan);
/* The planned launch and its quantization-plan entry for step `index`; layer_index_out and
 * tensor_name_out (capacity name_cap) may be NULL. */
MI355Q_API mi355q_status mi355q_plan_step_at(const mi355q_plan* plan, int32_t index,
                                             mi355q_step* out, int32_t* layer_index_out,
                                             char* tensor_name_out, size_t name_cap);
/* encodeSteps: enqueue steps [first, first+count) on `stream`; count 0 means "to the end". */
MI355Q_API mi355q_status mi355q_plan_encode(mi355q_plan* plan, void* stream, uint32_t first,
                                            uint32_t count);
/* Capture the whole plan into a HIP graph once, then replay it with one launch per token. */
MI355Q_API mi355q_status mi355q_plan_graph_build(mi355q_plan* plan, void* stream);
MI355Q_API mi355q_status mi355q_plan_graph_launch(mi355q_plan* plan, void* stream);

/* Device-to-device copy kernel (prompt-state snapshots copy runtime buffers,
 * MC/Execution/MetalPromptState.swift:3-19; also the known-size copy that calibrates the HBM
 * traffic counters).  Both pointers 16-byte aligned, bytes a multiple of 16. */
MI355Q_API mi355q_status mi355q_buffer_copy(mi355q_context* ctx, void* stream, void* dst_dev,
                                            const void* src_dev, size_t bytes);

/* ------------------------------------------------------------------------------------------
 * STAF container (model.staf): reader, validator, writer
 * ---------------------------------------------------------------------------------------- */
/* STAFLoader.load (MC/STAF/STAFLoader.swift:19-198): maps the file read-only and parses header, section
 * table, string table and metadata table (MC/STAF/STAFFormat.swift:10-80, 84-167).  Rejects what the
 * reference rejects (missing or <= 64-byte file, bad magic, a format version other than 0 or 2, a payload
 * that leaves the file, malformed metadata, no tensors) with MI355Q_ERR_INVALID_FILE, and also tables
 * that leave the file, which the reference reads unchecked. */
typedef struct mi355q_staf mi355q_staf;
/* STAFSectionEntry / STAFTensorEntry (STAFFormat.swift:132-167, STAFLoader.swift:299-311).  `name` points
 * into the mapping: name_length bytes of UTF-8, valid until mi355q_staf_close. */
typedef struct mi355q_staf_entry {
    const char* name;
    uint32_t name_length;
    uint8_t scheme_identifier, semantic_role, original_dtype, dimension_count;
    uint32_t shape[8];
    uint64_t payload_offset;   /* from the start of the file */
    uint64_t payload_size;
    uint64_t buffer_offset;    /* STAFTensorEntry.bufferOffset: from the start of the payload region */
    uint32_t alignment, block_size, group_size, checksum, shard_index;
} mi355q_staf_entry;
/* STAFMetadataValueType (MC/STAF/STAFMetadataValue.swift:12-19) */
enum { MI355Q_STAF_BOOL = 1, MI355Q_STAF_UINT32 = 2, MI355Q_STAF_UINT64 = 3, MI355Q_STAF_FLOAT32 = 4,
       MI355Q_STAF_FLOAT64 = 5, MI355Q_STAF_STRING = 6 };
/* One file-level metadata value (STAFMetadataValue).  payload0 holds the bool, the integer or the bit
 * pattern of the float; strings are text[0, text_length). */
typedef struct mi355q_staf_metadata {
    const char* key;
    uint8_t type;
    uint64_t payload0;
    const char* text;
    uint32_t text_length;
} mi355q_staf_metadata;
/* One tensor handed to the writer (STAFConversionEntry + its converted payload). */
typedef struct mi355q_staf_tensor {
    const char* name;
    uint8_t scheme_identifier, semantic_role, original_dtype;
    uint32_t dimension_count;
    uint32_t shape[8];         /* packed tensors: the MLX shape [N, K*bits/32] */
    const void* payload;
    uint64_t payload_size;
    uint32_t shard_index;
} mi355q_staf_tensor;

MI355Q_API mi355q_status mi355q_staf_open(const char* path, mi355q_staf** out);
MI355Q_API void mi355q_staf_close(mi355q_staf* staf);
MI355Q_API uint32_t mi355q_staf_format_version(const mi355q_staf* staf);
MI355Q_API uint32_t mi355q_staf_tensor_count(const mi355q_staf* staf);
MI355Q_API mi355q_status mi355q_staf_tensor_at(const mi355q_staf* staf, uint32_t index, mi355q_staf_entry* out);
/* STAFWeightStore.entries[name]; MI355Q_ERR_NOT_FOUND when absent. */
MI355Q_API mi355q_status mi355q_staf_find(const mi355q_staf* staf, const char* name, mi355q_staf_entry* out);
/* The payload region in host memory: first tensor to end of file, the span of the single MTLBuffer
 * (STAFLoader.swift:160-197). */
MI355Q_API const void* mi355q_staf_payload_region(const mi355q_staf* staf, uint64_t* bytes);
MI355Q_API uint32_t mi355q_staf_metadata_count(const mi355q_staf* staf);
MI355Q_API mi355q_status mi355q_staf_metadata_at(const mi355q_staf* staf, uint32_t index,
                                                 mi355q_staf_metadata* out);
/* STAFValidator.isValid (MC/STAF/STAFValidator.swift:5-78): format version 2, section table right after
 * the header, metadata table in bounds, every expected value present and equal, no source file newer than
 * the container.  *valid = 1 or 0; an unreadable path is MI355Q_ERR_IO (the reference throws). */
MI355Q_API mi355q_status mi355q_staf_is_valid(const char* staf_path, const char* const* source_paths,
                                              uint32_t source_count, const mi355q_staf_metadata* expected,
                                              uint32_t expected_count, int32_t* valid);
/* STAFWriter.write (MC/STAF/STAFWriter.swift:11-269) for payloads that are already converted: header,
 * section table, metadata table sorted by key, de-duplicated string table, payload region from the next
 * 4096-byte boundary with every tensor on a 256-byte one.  A payload whose size is not what its shape and
 * scheme imply (computePayloadSize, :240-262) is MI355Q_ERR_SIZE_MISMATCH. */
MI355Q_API mi355q_status mi355q_staf_write(const char* path, const mi355q_staf_tensor* tensors,
                                           uint32_t tensor_count, const mi355q_staf_metadata* metadata,
                                           uint32_t metadata_count);
/* The single device buffer of STAFWeightStore: copies the payload region to device memory (one
 * allocation, released with mi355q_buffer_free).  Tensor `t` then lives at *base_dev_out + t.buffer_offset. */
MI355Q_API mi355q_status mi355q_staf_upload(mi355q_context* ctx, const mi355q_staf* staf, void** base_dev_out,
                                            uint64_t* bytes_out);
/* resolvedBufferAccess for one packed 2-D tensor (STAFLoader.swift:213-299): MI355Q_LAYOUT_STAF_BLOCKS
 * borrows the bytes inside the uploaded region (zero copy); MI355Q_LAYOUT_PLANES / _TILE16 build this
 * library's specialized copy from the mapping, as STAFSpecializedWeightStoreBuilder does
 * (MC/STAF/STAFSpecializedWeightStoreBuilder.swift:15-31).  N = shape[0], K = shape[1] * 32 / bits. */
MI355Q_API mi355q_status mi355q_staf_weight(mi355q_context* ctx, const mi355q_staf* staf, const void* base_dev,
                                            const char* name, mi355q_layout layout, mi355q_weight** out);

/* ------------------------------------------------------------------------------------------
 * Quantized KV cache (the step on the other side of the attention projections)
 * ---------------------------------------------------------------------------------------- */
/* QuantizationSchemeIdentifier.isSupportedForKVCache (MC/STAF/STAFFormat.swift:239-262) for the schemes this
 * library writes and reads: dense 0x00 / 0x01 / 0x02, 8-bit 0x10-0x12, 4-bit 0x40-0x42.  The rotor schemes
 * (0x70, 0x71) need the Clifford pre-rotation, which is outside this path: 0. */
MI355Q_API int32_t mi355q_kv_scheme_is_supported(uint8_t scheme_identifier);
/* KVCacheSpecification.bytesPerHeadSlot (MC/Buffer/MetalGraphAllocator.swift:60-114): ceil(headDim /
 * weightsPerBlock) blocks rounded up to 64 bytes (packed) or 256 bytes (dense); every registered format is
 * sizable, also those without kernels; rotor schemes size as their base scheme; 0 = no registered format. */
MI355Q_API uint32_t mi355q_kv_bytes_per_head_slot(uint8_t scheme_identifier, uint32_t head_dimension);
/* The uniforms of the cache kernels (kvHeadCount, headDimension, maxSequenceLength, layoutMode, k/vQuantScheme,
 * k/vHeadSlotBytes; MC/Generator/MetalSourceGenerator+Attention.swift:1199-1216).  layout_mode 0 =
 * [head][position] (sequence-major), 1 = [position][head] (head-major); one layer's K or V buffer. */
typedef struct mi355q_kv_layout {
    uint8_t scheme;
    uint8_t layout_mode;
    uint16_t reserved0;
    uint32_t kv_head_count, head_dimension, maximum_sequence_length, head_slot_bytes;
} mi355q_kv_layout;
/* write_kv_quantized / write_kv_element_dense for positions [first_position, +sequence_length) of every head
 * (:2057-2180, :1958-1971; addressing :762-769): src is [sequence_length, input_row_stride] with head h at
 * columns [h * headDim, +headDim) (0 = dense rows).  Per group: scale = (max - min) / levels (at least 1e-10),
 * header f16(scale), f16(min), codes round((v - min) / scale) clamped. */
MI355Q_API mi355q_status mi355q_kv_cache_write(mi355q_context* ctx, void* stream, const mi355q_kv_layout* layout,
                                               void* cache_dev, const void* src_dev, mi355q_dtype src_dtype,
                                               uint32_t input_row_stride, uint32_t first_position,
                                               uint32_t sequence_length);
/* read_kv_element (:1923-1956) over whole slots: out is [sequence_length, out_row_stride] in out_dtype. */
MI355Q_API mi355q_status mi355q_kv_cache_read(mi355q_context* ctx, void* stream, const mi355q_kv_layout* layout,
                                              const void* cache_dev, void* out_dev, mi355q_dtype out_dtype,
                                              uint32_t out_row_stride, uint32_t first_position,
                                              uint32_t sequence_length);

#ifdef __cplusplus
}
#endif
#endif /* MI355_QLINEAR_H */
