// Format registry: the QuantizationFormat descriptors of the affine block formats
// (reference: Sources/MetalCompiler/STAF/QuantizationFormat.swift:463-1036 for the structs,
// :1284-1335 for the two lookup functions; scheme ids Sources/MetalCompiler/STAF/STAFFormat.swift:175-217).
#include <mutex>
#include <vector>

#include "common.h"

namespace mi355q {
namespace {

struct Row {
    uint8_t scheme;
    int bits, group;
    bool direct_gemm;   // Q4G64 / Q4G128 / Q8G32 / Q8G64 declare a direct GEMM kernel
    bool batched;       // Q4G64 / Q4G128 declare batched direct kernels (count 2 and 3)
    bool in_reference;
};

// (bits, group) pairs as registered by formatForMLXQuantization; 0x22 and 0x62 are additions
// of this library (next free id of their family; ids are append-only).
const Row kRows[] = {
    {0x60, 2, 16, false, false, true},  {0x61, 2, 32, false, false, true},
    {0x62, 2, 64, false, false, false}, {0x50, 3, 16, false, false, true},
    {0x51, 3, 32, false, false, true},  {0x52, 3, 64, false, false, true},
    {0x40, 4, 64, true, true, true},    {0x41, 4, 128, true, true, true},
    {0x30, 5, 32, false, false, true},  {0x31, 5, 64, false, false, true},
    {0x20, 6, 16, false, false, true},  {0x21, 6, 32, false, false, true},
    {0x22, 6, 64, false, false, false}, {0x10, 8, 32, true, false, true},
    {0x11, 8, 64, true, false, true},   {0x12, 8, 128, false, false, true},
};

std::vector<mi355q_format> build_table() {
    std::vector<mi355q_format> t;
    for (const Row& r : kRows) {
        mi355q_format f;
        std::memset(&f, 0, sizeof f);
        f.scheme_identifier = r.scheme;
        f.bits = (uint8_t)r.bits;
        f.is_quantized = 1;
        f.is_aligned = (r.bits == 2 || r.bits == 4 || r.bits == 8) ? 1 : 0;
        f.group_size = (uint32_t)r.group;
        f.weights_per_block = (uint32_t)r.group;
        f.bytes_per_block = (uint32_t)(4 + r.group * r.bits / 8);
        f.has_direct_gemm = r.direct_gemm ? 1 : 0;
        f.batched_gemm_counts = r.batched ? (uint8_t)((1u << 2) | (1u << 3)) : 0;
        f.in_reference_registry = r.in_reference ? 1 : 0;
        // max(groupSize*2, 256) * sizeof(float)
        f.direct_gemm_threadgroup_memory_length =
            r.direct_gemm ? (uint32_t)((r.group * 2 > 256 ? r.group * 2 : 256) * 4) : 0;
        std::snprintf(f.block_struct_name, sizeof f.block_struct_name, "BlockQ%dAffine%d", r.bits,
                      r.group);
        std::snprintf(f.gemv_kernel_name, sizeof f.gemv_kernel_name, "gemv_q%d_g%d", r.bits,
                      r.group);
        std::snprintf(f.gemm_kernel_name_f32s, sizeof f.gemm_kernel_name_f32s,
                      "gemm_q%d_g%d_f32s", r.bits, r.group);
        std::snprintf(f.gemm_kernel_name, sizeof f.gemm_kernel_name, "gemm_q%d_g%d", r.bits,
                      r.group);
        std::snprintf(f.dequant_to_bfloat_kernel_name, sizeof f.dequant_to_bfloat_kernel_name,
                      "dequant_q%d_g%d_bf16", r.bits, r.group);
        std::snprintf(f.embedding_lookup_token, sizeof f.embedding_lookup_token, "q%d_g%d", r.bits,
                      r.group);
        t.push_back(f);
    }
    return t;
}

const std::vector<mi355q_format>& table() {
    static const std::vector<mi355q_format> t = build_table();
    return t;
}

}  // namespace

const mi355q_format* find_format_mlx(int bits, int group) {
    for (const auto& f : table())
        if (f.bits == bits && (int)f.group_size == group) return &f;
    return nullptr;
}

const mi355q_format* find_format_scheme(uint8_t scheme) {
    if (scheme == 0x42) scheme = 0x41;  // q4Group128ScaleF16Zero shares the q4g128 block layout
    for (const auto& f : table())
        if (f.scheme_identifier == scheme) return &f;
    return nullptr;
}

int format_count() { return (int)table().size(); }
const mi355q_format* format_at(int i) {
    return (i >= 0 && i < format_count()) ? &table()[(size_t)i] : nullptr;
}

// ---- error plumbing ------------------------------------------------------------------------
namespace {
thread_local std::string g_last_error;
}

void set_error(const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
}

mi355q_status fail(mi355q_status code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

const char* last_error_cstr();
const char* last_error_cstr() { return g_last_error.c_str(); }

}  // namespace mi355q

extern "C" {

const char* mi355q_last_error(void) { return mi355q::last_error_cstr(); }
int32_t mi355q_abi_version(void) { return MI355Q_ABI_VERSION; }

mi355q_status mi355q_format_for_mlx_quantization(int bits, int group_size, mi355q_format* out) {
    if (!out) return mi355q::fail(MI355Q_ERR_INVALID_ARGUMENT, "format out pointer is null");
    const mi355q_format* f = mi355q::find_format_mlx(bits, group_size);
    if (!f)
        return mi355q::fail(MI355Q_ERR_UNSUPPORTED_FORMAT,
                            "unsupported quantization: bits=%d group_size=%d", bits, group_size);
    *out = *f;
    return MI355Q_OK;
}

mi355q_status mi355q_format_for_scheme(uint8_t scheme_identifier, mi355q_format* out) {
    if (!out) return mi355q::fail(MI355Q_ERR_INVALID_ARGUMENT, "format out pointer is null");
    const mi355q_format* f = mi355q::find_format_scheme(scheme_identifier);
    if (!f)
        return mi355q::fail(MI355Q_ERR_UNSUPPORTED_FORMAT,
                            "scheme 0x%02x is not an affine block format of this path",
                            scheme_identifier);
    *out = *f;
    return MI355Q_OK;
}

int32_t mi355q_format_count(void) { return mi355q::format_count(); }

mi355q_status mi355q_format_at(int32_t index, mi355q_format* out) {
    const mi355q_format* f = mi355q::format_at(index);
    if (!f || !out) return mi355q::fail(MI355Q_ERR_INVALID_ARGUMENT, "format index out of range");
    *out = *f;
    return MI355Q_OK;
}

uint16_t mi355q_bf16_from_f32(float value) {
    uint32_t bits;
    std::memcpy(&bits, &value, 4);
    uint32_t lsb = (bits >> 16) & 1u;
    return (uint16_t)((bits + 0x7FFFu + lsb) >> 16);
}

}  // extern "C"
