// The STAF on-disk container: reader, validator and writer (host side).
//
// Layout (packed, little-endian; Sources/MetalCompiler/STAF/STAFFormat.swift:10-80, 84-167):
//   header, 64 bytes:   0 magic "STAF" | 4 formatVersion | 8 metadataEntryCount | 12 metadataTableOffset |
//                       40 sectionCount | 44 sectionTableOffset | 48 stringTableOffset | 52 stringTableSize
//   section entry, 128: 0 nameOffset | 4 nameLength | 8 scheme | 9 role | 10 original dtype | 11 ndim |
//                       12 shape[8] | 44 payloadOffset u64 | 52 payloadSize u64 | 60 alignment | 64 blockSize |
//                       68 groupSize | 72 checksum | 76 shardIndex | 80 reserved[48]
//   metadata entry, 32: 0 keyOffset | 4 keyLength | 8 valueType u8 | 12 payload0 u64 | 20 payload1 u64
//   string table, then the payload region from the next 4096-byte boundary, every tensor at a 256-byte one.
// The reader follows STAFLoader.load (STAFLoader.swift:19-198) and STAFMetadataDecoder, the validator
// STAFValidator.isValid (STAFValidator.swift:5-78), the writer STAFWriter.write (STAFWriter.swift:11-269).
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cstdio>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "common.h"

using mi355q::fail;

namespace {

constexpr uint32_t kMagic = 0x46415453u;          // "STAF"
constexpr uint32_t kCurrentFormatVersion = 2, kLegacyFormatVersion = 0;
constexpr size_t kHeaderSize = 64, kSectionEntrySize = 128, kMetadataEntrySize = 32;
constexpr size_t kPayloadAlignment = 4096, kTensorAlignment = 256;

template <typename T>
T load(const uint8_t* p) {
    T v;
    std::memcpy(&v, p, sizeof v);
    return v;
}
template <typename T>
void store(uint8_t* p, T v) { std::memcpy(p, &v, sizeof v); }

size_t align_up(size_t v, size_t a) { return v % a ? v + (a - v % a) : v; }

struct Header {
    uint32_t magic, format_version, metadata_count, metadata_offset, section_count, section_offset, string_offset,
        string_size;
    bool supports_metadata() const {        // STAFHeader.supportsMetadataTable (STAFFormat.swift:122-128)
        return format_version >= kCurrentFormatVersion && metadata_count > 0 && metadata_offset > 0;
    }
};
Header parse_header(const uint8_t* p) {
    return Header{load<uint32_t>(p + 0),  load<uint32_t>(p + 4),  load<uint32_t>(p + 8),  load<uint32_t>(p + 12),
                  load<uint32_t>(p + 40), load<uint32_t>(p + 44), load<uint32_t>(p + 48), load<uint32_t>(p + 52)};
}

struct Metadata {
    std::string key;
    uint8_t type;
    uint64_t payload0, payload1;
    std::string text;     // string values
};

// STAFMetadataDecoder.decode (STAFMetadataDecoder.swift:31-145).  Returns an empty message on success.
std::string decode_metadata(const uint8_t* file, size_t file_size, const Header& h, std::vector<Metadata>* out) {
    out->clear();
    if (!h.supports_metadata()) return "";
    const size_t table = h.metadata_offset, bytes = (size_t)h.metadata_count * kMetadataEntrySize;
    if (table < kHeaderSize || table + bytes > file_size) return "Metadata table is out of bounds";
    if ((size_t)h.string_offset + h.string_size > file_size) return "String table is out of bounds";
    auto text = [&](uint64_t off, uint64_t len, std::string* s) {
        if (off + len > h.string_size || off + len < off) return false;
        s->assign((const char*)file + h.string_offset + off, (size_t)len);
        return true;
    };
    std::map<std::string, size_t> seen;    // a repeated key keeps its last value, as the dictionary does
    for (uint32_t i = 0; i < h.metadata_count; i++) {
        const uint8_t* e = file + table + (size_t)i * kMetadataEntrySize;
        Metadata m;
        m.type = e[8];
        m.payload0 = load<uint64_t>(e + 12);
        m.payload1 = load<uint64_t>(e + 20);
        if (m.type < 1 || m.type > 6) return "Unknown metadata value type: " + std::to_string(m.type);
        if (!text(load<uint32_t>(e + 0), load<uint32_t>(e + 4), &m.key)) return "Metadata string is out of bounds";
        if (m.type == MI355Q_STAF_STRING && !text(m.payload0, m.payload1, &m.text))
            return "Metadata string is out of bounds";
        auto it = seen.find(m.key);
        if (it != seen.end()) (*out)[it->second] = m;
        else { seen[m.key] = out->size(); out->push_back(m); }
    }
    return "";
}

// STAFMetadataValue's synthesized == per case
bool metadata_equal(const Metadata& a, uint8_t type, uint64_t payload0, const char* text, size_t text_len) {
    if (a.type != type) return false;
    switch (type) {
    case MI355Q_STAF_BOOL: return (a.payload0 != 0) == (payload0 != 0);
    case MI355Q_STAF_UINT32: return (uint32_t)a.payload0 == (uint32_t)payload0;
    case MI355Q_STAF_UINT64: return a.payload0 == payload0;
    case MI355Q_STAF_FLOAT32: {
        float x, y;
        const uint32_t bx = (uint32_t)a.payload0, by = (uint32_t)payload0;
        std::memcpy(&x, &bx, 4); std::memcpy(&y, &by, 4);
        return x == y;
    }
    case MI355Q_STAF_FLOAT64: {
        double x, y;
        std::memcpy(&x, &a.payload0, 8); std::memcpy(&y, &payload0, 8);
        return x == y;
    }
    case MI355Q_STAF_STRING: return a.text.size() == text_len && std::memcmp(a.text.data(), text, text_len) == 0;
    default: return false;
    }
}

// STAFWriter.computePayloadSize (STAFWriter.swift:240-262); 0 with *known = false when the scheme has no formula
size_t payload_size_for(uint8_t scheme, const uint32_t* shape, uint32_t ndim, bool* quantized) {
    size_t elements = 1;
    for (uint32_t d = 0; d < ndim; d++) elements *= shape[d];
    *quantized = false;
    if (scheme == 0x02) return elements * 4;                       // fp32RowMajor
    mi355q_format f;
    if (scheme <= 0x01 || scheme == 0xFF || mi355q_format_for_scheme(scheme, &f) != MI355Q_OK)
        return elements * 2;                                       // fp16 / bf16 / passthrough / unregistered
    *quantized = true;
    const size_t n = ndim >= 1 ? shape[0] : 1, packed = ndim >= 2 ? shape[1] : 1;
    const size_t k = packed * 32 / f.bits;                         // must match repackMLXQuantized
    return n * (k / f.group_size) * f.bytes_per_block;
}

}  // namespace

struct mi355q_staf {
    uint8_t* base = nullptr;       // mmap of the whole file, read-only
    size_t size = 0;
    Header header{};
    std::vector<mi355q_staf_entry> entries;
    std::map<std::string, uint32_t> by_name;
    std::vector<Metadata> metadata;
    uint64_t first_payload_offset = 0;
};

extern "C" {

mi355q_status mi355q_staf_open(const char* path, mi355q_staf** out) {
    if (!path || !out) return fail(MI355Q_ERR_INVALID_ARGUMENT, "path and out must not be null");
    *out = nullptr;
    struct stat st;
    if (::stat(path, &st) != 0) return fail(MI355Q_ERR_INVALID_FILE, "File too small or missing: %s", path);
    if ((size_t)st.st_size <= kHeaderSize) return fail(MI355Q_ERR_INVALID_FILE, "File too small or missing: %s", path);
    const int fd = ::open(path, O_RDONLY);
    if (fd < 0) return fail(MI355Q_ERR_INVALID_FILE, "Cannot open: %s", path);
    void* map = ::mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    ::close(fd);
    if (map == MAP_FAILED) return fail(MI355Q_ERR_IO, "mmap failed for: %s", path);
    mi355q_staf* s = new mi355q_staf;
    s->base = (uint8_t*)map;
    s->size = (size_t)st.st_size;
    auto reject = [&](mi355q_status code, const std::string& msg) {
        ::munmap(s->base, s->size);
        delete s;
        return fail(code, "%s", msg.c_str());
    };
    s->header = parse_header(s->base);
    const Header& h = s->header;
    if (h.magic != kMagic) return reject(MI355Q_ERR_INVALID_FILE, "Bad magic: expected STAF");
    if (h.format_version != kLegacyFormatVersion && h.format_version != kCurrentFormatVersion)
        return reject(MI355Q_ERR_INVALID_FILE, "Unsupported STAF format version: " + std::to_string(h.format_version));
    const std::string merr = decode_metadata(s->base, s->size, h, &s->metadata);
    if (!merr.empty()) return reject(MI355Q_ERR_INVALID_FILE, merr);
    // The reference reads the tables unchecked; here a table that leaves the file is an invalid file.
    if ((size_t)h.section_offset + (size_t)h.section_count * kSectionEntrySize > s->size)
        return reject(MI355Q_ERR_INVALID_FILE, "Section table is out of bounds");
    if ((size_t)h.string_offset + h.string_size > s->size)
        return reject(MI355Q_ERR_INVALID_FILE, "String table is out of bounds");
    s->entries.resize(h.section_count);
    uint64_t first = UINT64_MAX;
    for (uint32_t i = 0; i < h.section_count; i++) {
        const uint8_t* e = s->base + h.section_offset + (size_t)i * kSectionEntrySize;
        mi355q_staf_entry& t = s->entries[i];
        std::memset(&t, 0, sizeof t);
        const uint32_t name_offset = load<uint32_t>(e + 0);
        t.name_length = load<uint32_t>(e + 4);
        t.scheme_identifier = e[8];
        t.semantic_role = e[9];
        t.original_dtype = e[10];
        t.dimension_count = e[11] < 8 ? e[11] : 8;
        for (uint32_t d = 0; d < t.dimension_count; d++) t.shape[d] = load<uint32_t>(e + 12 + 4 * d);
        t.payload_offset = load<uint64_t>(e + 44);
        t.payload_size = load<uint64_t>(e + 52);
        t.alignment = load<uint32_t>(e + 60);
        t.block_size = load<uint32_t>(e + 64);
        t.group_size = load<uint32_t>(e + 68);
        t.checksum = load<uint32_t>(e + 72);
        t.shard_index = load<uint32_t>(e + 76);
        if (t.payload_offset > s->size || t.payload_size > s->size || t.payload_offset + t.payload_size > s->size)
            return reject(MI355Q_ERR_INVALID_FILE,
                          "Payload overflow in section " + std::to_string(i) + "/" + std::to_string(h.section_count) +
                              ": fileSize=" + std::to_string(s->size) + ", payloadOffset=" +
                              std::to_string(t.payload_offset) + ", payloadSize=" + std::to_string(t.payload_size));
        if ((uint64_t)name_offset + t.name_length > h.string_size)
            return reject(MI355Q_ERR_INVALID_FILE, "Tensor name of section " + std::to_string(i) + " is out of bounds");
        t.name = (const char*)s->base + h.string_offset + name_offset;
        s->by_name[std::string(t.name, t.name_length)] = i;       // a repeated name resolves to its last entry
        first = std::min(first, t.payload_offset);
    }
    if (s->entries.empty()) return reject(MI355Q_ERR_INVALID_FILE, "No tensors in STAF");
    s->first_payload_offset = first;
    for (auto& t : s->entries) t.buffer_offset = t.payload_offset - first;     // STAFTensorEntry.bufferOffset
    *out = s;
    return MI355Q_OK;
}

void mi355q_staf_close(mi355q_staf* s) {
    if (!s) return;
    if (s->base) ::munmap(s->base, s->size);
    delete s;
}

uint32_t mi355q_staf_format_version(const mi355q_staf* s) { return s ? s->header.format_version : 0; }
uint32_t mi355q_staf_tensor_count(const mi355q_staf* s) { return s ? (uint32_t)s->entries.size() : 0; }

mi355q_status mi355q_staf_tensor_at(const mi355q_staf* s, uint32_t index, mi355q_staf_entry* out) {
    if (!s || !out) return fail(MI355Q_ERR_NULL_HANDLE, "null container or output");
    if (index >= s->entries.size()) return fail(MI355Q_ERR_INVALID_ARGUMENT, "tensor index %u out of range", index);
    *out = s->entries[index];
    return MI355Q_OK;
}

mi355q_status mi355q_staf_find(const mi355q_staf* s, const char* name, mi355q_staf_entry* out) {
    if (!s || !name || !out) return fail(MI355Q_ERR_NULL_HANDLE, "null container, name or output");
    const auto it = s->by_name.find(name);
    if (it == s->by_name.end()) return fail(MI355Q_ERR_NOT_FOUND, "no tensor named '%s'", name);
    *out = s->entries[it->second];
    return MI355Q_OK;
}

const void* mi355q_staf_payload_region(const mi355q_staf* s, uint64_t* bytes) {
    if (!s) return nullptr;
    if (bytes) *bytes = s->size - s->first_payload_offset;
    return s->base + s->first_payload_offset;
}

uint32_t mi355q_staf_metadata_count(const mi355q_staf* s) { return s ? (uint32_t)s->metadata.size() : 0; }

mi355q_status mi355q_staf_metadata_at(const mi355q_staf* s, uint32_t index, mi355q_staf_metadata* out) {
    if (!s || !out) return fail(MI355Q_ERR_NULL_HANDLE, "null container or output");
    if (index >= s->metadata.size()) return fail(MI355Q_ERR_INVALID_ARGUMENT, "metadata index %u out of range", index);
    const Metadata& m = s->metadata[index];
    out->key = m.key.c_str();
    out->type = m.type;
    out->payload0 = m.payload0;
    out->text = m.type == MI355Q_STAF_STRING ? m.text.data() : nullptr;
    out->text_length = m.type == MI355Q_STAF_STRING ? (uint32_t)m.text.size() : 0;
    return MI355Q_OK;
}

mi355q_status mi355q_staf_is_valid(const char* staf_path, const char* const* source_paths, uint32_t source_count,
                                   const mi355q_staf_metadata* expected, uint32_t expected_count, int32_t* valid) {
    if (!staf_path || !valid || (source_count && !source_paths) || (expected_count && !expected))
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "null argument");
    *valid = 0;
    struct stat st;
    if (::stat(staf_path, &st) != 0) return fail(MI355Q_ERR_IO, "cannot read %s: %s", staf_path, std::strerror(errno));
    const size_t size = (size_t)st.st_size;
    if (size < kHeaderSize) return MI355Q_OK;
    const int fd = ::open(staf_path, O_RDONLY);
    if (fd < 0) return fail(MI355Q_ERR_IO, "cannot open %s: %s", staf_path, std::strerror(errno));
    void* map = ::mmap(nullptr, size, PROT_READ, MAP_PRIVATE, fd, 0);
    ::close(fd);
    if (map == MAP_FAILED) return fail(MI355Q_ERR_IO, "mmap failed for: %s", staf_path);
    const uint8_t* file = (const uint8_t*)map;
    const Header h = parse_header(file);
    bool ok = h.magic == kMagic && h.section_count > 0 && h.format_version == kCurrentFormatVersion &&
              h.section_offset == kHeaderSize;
    if (ok && h.supports_metadata()) {
        const size_t minimum = kHeaderSize + (size_t)h.section_count * kSectionEntrySize;
        ok = h.metadata_offset >= minimum && (size_t)h.metadata_offset + (size_t)h.metadata_count * kMetadataEntrySize <= size;
    }
    if (ok && size > kHeaderSize + kSectionEntrySize)          // the first section's payload must fit the file
        ok = load<uint64_t>(file + kHeaderSize + 52) <= size;
    if (ok && expected_count) {
        std::vector<Metadata> actual;
        ok = decode_metadata(file, size, h, &actual).empty();
        for (uint32_t i = 0; ok && i < expected_count; i++) {
            const mi355q_staf_metadata& want = expected[i];
            bool found = false;
            for (const Metadata& m : actual)
                if (want.key && m.key == want.key)
                    found = metadata_equal(m, want.type, want.payload0, want.text ? want.text : "", want.text_length);
            ok = found;
        }
    }
    ::munmap(map, size);
    if (!ok) return MI355Q_OK;
    for (uint32_t i = 0; i < source_count; i++) {              // a source newer than the cache invalidates it
        struct stat src;
        if (::stat(source_paths[i], &src) != 0)                // follows symbolic links, as resolvingSymlinksInPath
            return fail(MI355Q_ERR_IO, "cannot read %s: %s", source_paths[i], std::strerror(errno));
        if (src.st_mtim.tv_sec > st.st_mtim.tv_sec ||
            (src.st_mtim.tv_sec == st.st_mtim.tv_sec && src.st_mtim.tv_nsec > st.st_mtim.tv_nsec))
            return MI355Q_OK;
    }
    *valid = 1;
    return MI355Q_OK;
}

mi355q_status mi355q_staf_write(const char* path, const mi355q_staf_tensor* tensors, uint32_t tensor_count,
                                const mi355q_staf_metadata* metadata, uint32_t metadata_count) {
    if (!path || (tensor_count && !tensors) || (metadata_count && !metadata))
        return fail(MI355Q_ERR_INVALID_ARGUMENT, "null argument");
    std::vector<uint8_t> strings;
    std::map<std::string, uint32_t> offsets;
    auto append = [&](const std::string& s) {                 // one copy per distinct string, NUL-terminated
        const auto it = offsets.find(s);
        if (it != offsets.end()) return it->second;
        const uint32_t off = (uint32_t)strings.size();
        strings.insert(strings.end(), s.begin(), s.end());
        strings.push_back(0);
        offsets[s] = off;
        return off;
    };
    std::vector<uint32_t> name_offsets(tensor_count);
    for (uint32_t i = 0; i < tensor_count; i++) {
        const mi355q_staf_tensor& t = tensors[i];
        if (!t.name || (t.payload_size && !t.payload) || t.dimension_count > 8)
            return fail(MI355Q_ERR_INVALID_ARGUMENT, "tensor %u: null name or payload, or more than 8 dimensions", i);
        bool quantized;
        const size_t want = payload_size_for(t.scheme_identifier, t.shape, t.dimension_count, &quantized);
        if (want != t.payload_size)
            return fail(MI355Q_ERR_SIZE_MISMATCH, "tensor '%s': payload is %llu bytes, its shape and scheme 0x%02X need %zu",
                        t.name, (unsigned long long)t.payload_size, (unsigned)t.scheme_identifier, want);
        name_offsets[i] = append(t.name);
    }
    std::vector<uint32_t> order(metadata_count);
    for (uint32_t i = 0; i < metadata_count; i++) {
        if (!metadata[i].key || metadata[i].type < 1 || metadata[i].type > 6 ||
            (metadata[i].type == MI355Q_STAF_STRING && metadata[i].text_length && !metadata[i].text))
            return fail(MI355Q_ERR_INVALID_ARGUMENT, "metadata %u: null key, unknown type or null string", i);
        order[i] = i;
    }
    std::stable_sort(order.begin(), order.end(),
                     [&](uint32_t a, uint32_t b) { return std::strcmp(metadata[a].key, metadata[b].key) < 0; });
    const size_t section_offset = kHeaderSize, metadata_offset = section_offset + (size_t)tensor_count * kSectionEntrySize;
    std::vector<uint8_t> table((size_t)metadata_count * kMetadataEntrySize, 0);
    for (uint32_t j = 0; j < metadata_count; j++) {
        const mi355q_staf_metadata& m = metadata[order[j]];
        uint8_t* e = table.data() + (size_t)j * kMetadataEntrySize;
        store<uint32_t>(e + 0, append(m.key));
        store<uint32_t>(e + 4, (uint32_t)std::strlen(m.key));
        e[8] = m.type;
        uint64_t p0 = m.payload0, p1 = 0;
        if (m.type == MI355Q_STAF_BOOL) p0 = m.payload0 ? 1 : 0;
        else if (m.type == MI355Q_STAF_UINT32 || m.type == MI355Q_STAF_FLOAT32) p0 = (uint32_t)m.payload0;
        else if (m.type == MI355Q_STAF_STRING) {
            p0 = append(std::string(m.text ? m.text : "", m.text_length));
            p1 = m.text_length;
        }
        store<uint64_t>(e + 12, p0);
        store<uint64_t>(e + 20, p1);
    }
    const size_t string_offset = metadata_offset + table.size();
    const size_t payload_start = align_up(string_offset + strings.size(), kPayloadAlignment);
    std::vector<uint64_t> payload_offsets(tensor_count);
    size_t cursor = payload_start;
    for (uint32_t i = 0; i < tensor_count; i++) {
        payload_offsets[i] = align_up(cursor, kTensorAlignment);
        cursor = payload_offsets[i] + tensors[i].payload_size;
    }
    if (string_offset + strings.size() > UINT32_MAX) return fail(MI355Q_ERR_INVALID_ARGUMENT, "tables exceed 4 GiB");

    std::vector<uint8_t> head(payload_start, 0);
    uint8_t* h = head.data();
    store<uint32_t>(h + 0, kMagic);
    store<uint32_t>(h + 4, kCurrentFormatVersion);
    store<uint32_t>(h + 8, metadata_count);
    store<uint32_t>(h + 12, (uint32_t)metadata_offset);
    store<uint32_t>(h + 40, tensor_count);
    store<uint32_t>(h + 44, (uint32_t)section_offset);
    store<uint32_t>(h + 48, (uint32_t)string_offset);
    store<uint32_t>(h + 52, (uint32_t)strings.size());
    for (uint32_t i = 0; i < tensor_count; i++) {
        const mi355q_staf_tensor& t = tensors[i];
        uint8_t* e = h + section_offset + (size_t)i * kSectionEntrySize;
        store<uint32_t>(e + 0, name_offsets[i]);
        store<uint32_t>(e + 4, (uint32_t)std::strlen(t.name));
        e[8] = t.scheme_identifier; e[9] = t.semantic_role; e[10] = t.original_dtype; e[11] = (uint8_t)t.dimension_count;
        for (uint32_t d = 0; d < 8; d++) store<uint32_t>(e + 12 + 4 * d, d < t.dimension_count ? t.shape[d] : 0);
        store<uint64_t>(e + 44, payload_offsets[i]);
        store<uint64_t>(e + 52, t.payload_size);
        store<uint32_t>(e + 60, (uint32_t)kTensorAlignment);
        // weightsPerBlock and groupSize of the registered format, 1 and 1 without one (dense formats are 1 / 1)
        mi355q_format f;
        const bool packed = t.scheme_identifier >= 0x10 && t.scheme_identifier != 0xFF &&
                            mi355q_format_for_scheme(t.scheme_identifier, &f) == MI355Q_OK;
        store<uint32_t>(e + 64, packed ? f.group_size : 1);
        store<uint32_t>(e + 68, packed ? f.group_size : 1);
        store<uint32_t>(e + 72, 0);
        store<uint32_t>(e + 76, t.shard_index);
    }
    if (!table.empty()) std::memcpy(h + metadata_offset, table.data(), table.size());
    if (!strings.empty()) std::memcpy(h + string_offset, strings.data(), strings.size());

    FILE* f = std::fopen(path, "wb");
    if (!f) return fail(MI355Q_ERR_IO, "cannot create %s: %s", path, std::strerror(errno));
    bool ok = std::fwrite(head.data(), 1, head.size(), f) == head.size();
    size_t written = head.size();
    static const uint8_t zeros[kTensorAlignment] = {0};
    for (uint32_t i = 0; ok && i < tensor_count; i++) {
        const size_t pad = (size_t)payload_offsets[i] - written;
        ok = std::fwrite(zeros, 1, pad, f) == pad &&
             std::fwrite(tensors[i].payload, 1, tensors[i].payload_size, f) == tensors[i].payload_size;
        written = (size_t)payload_offsets[i] + tensors[i].payload_size;
    }
    ok = (std::fclose(f) == 0) && ok;
    if (!ok) return fail(MI355Q_ERR_IO, "short write to %s", path);
    return MI355Q_OK;
}

}  // extern "C"
