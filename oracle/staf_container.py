"""CPU restatement of the STAF on-disk container (test infrastructure, never imported by the product).

Follows the reference's writer and loader field by field:
  * constants and header / section-entry layout: Sources/MetalCompiler/STAF/STAFFormat.swift:10-80, 84-167
  * writer: Sources/MetalCompiler/STAF/STAFWriter.swift:11-120 (file assembly), :122-146 (header),
    :148-184 (section entry), :186-238 (metadata entry), :240-262 (payload size)
  * loader: Sources/MetalCompiler/STAF/STAFLoader.swift:38-198; metadata: STAFMetadataDecoder.swift:31-145
  * validator: Sources/MetalCompiler/STAF/STAFValidator.swift:5-78

Pinned by: a file assembled by hand at the literal byte offsets the loader's comment table lists
(tests/test_staf_container.py), the structural facts the reference's own tests check (256-byte tensor
alignment, 4096-byte payload start, non-overlap, shapes, long names: Tests/MetalCompilerTests/Core/
STAFDeepTests.swift:222-289, 703-745, 746-790, 958-993) and byte equality with the library's writer, an
independent implementation.  The reference holds no literal model.staf bytes to compare with.
"""
from __future__ import annotations

import struct

MAGIC = 0x46415453                 # "STAF", STAFFormat.swift:13
CURRENT_FORMAT_VERSION = 2         # :26
LEGACY_FORMAT_VERSION = 0          # :29
CURRENT_CONVERTER_VERSION = 3      # :50
CURRENT_METADATA_SCHEMA_VERSION = 1
HEADER_SIZE, SECTION_ENTRY_SIZE, METADATA_ENTRY_SIZE = 64, 128, 32     # :53-59
PAYLOAD_ALIGNMENT, TENSOR_ALIGNMENT = 4096, 256                         # :62-65

BOOL, UINT32, UINT64, FLOAT32, FLOAT64, STRING = 1, 2, 3, 4, 5, 6       # STAFMetadataValue.swift:12-19

# scheme -> (bits, group, bytes per block); the registry of QuantizationFormat.swift:1284-1312 (+ 0x42 alias)
_PACKED = {0x10: (8, 32), 0x11: (8, 64), 0x12: (8, 128), 0x20: (6, 16), 0x21: (6, 32), 0x30: (5, 32), 0x31: (5, 64),
           0x40: (4, 64), 0x41: (4, 128), 0x42: (4, 128), 0x50: (3, 16), 0x51: (3, 32), 0x52: (3, 64),
           0x60: (2, 16), 0x61: (2, 32)}


def align_up(v: int, a: int) -> int:
    return v if v % a == 0 else v + (a - v % a)


def payload_size(scheme: int, shape) -> int:
    """STAFWriter.computePayloadSize (STAFWriter.swift:240-262)."""
    elements = 1
    for d in shape:
        elements *= d
    if scheme in (0x00, 0x01, 0xFF):
        return elements * 2
    if scheme == 0x02:
        return elements * 4
    if scheme not in _PACKED:
        return elements * 2
    bits, group = _PACKED[scheme]
    n = shape[0]
    packed = shape[1] if len(shape) >= 2 else 1
    k = packed * 32 // bits
    return n * (k // group) * (4 + group * bits // 8)


def write_staf(tensors, metadata=None) -> bytes:
    """tensors: list of dicts (name, scheme_identifier, shape, payload, semantic_role, original_dtype,
    shard_index); metadata: {key: (type, value)}.  Returns the file image (STAFWriter.write)."""
    metadata = metadata or {}
    n = len(tensors)
    section_offset = HEADER_SIZE
    metadata_offset = section_offset + n * SECTION_ENTRY_SIZE
    items = sorted(metadata.items(), key=lambda kv: kv[0].encode())
    strings = bytearray()
    offsets = {}

    def append(text: str) -> int:
        if text in offsets:
            return offsets[text]
        off = len(strings)
        strings.extend(text.encode())
        strings.append(0)
        offsets[text] = off
        return off

    name_offsets = [append(t["name"]) for t in tensors]
    table = bytearray()
    for key, (typ, value) in items:
        key_offset = append(key)
        p0 = p1 = 0
        if typ == BOOL:
            p0 = 1 if value else 0
        elif typ == UINT32:
            p0 = value & 0xFFFFFFFF
        elif typ == UINT64:
            p0 = value
        elif typ == FLOAT32:
            p0 = struct.unpack("<I", struct.pack("<f", value))[0]
        elif typ == FLOAT64:
            p0 = struct.unpack("<Q", struct.pack("<d", value))[0]
        elif typ == STRING:
            p0, p1 = append(value), len(value.encode())
        entry = bytearray(METADATA_ENTRY_SIZE)
        struct.pack_into("<II", entry, 0, key_offset, len(key.encode()))
        entry[8] = typ
        struct.pack_into("<QQ", entry, 12, p0, p1)
        table += entry
    string_offset = metadata_offset + len(table)
    payload_start = align_up(string_offset + len(strings), PAYLOAD_ALIGNMENT)
    payload_offsets, cursor = [], payload_start
    for t in tensors:
        off = align_up(cursor, TENSOR_ALIGNMENT)
        payload_offsets.append(off)
        cursor = off + len(bytes(t["payload"]))

    out = bytearray(HEADER_SIZE)
    struct.pack_into("<IIII", out, 0, MAGIC, CURRENT_FORMAT_VERSION, len(items), metadata_offset)
    struct.pack_into("<IIII", out, 40, n, section_offset, string_offset, len(strings))
    for i, t in enumerate(tensors):
        e = bytearray(SECTION_ENTRY_SIZE)
        shape = list(t["shape"])
        struct.pack_into("<II", e, 0, name_offsets[i], len(t["name"].encode()))
        e[8], e[9], e[10] = t["scheme_identifier"], t.get("semantic_role", 0), t.get("original_dtype", 0xFF)
        e[11] = min(len(shape), 8)
        for d in range(8):
            struct.pack_into("<I", e, 12 + 4 * d, shape[d] if d < len(shape) else 0)
        struct.pack_into("<QQ", e, 44, payload_offsets[i], len(bytes(t["payload"])))
        group = _PACKED[t["scheme_identifier"]][1] if t["scheme_identifier"] in _PACKED else 1
        struct.pack_into("<IIIII", e, 60, TENSOR_ALIGNMENT, group, group, 0, t.get("shard_index", 0))
        out += e
    out += table
    out += strings
    out += bytes(payload_start - len(out))
    for i, t in enumerate(tensors):
        out += bytes(payload_offsets[i] - len(out))
        out += bytes(t["payload"])
    return bytes(out)


class InvalidFile(ValueError):
    pass


def parse_staf(data: bytes) -> dict:
    """STAFLoader.load without the device: {'format_version', 'entries': [...], 'metadata': {...},
    'first_payload_offset'}; raises InvalidFile where the loader throws invalidFile."""
    if len(data) <= HEADER_SIZE:
        raise InvalidFile("File too small or missing")
    magic, version, md_count, md_offset = struct.unpack_from("<IIII", data, 0)
    count, section_offset, string_offset, string_size = struct.unpack_from("<IIII", data, 40)
    if magic != MAGIC:
        raise InvalidFile("Bad magic: expected STAF")
    if version not in (LEGACY_FORMAT_VERSION, CURRENT_FORMAT_VERSION):
        raise InvalidFile(f"Unsupported STAF format version: {version}")
    metadata = {}
    if version >= CURRENT_FORMAT_VERSION and md_count > 0 and md_offset > 0:
        if md_offset < HEADER_SIZE or md_offset + md_count * METADATA_ENTRY_SIZE > len(data):
            raise InvalidFile("Metadata table is out of bounds")
        if string_offset + string_size > len(data):
            raise InvalidFile("String table is out of bounds")

        def text(off, length):
            if off + length > string_size:
                raise InvalidFile("Metadata string is out of bounds")
            return data[string_offset + off:string_offset + off + length].decode()

        for i in range(md_count):
            base = md_offset + i * METADATA_ENTRY_SIZE
            key_offset, key_length = struct.unpack_from("<II", data, base)
            typ = data[base + 8]
            p0, p1 = struct.unpack_from("<QQ", data, base + 12)
            if typ not in (BOOL, UINT32, UINT64, FLOAT32, FLOAT64, STRING):
                raise InvalidFile(f"Unknown metadata value type: {typ}")
            key = text(key_offset, key_length)
            if typ == BOOL:
                value = p0 != 0
            elif typ == UINT32:
                value = p0 & 0xFFFFFFFF
            elif typ == UINT64:
                value = p0
            elif typ == FLOAT32:
                value = struct.unpack("<f", struct.pack("<I", p0 & 0xFFFFFFFF))[0]
            elif typ == FLOAT64:
                value = struct.unpack("<d", struct.pack("<Q", p0))[0]
            else:
                value = text(p0, p1)
            metadata[key] = (typ, value)
    entries = []
    for i in range(count):
        base = section_offset + i * SECTION_ENTRY_SIZE
        name_offset, name_length = struct.unpack_from("<II", data, base)
        ndim = min(data[base + 11], 8)
        shape = struct.unpack_from(f"<{ndim}I", data, base + 12) if ndim else ()
        payload_offset, size = struct.unpack_from("<QQ", data, base + 44)
        alignment, block, group, checksum, shard = struct.unpack_from("<IIIII", data, base + 60)
        if payload_offset > len(data) or size > len(data):
            raise InvalidFile(f"Payload overflow in section {i}/{count}")
        name = data[string_offset + name_offset:string_offset + name_offset + name_length].decode()
        entries.append(dict(name=name, scheme_identifier=data[base + 8], semantic_role=data[base + 9],
                            original_dtype=data[base + 10], shape=tuple(shape), payload_offset=payload_offset,
                            payload_size=size, alignment=alignment, block_size=block, group_size=group,
                            checksum=checksum, shard_index=shard))
    if not entries:
        raise InvalidFile("No tensors in STAF")
    first = min(e["payload_offset"] for e in entries)
    for e in entries:
        e["buffer_offset"] = e["payload_offset"] - first
    return dict(format_version=version, entries=entries, metadata=metadata, first_payload_offset=first)
