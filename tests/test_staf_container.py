"""CPU tests of the STAF container reader / validator / writer (host code of the shared library; no GPU).

The layout is pinned three ways: (1) a file assembled here by hand at the byte offsets the reference loader
documents (STAFLoader.swift:70-88, STAFFormat.swift:68-80), (2) byte equality between the library's writer
and the oracle's independent restatement of STAFWriter.swift, (3) the structural checks of the reference's
own tests (STAFDeepTests.swift: 100 tensors, 256-byte alignment, shapes, long names, truncated file, bad
magic, validator cases)."""
import os
import struct
import time

import numpy as np
import pytest

import kat
import oracle
from oracle import staf_container as orc

from __graft_entry__ import load_package

pkg = load_package()


def _f16(values):
    return np.asarray(values, np.float16).tobytes()


def _q_payload(bits, group, n, k, seed):
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 1 << bits, (n, k), dtype=np.uint8)
    s = rng.choice([0.5, 0.25, 0.125], (n, k // group)); z = rng.integers(-8, 8, (n, k // group)) * 0.25
    return kat.staf_blocks(codes, s, z, bits, group).tobytes(), codes, s, z


def _mixed_tensors():
    q4, *_ = _q_payload(4, 64, 6, 256, 1)
    q4b, *_ = _q_payload(4, 128, 3, 256, 2)
    q8, *_ = _q_payload(8, 32, 5, 64, 3)
    q3, *_ = _q_payload(3, 64, 4, 128, 4)
    return [
        dict(name="model.embed_tokens.weight", scheme_identifier=0x00, shape=[4, 16], payload=_f16(np.arange(64)),
             semantic_role=0x01, original_dtype=0x01),
        dict(name="model.layers.0.self_attn.q_proj.weight", scheme_identifier=0x40, shape=[6, 256 * 4 // 32],
             payload=q4, semantic_role=0x02, original_dtype=0x06),
        dict(name="model.layers.0.mlp.gate_proj.weight", scheme_identifier=0x41, shape=[3, 256 * 4 // 32], payload=q4b,
             semantic_role=0x06, original_dtype=0x06, shard_index=1),
        dict(name="model.layers.0.mlp.up_proj.weight", scheme_identifier=0x10, shape=[5, 64 * 8 // 32], payload=q8,
             semantic_role=0x07, original_dtype=0x06),
        dict(name="model.layers.0.mlp.down_proj.weight", scheme_identifier=0x52, shape=[4, 128 * 3 // 32], payload=q3,
             semantic_role=0x08, original_dtype=0x06),
        dict(name="model.norm.weight", scheme_identifier=0x01, shape=[8], payload=bytes(range(16)), semantic_role=0x09,
             original_dtype=0x02),
        dict(name="lm_head.bias", scheme_identifier=0x02, shape=[2, 3], payload=np.arange(6, dtype=np.float32).tobytes(),
             semantic_role=0xFF, original_dtype=0x00),
    ]


_METADATA = {
    "general.source_format": (orc.STRING, "safetensors"),
    "staf.converter_version": (orc.UINT32, orc.CURRENT_CONVERTER_VERSION),
    "staf.source_shard_count": (orc.UINT64, 2),
    "staf.metadata_schema_version": (orc.UINT32, orc.CURRENT_METADATA_SCHEMA_VERSION),
    "model.tied_embeddings": (orc.BOOL, True),
    "model.rope_theta": (orc.FLOAT32, 500000.0),
    "model.some_double": (orc.FLOAT64, 1e-5),
    # a string value equal to a tensor name shares that name's bytes in the string table
    "alias": (orc.STRING, "model.norm.weight"),
}


def test_writer_matches_the_oracle_writer_byte_for_byte(tmp_path):
    path = tmp_path / "model.staf"
    tensors = _mixed_tensors()
    pkg.staf_write(str(path), tensors, _METADATA)
    got = path.read_bytes()
    want = orc.write_staf(tensors, _METADATA)
    assert len(got) == len(want)
    assert got == want
    # without metadata and without tensors the header still carries the table offsets
    pkg.staf_write(str(path), tensors[:1], None)
    assert path.read_bytes() == orc.write_staf(tensors[:1], None)
    pkg.staf_write(str(path), [], None)
    assert path.read_bytes() == orc.write_staf([], None) and path.stat().st_size == 4096


def _hand_built_file():
    """One bf16 tensor and one q4 g64 tensor, two metadata values, written field by field at the literal
    offsets of the loader's table (STAFLoader.swift:70-88) -- no code shared with either writer."""
    names = b"w.a\x00w.b\x00k1\x00k2\x00text\x00"
    f = bytearray(8192 + 512)
    struct.pack_into("<I", f, 0, 0x46415453)      # "STAF"
    struct.pack_into("<I", f, 4, 2)               # format version
    struct.pack_into("<I", f, 8, 2)               # metadata entries
    struct.pack_into("<I", f, 12, 64 + 2 * 128)   # metadata table
    struct.pack_into("<I", f, 40, 2)              # sections
    struct.pack_into("<I", f, 44, 64)             # section table
    struct.pack_into("<I", f, 48, 64 + 2 * 128 + 2 * 32)   # string table
    struct.pack_into("<I", f, 52, len(names))
    e = 64                                         # entry 0: "w.a", bf16 [2, 4] at 4096
    struct.pack_into("<II", f, e, 0, 3)
    f[e + 8], f[e + 9], f[e + 10], f[e + 11] = 0x01, 0x09, 0x02, 2
    struct.pack_into("<II", f, e + 12, 2, 4)
    struct.pack_into("<Q", f, e + 44, 4096); struct.pack_into("<Q", f, e + 52, 16)
    struct.pack_into("<IIIII", f, e + 60, 256, 1, 1, 0, 0)
    e = 64 + 128                                   # entry 1: "w.b", q4 g64 [3, 8 words] at 8192
    struct.pack_into("<II", f, e, 4, 3)
    f[e + 8], f[e + 9], f[e + 10], f[e + 11] = 0x40, 0x06, 0x06, 2
    struct.pack_into("<II", f, e + 12, 3, 8)
    struct.pack_into("<Q", f, e + 44, 8192); struct.pack_into("<Q", f, e + 52, 3 * 36)
    struct.pack_into("<IIIII", f, e + 60, 256, 64, 64, 0xDEADBEEF, 7)
    m = 64 + 2 * 128                               # metadata 0: k1 = uint32 3; metadata 1: k2 = string "text"
    struct.pack_into("<II", f, m, 8, 2); f[m + 8] = 2; struct.pack_into("<QQ", f, m + 12, 3, 0)
    struct.pack_into("<II", f, m + 32, 11, 2); f[m + 32 + 8] = 6; struct.pack_into("<QQ", f, m + 32 + 12, 14, 4)
    f[64 + 2 * 128 + 64:64 + 2 * 128 + 64 + len(names)] = names
    f[4096:4112] = bytes(range(100, 116))
    f[8192:8192 + 108] = bytes((i * 7) & 0xFF for i in range(108))
    return bytes(f)


def test_reader_on_a_file_assembled_at_the_documented_offsets(tmp_path):
    data = _hand_built_file()
    path = tmp_path / "hand.staf"
    path.write_bytes(data)
    f = pkg.STAFFile(str(path))
    assert f.format_version == 2
    a, b = f.entries
    assert (a.name, a.scheme_identifier, a.semantic_role, a.original_dtype, a.shape) == ("w.a", 0x01, 0x09, 0x02, (2, 4))
    assert (a.payload_offset, a.payload_size, a.buffer_offset, a.alignment, a.block_size, a.group_size) == (4096, 16, 0, 256, 1, 1)
    assert (b.name, b.scheme_identifier, b.shape, b.payload_offset, b.payload_size) == ("w.b", 0x40, (3, 8), 8192, 108)
    assert (b.buffer_offset, b.block_size, b.group_size, b.checksum, b.shard_index) == (4096, 64, 64, 0xDEADBEEF, 7)
    assert f.metadata == {"k1": (orc.UINT32, 3), "k2": (orc.STRING, "text")}
    assert f.find("w.b") == b
    with pytest.raises(pkg.MI355QError) as err:
        f.find("w.c")
    assert err.value.status_name == "NOT_FOUND"
    assert f.payload(a).tobytes() == bytes(range(100, 116))
    assert f.payload(b).tobytes() == bytes((i * 7) & 0xFF for i in range(108))
    assert f.payload_region().size == len(data) - 4096          # first tensor to end of file
    f.close()
    # the oracle's parser reads the same file the same way
    parsed = orc.parse_staf(data)
    assert [e["name"] for e in parsed["entries"]] == ["w.a", "w.b"] and parsed["metadata"] == f_metadata_expected()


def f_metadata_expected():
    return {"k1": (orc.UINT32, 3), "k2": (orc.STRING, "text")}


def test_reader_and_oracle_parser_agree_on_each_others_files(tmp_path):
    tensors = _mixed_tensors()
    path = tmp_path / "a.staf"
    path.write_bytes(orc.write_staf(tensors, _METADATA))           # oracle writes, library reads
    f = pkg.STAFFile(str(path))
    entries = f.entries
    assert [e.name for e in entries] == [t["name"] for t in tensors]
    for e, t in zip(entries, tensors):
        assert e.shape == tuple(t["shape"]) and e.scheme_identifier == t["scheme_identifier"]
        assert e.semantic_role == t.get("semantic_role", 0) and e.shard_index == t.get("shard_index", 0)
        assert f.payload(e).tobytes() == bytes(t["payload"])
    md = f.metadata
    assert set(md) == set(_METADATA)
    for k, (typ, v) in _METADATA.items():
        assert md[k][0] == typ and (md[k][1] == v or (typ == orc.FLOAT32 and md[k][1] == np.float32(v)))
    f.close()
    pkg.staf_write(str(path), tensors, _METADATA)                   # library writes, oracle parses
    parsed = orc.parse_staf(path.read_bytes())
    assert [(e["name"], e["shape"], e["payload_size"]) for e in parsed["entries"]] == \
        [(t["name"], tuple(t["shape"]), len(t["payload"])) for t in tensors]
    assert parsed["metadata"].keys() == _METADATA.keys()


def test_hundred_tensors_aligned_and_not_overlapping(tmp_path):
    """STAFDeepTests.swift:222-289 and :703-745: every payload on a 256-byte boundary, the payload region on
    a 4096-byte one, no two payloads overlapping, values intact."""
    rng = np.random.default_rng(5)
    tensors = []
    for i in range(100):
        n = int(rng.integers(1, 300))
        tensors.append(dict(name=f"layer.{i}.weight", scheme_identifier=0x00, shape=[1, n],
                            payload=_f16(np.full(n, i + 1))))
    path = tmp_path / "many.staf"
    pkg.staf_write(str(path), tensors, None)
    f = pkg.STAFFile(str(path))
    entries = f.entries
    assert len(entries) == 100
    spans = sorted((e.payload_offset, e.payload_offset + e.payload_size) for e in entries)
    assert spans[0][0] % 4096 == 0
    assert all(lo % 256 == 0 for lo, _ in spans)
    assert all(spans[i][1] <= spans[i + 1][0] for i in range(99))
    for i, e in enumerate(entries):
        assert np.all(f.payload(e).view(np.float16) == np.float16(i + 1))
    f.close()


def test_shapes_long_names_and_f16_edge_values_survive(tmp_path):
    """STAFDeepTests.swift:746-790 (shapes), :958-993 (long names), :792-845 (f16 edge values)."""
    long_name = "model.language_model.layers.31.self_attn." + "very_long_component_name." * 8 + "weight"
    edge = np.array([0x0000, 0x8000, 0x7BFF, 0xFBFF, 0x0001, 0x0400, 0x7C00, 0xFC00], np.uint16)
    shapes = [[128], [4, 32], [2, 4, 16], [2, 2, 2, 2, 8], [1, 1, 1, 1, 1, 1, 1, 8]]
    tensors = [dict(name=f"t{i}", scheme_identifier=0x00, shape=s, payload=bytes(int(np.prod(s)) * 2))
               for i, s in enumerate(shapes)]
    tensors.append(dict(name=long_name, scheme_identifier=0x00, shape=[1, 2], payload=_f16([42.0, 43.0])))
    tensors.append(dict(name="edge", scheme_identifier=0x00, shape=[1, 8], payload=edge.tobytes()))
    path = tmp_path / "s.staf"
    pkg.staf_write(str(path), tensors, None)
    f = pkg.STAFFile(str(path))
    for i, s in enumerate(shapes):
        assert f.find(f"t{i}").shape == tuple(s)
    e = f.find(long_name)
    assert e.name == long_name and np.array_equal(f.payload(e).view(np.float16), np.float16([42.0, 43.0]))
    assert np.array_equal(f.payload(f.find("edge")).view(np.uint16), edge)
    f.close()


def test_writer_checks_the_payload_size_formula(tmp_path):
    """computePayloadSize (STAFWriter.swift:240-262): K = packedDim * 32 / bits, also for widths that do not
    divide 32; dense payloads by element size."""
    path = str(tmp_path / "x.staf")
    for bits, group, scheme in [(3, 64, 0x52), (5, 32, 0x30), (6, 16, 0x20), (4, 64, 0x40), (8, 128, 0x12)]:
        n, k = 3, group * 32 // np.gcd(group * bits, 32) * 2
        payload, *_ = _q_payload(bits, group, n, k, bits)
        assert len(payload) == orc.payload_size(scheme, [n, k * bits // 32])
        good = dict(name="w", scheme_identifier=scheme, shape=[n, k * bits // 32], payload=payload)
        pkg.staf_write(path, [good], None)
        with pytest.raises(pkg.MI355QError) as err:
            pkg.staf_write(path, [dict(good, payload=payload[:-1])], None)
        assert err.value.status_name == "SIZE_MISMATCH"
    with pytest.raises(pkg.MI355QError):
        pkg.staf_write(path, [dict(name="d", scheme_identifier=0x02, shape=[2, 2], payload=bytes(8))], None)


def test_loader_rejects_what_the_reference_rejects(tmp_path):
    """STAFDeepTests.swift:914-956 (truncated file, bad magic) and the other invalidFile exits of
    STAFLoader.load."""
    good = bytearray(_hand_built_file())
    path = tmp_path / "bad.staf"

    def rejected(data, name="INVALID_FILE"):
        path.write_bytes(bytes(data))
        with pytest.raises(pkg.MI355QError) as err:
            pkg.STAFFile(str(path))
        assert err.value.status_name == name
        return str(err.value)

    assert "too small" in rejected(good[:32])
    assert "too small" in rejected(good[:64])
    bad = bytearray(good); bad[0:4] = b"NOPE"
    assert "Bad magic" in rejected(bad)
    bad = bytearray(good); struct.pack_into("<I", bad, 4, 1)
    assert "Unsupported STAF format version: 1" in rejected(bad)
    bad = bytearray(good); struct.pack_into("<Q", bad, 64 + 44, len(good) + 1)
    assert "Payload overflow" in rejected(bad)
    bad = bytearray(good); struct.pack_into("<Q", bad, 64 + 128 + 52, len(good))
    assert "Payload overflow" in rejected(bad)
    bad = bytearray(good); bad[64 + 2 * 128 + 8] = 9
    assert "Unknown metadata value type: 9" in rejected(bad)
    bad = bytearray(good); struct.pack_into("<I", bad, 12, len(good) - 8)
    assert "Metadata table is out of bounds" in rejected(bad)
    bad = bytearray(good); struct.pack_into("<Q", bad, 64 + 2 * 128 + 32 + 12, 100)
    assert "Metadata string is out of bounds" in rejected(bad)
    bad = bytearray(good); struct.pack_into("<I", bad, 40, 0)
    assert "No tensors" in rejected(bad)
    with pytest.raises(pkg.MI355QError):
        pkg.STAFFile(str(tmp_path / "missing.staf"))
    # the oracle's parser raises at the same places
    for mutate in (lambda b: b.__setitem__(slice(0, 4), b"NOPE"), lambda b: struct.pack_into("<I", b, 4, 1),
                   lambda b: struct.pack_into("<I", b, 40, 0)):
        bad = bytearray(good); mutate(bad)
        with pytest.raises(orc.InvalidFile):
            orc.parse_staf(bytes(bad))


def test_legacy_version_zero_loads_without_metadata(tmp_path):
    data = bytearray(_hand_built_file())
    struct.pack_into("<I", data, 4, 0)
    path = tmp_path / "legacy.staf"
    path.write_bytes(bytes(data))
    f = pkg.STAFFile(str(path))
    assert f.format_version == 0 and f.metadata == {} and len(f.entries) == 2
    f.close()
    assert not pkg.staf_is_valid(str(path))                      # the validator wants the current version


def test_validator_cases(tmp_path):
    """STAFDeepTests.swift:1038-1112: invalid when a source is newer, valid / invalid on expected metadata."""
    path = tmp_path / "model.staf"
    src = tmp_path / "model.safetensors"
    src.write_bytes(b"source")
    pkg.staf_write(str(path), _mixed_tensors(), _METADATA)
    now = time.time()
    os.utime(src, (now - 100, now - 100)); os.utime(path, (now, now))
    assert pkg.staf_is_valid(str(path), [str(src)])
    assert pkg.staf_is_valid(str(path), [str(src)], {"staf.converter_version": (orc.UINT32, 3),
                                                     "general.source_format": (orc.STRING, "safetensors"),
                                                     "model.tied_embeddings": (orc.BOOL, True),
                                                     "model.rope_theta": (orc.FLOAT32, 500000.0)})
    assert not pkg.staf_is_valid(str(path), [str(src)], {"staf.converter_version": (orc.UINT32, 2)})
    assert not pkg.staf_is_valid(str(path), [str(src)], {"staf.converter_version": (orc.UINT64, 3)})   # same number, other type
    assert not pkg.staf_is_valid(str(path), [str(src)], {"missing.key": (orc.BOOL, True)})
    assert not pkg.staf_is_valid(str(path), [str(src)], {"general.source_format": (orc.STRING, "gguf")})
    os.utime(src, (now + 100, now + 100))
    assert not pkg.staf_is_valid(str(path), [str(src)])
    link = tmp_path / "link.safetensors"                            # symbolic links resolve to their target's time
    os.symlink(src, link)
    assert not pkg.staf_is_valid(str(path), [str(link)])
    os.utime(src, (now - 100, now - 100))
    assert pkg.staf_is_valid(str(path), [str(link)])
    with pytest.raises(pkg.MI355QError):
        pkg.staf_is_valid(str(path), [str(tmp_path / "gone.safetensors")])
    with pytest.raises(pkg.MI355QError):
        pkg.staf_is_valid(str(tmp_path / "gone.staf"))
    # structural reasons: short file, wrong magic, no sections, section table not right after the header,
    # metadata table overlapping the section table, first payload larger than the file
    data = bytearray(path.read_bytes())
    other = tmp_path / "v.staf"

    def valid(d):
        other.write_bytes(bytes(d))
        return pkg.staf_is_valid(str(other))

    assert valid(data)
    assert not valid(data[:40])
    bad = bytearray(data); bad[0] ^= 1; assert not valid(bad)
    bad = bytearray(data); struct.pack_into("<I", bad, 40, 0); assert not valid(bad)
    bad = bytearray(data); struct.pack_into("<I", bad, 44, 128); assert not valid(bad)
    bad = bytearray(data); struct.pack_into("<I", bad, 12, 64 + 128); assert not valid(bad)
    bad = bytearray(data); struct.pack_into("<Q", bad, 64 + 52, len(data) + 1); assert not valid(bad)


def test_q4_repack_bytes_through_the_container(tmp_path):
    """STAFDeepTests.swift:346-427: an MLX q4 tensor of all-zero codes with scale 1 and bias 0 lands in the
    container as blocks of (f16 1.0, f16 0.0, 32 zero bytes); here with the 0x76543210 word as well."""
    fmt = pkg.QuantizationFormatRegistry.format_for_mlx_quantization(4, 64)
    words = np.zeros((2, 8), np.uint32); words[1, :] = 0x76543210
    s = np.full((2, 1), 0x3C00, np.uint16); z = np.zeros((2, 1), np.uint16)
    blocks = pkg.repack_mlx_to_staf(fmt, words, s, z, pkg.F16)
    path = tmp_path / "q.staf"
    pkg.staf_write(str(path), [dict(name="q.weight", scheme_identifier=0x40, shape=[2, 8], payload=blocks.tobytes())], None)
    f = pkg.STAFFile(str(path))
    e = f.find("q.weight")
    assert e.scheme_identifier == 0x40 and e.payload_size == 2 * 36 and e.block_size == 64 and e.group_size == 64
    raw = f.payload(e)
    assert raw[:4].tobytes() == struct.pack("<HH", 0x3C00, 0x0000) and not raw[4:36].any()
    assert raw[36:40].tobytes() == struct.pack("<HH", 0x3C00, 0x0000)
    assert raw[40:72].tobytes() == bytes([0x10, 0x32, 0x54, 0x76] * 8)
    assert np.array_equal(oracle.unpack_staf_codes(4, 64, 2, 64, raw)[1, :8], np.arange(8))
    f.close()
