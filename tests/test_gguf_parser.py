"""The GGUF reader of the library against the reference's own parser tests (the same file images,
assembled byte for byte as crates/oxillama-gguf/src/{header,parser,loader}.rs tests do) and against
an independent Python parser on randomized files.  CPU only: parsing touches no device."""
import struct

import numpy as np
import pytest

import gguf_build as B
from oxillama_amd import gguf

Q4_0, Q8_0, F32, F16 = 2, 8, 0, 1


def build_test_gguf():  # parser.rs:232-270
    return B.build(3, [("general.architecture", B.STRING, "llama"), ("llama.block_count", B.U32, 32)],
                   [("output.weight", [32, 32], Q4_0, 0)], b"\xAB" * 1024)


def test_parse_full_gguf():  # parser.rs:277-292
    g = gguf.GgufModel.from_bytes(build_test_gguf())
    assert (g.version, g.tensor_count, g.metadata_kv_count) == (3, 1, 2)
    assert g.architecture() == "llama" and g.metadata("llama.block_count") == 32
    assert g.n_tensors == 1
    t = g.tensor("output.weight")
    assert (t.n_dims, t.dimensions, t.tensor_type) == (2, [32, 32], Q4_0)
    assert t.n_elements() == 1024 and t.data_size() == 32 * 18  # tensor_info.rs:35-50
    data = g.tensor_data("output.weight")  # parser.rs:295-300
    assert data.size == 576 and np.all(data == 0xAB)
    with pytest.raises(gguf.TensorNotFound):  # parser.rs:303-307
        g.tensor_data("nonexistent")
    assert g.alignment == 32 and g.data_offset % 32 == 0 and g.file_size() == len(build_test_gguf())
    g.close()


def test_model_name_present_and_absent():  # parser.rs:310-345
    img = B.build(3, [("general.architecture", B.STRING, "llama"), ("general.name", B.STRING, "TestModel")], [])
    g = gguf.GgufModel.from_bytes(img)
    assert g.model_name() == "TestModel" and g.architecture() == "llama"
    g = gguf.GgufModel.from_bytes(B.build(3, [("general.architecture", B.STRING, "llama")], []))
    assert g.model_name() is None


def test_header_versions():  # header.rs:100-190, parser.rs:375-383,615-680
    g = gguf.GgufModel.from_bytes(B.build(2, [("general.architecture", B.STRING, "qwen")], []))
    assert (g.version, g.tensor_count, g.metadata_kv_count, g.architecture(), g.n_tensors) == (2, 0, 1, "qwen", 0)
    # v2 with a tensor: u32 counts, string lengths and dims, u64 offset (parser.rs:520-578)
    img = B.build(2, [("general.architecture", B.STRING, "llama")], [("embed.weight", [64, 32], Q8_0, 0)], b"\xCD" * 4096)
    g = gguf.GgufModel.from_bytes(img)
    t = g.tensor("embed.weight")
    assert (g.version, t.n_dims, t.dimensions, t.tensor_type) == (2, 2, [64, 32], Q8_0)
    assert g.tensor_data("embed.weight").size == 64 * 34
    # v1: u32 offset as well (parser.rs:581-632)
    img = B.build(1, [("general.architecture", B.STRING, "gpt2")], [("token_embd.weight", [16, 16], F16, 0)], b"\xAA" * 1024)
    g = gguf.GgufModel.from_bytes(img)
    t = g.tensor("token_embd.weight")
    assert (g.version, g.architecture(), t.dimensions, t.tensor_type, t.offset) == (1, "gpt2", [16, 16], F16, 0)
    g = gguf.GgufModel.from_bytes(B.build(1, [("general.architecture", B.STRING, "phi")], []))
    assert (g.version, g.architecture(), g.n_tensors) == (1, "phi", 0)
    # header sizes: 24 bytes in v3, 16 before (header.rs:115-155)
    g = gguf.GgufModel.from_bytes(struct.pack("<IIQQ", B.MAGIC, 3, 0, 0))
    assert g.data_offset == 32 and g.file_size() == 24  # aligned up past the end of a file with no tensors
    g = gguf.GgufModel.from_bytes(b"GGUF" + struct.pack("<IQQ", 3, 0, 0))  # the literal magic bytes (header.rs:175-190)
    assert g.version == 3


def test_header_errors():
    with pytest.raises(gguf.InvalidMagic) as e:  # header.rs:121-125
        gguf.GgufModel.from_bytes(bytes([0, 0, 0, 0, 3, 0, 0, 0]))
    assert e.value.magic == 0
    for v in (0, 4):  # header.rs:158-167, parser.rs:653-680
        with pytest.raises(gguf.UnsupportedVersion) as e:
            gguf.GgufModel.from_bytes(struct.pack("<IIII", B.MAGIC, v, 0, 0))
        assert e.value.version == v
    with pytest.raises(gguf.UnexpectedEof):  # loader.rs: truncated after the magic
        gguf.GgufModel.from_bytes(b"GGUF")
    with pytest.raises(gguf.UnexpectedEof) as e:
        gguf.GgufModel.from_bytes(b"GG")
    assert e.value.offset == 0
    with pytest.raises(gguf.UnexpectedEof) as e:  # count field cut short: offset of the field
        gguf.GgufModel.from_bytes(struct.pack("<II", B.MAGIC, 3) + b"\0\0\0")
    assert e.value.offset == 8
    with pytest.raises(gguf.IoError):  # loader.rs: load of a missing file
        gguf.GgufModel.load("/nonexistent/path/does_not_exist.gguf")


def test_all_scalar_value_types_and_arrays():  # parser.rs:406-497, 683-707
    kvs = [("k.u8", B.U8, 200), ("k.i8", B.I8, -100), ("k.u16", B.U16, 60000), ("k.i16", B.I16, -30000),
           ("k.u32", B.U32, 4000000000), ("k.i32", B.I32, -2000000000), ("k.f32", B.F32, 1.5), ("k.bool", B.BOOL, 1),
           ("k.str", B.STRING, "héllo"), ("k.u64", B.U64, 2 ** 63 + 5), ("k.i64", B.I64, -2 ** 62), ("k.f64", B.F64, 2.25),
           ("k.arr", B.ARRAY, (B.U32, [1, 2, 3])), ("k.sarr", B.ARRAY, (B.STRING, ["a", "bc", ""])),
           ("k.nested", B.ARRAY, (B.ARRAY, [(B.U8, [1, 2]), (B.U8, [])]))]
    for version in (2, 3):
        g = gguf.GgufModel.from_bytes(B.build(version, kvs, []))
        assert g.n_metadata == len(kvs)
        got = dict(g.metadata_items())
        assert got["k.u8"] == 200 and got["k.i8"] == -100 and got["k.u16"] == 60000 and got["k.i16"] == -30000
        assert got["k.u32"] == 4000000000 and got["k.i32"] == -2000000000 and got["k.f32"] == 1.5 and got["k.bool"] is True
        assert got["k.str"] == "héllo" and got["k.u64"] == 2 ** 63 + 5 and got["k.i64"] == -2 ** 62 and got["k.f64"] == 2.25
        assert got["k.arr"] == ("array", B.U32, 3) and got["k.sarr"] == ("array", B.STRING, 3)
        assert got["k.nested"] == ("array", B.ARRAY, 2)
        assert [k for k, _ in g.metadata_items()] == [k for k, _, _ in kvs]  # file order
        # array payloads stay readable (tokenizer lists live in such arrays)
        assert g.metadata_array("k.arr") == [1, 2, 3] and g.metadata_array("k.sarr") == ["a", "bc", ""]
        with pytest.raises(gguf.InvalidMetadata):
            g.metadata_array("k.u8")
        with pytest.raises(gguf.InvalidMetadata):
            g.metadata_array("k.nested")
    with pytest.raises(gguf.InvalidMetadata):  # a missing key (MetadataStore::get_string, metadata.rs:162-169)
        g.metadata("absent")


def test_metadata_errors():
    bad_type = struct.pack("<IIQQ", B.MAGIC, 3, 0, 1) + B.string(3, "k") + struct.pack("<I", 13)
    with pytest.raises(gguf.InvalidMetadata):  # parser.rs:103-107: unknown value type
        gguf.GgufModel.from_bytes(bad_type)
    bad_elem = struct.pack("<IIQQ", B.MAGIC, 3, 0, 1) + B.string(3, "k") + struct.pack("<II", B.ARRAY, 99) + struct.pack("<Q", 0)
    with pytest.raises(gguf.InvalidMetadata):  # parser.rs:139-145
        gguf.GgufModel.from_bytes(bad_elem)
    bad_utf8 = struct.pack("<IIQQ", B.MAGIC, 3, 0, 1) + struct.pack("<Q", 2) + b"\xff\xfe"
    with pytest.raises(gguf.InvalidString) as e:  # reader.rs:182-185
        gguf.GgufModel.from_bytes(bad_utf8)
    assert e.value.offset == 32
    huge = struct.pack("<IIQQ", B.MAGIC, 3, 0, 1) + struct.pack("<Q", 2 ** 60)
    with pytest.raises(gguf.UnexpectedEof) as e:  # a string length far past the end must not be trusted
        gguf.GgufModel.from_bytes(huge)
    assert e.value.offset == 32
    many = struct.pack("<IIQQ", B.MAGIC, 3, 2 ** 40, 0)
    with pytest.raises(gguf.UnexpectedEof):  # tensor_count far beyond the file
        gguf.GgufModel.from_bytes(many)


def test_more_than_four_dimensions_parse_and_show_the_first_four():
    g = gguf.GgufModel.from_bytes(B.build(3, [], [("t5", [2, 3, 4, 5, 6], F32, 0)], b"\0" * (720 * 4)))
    t = g.tensor("t5")
    assert t.n_dims == 5 and t.dimensions == [2, 3, 4, 5] and t.n_elements() == 720 and t.data_size() == 2880
    assert len(g.tensor_data("t5")) == 2880


def test_array_element_of_unknown_type_is_an_error_not_a_half_parsed_file():
    # an array whose element type id is past the last known one (parser.rs:118-169)
    img = struct.pack("<IIQQ", B.MAGIC, 3, 0, 1) + B.string(3, "k") + struct.pack("<I", B.ARRAY) + \
        struct.pack("<I", 13) + struct.pack("<Q", 1) + b"\0" * 8
    with pytest.raises(gguf.InvalidMetadata):
        gguf.GgufModel.from_bytes(img)


def test_tensor_errors():
    img = B.build(3, [], [("w", [4], 5, 0)])  # ids 4 and 5 were never assigned (types.rs:154-196)
    with pytest.raises(gguf.UnsupportedQuantType) as e:
        gguf.GgufModel.from_bytes(img)
    assert e.value.type_id == 5
    # parser.rs:499-517: data section far too small for the tensor
    img = B.build(3, [], [("w", [128, 128], F32, 0)], b"\0" * 4)
    g = gguf.GgufModel.from_bytes(img)
    with pytest.raises(gguf.UnexpectedEof) as e:
        g.tensor_data("w")
    assert e.value.offset == g.data_offset
    # an offset beyond the file, and one that would overflow
    g = gguf.GgufModel.from_bytes(B.build(3, [], [("w", [32], Q8_0, 10 ** 9), ("v", [32], Q8_0, 2 ** 64 - 8)], b"\0" * 64))
    for name in ("w", "v"):
        with pytest.raises(gguf.UnexpectedEof):
            g.tensor_data(name)
    # dimensions whose product does not fit 64 bits
    g = gguf.GgufModel.from_bytes(B.build(3, [], [("big", [2 ** 40, 2 ** 40], F32, 0)], b"\0" * 64))
    with pytest.raises(gguf.UnexpectedEof):
        g.tensor_data("big")


def test_alignment_and_duplicates():
    # general.alignment moves the data section (parser.rs:41-52); a tensor at a non-zero offset
    data = bytes(range(256)) * 2
    img = B.build(3, [("general.alignment", B.U32, 64)], [("a", [32], Q8_0, 0), ("b", [64], F32, 64)], data, alignment=64)
    g = gguf.GgufModel.from_bytes(img)
    assert g.alignment == 64 and g.data_offset % 64 == 0
    assert bytes(g.tensor_data("a")) == data[:34] and bytes(g.tensor_data("b")) == data[64:64 + 256]
    # a later entry of the same name replaces the earlier one (HashMap insert, tensor_info.rs:79-81)
    img = B.build(3, [("k", B.U32, 1), ("k", B.U32, 2)], [("t", [32], Q8_0, 0), ("t", [64], Q8_0, 34)], b"\0" * 128)
    g = gguf.GgufModel.from_bytes(img)
    assert (g.tensor_count, g.n_tensors, g.n_metadata) == (2, 1, 1)
    assert g.tensor("t").dimensions == [64] and g.tensor("t").offset == 34 and g.metadata("k") == 2
    # align_up cases of parser.rs:386-403
    assert (B.align_up(32, 32), B.align_up(33, 32), B.align_up(7, 0)) == (32, 64, 7)


def test_every_tensor_type_size():  # types.rs:199-262 through TensorInfo::data_size
    tensors, off = [], 0
    for tid, (bs, bb) in sorted(B.LAYOUT.items()):
        tensors.append((f"t{tid}", [3, 2 * bs], tid, off))
        off += 6 * bb
    g = gguf.GgufModel.from_bytes(B.build(3, [], tensors, b"\0" * off))
    for (name, dims, tid, o), t in zip(tensors, g.tensors()):
        bs, bb = B.LAYOUT[tid]
        assert (t.name, t.tensor_type, t.offset, t.n_elements(), t.data_size()) == (name, tid, o, 6 * bs, 6 * bb)
        assert g.tensor_data(name).size == 6 * bb
    # ragged element counts round up to whole blocks (div_ceil, tensor_info.rs:47)
    g = gguf.GgufModel.from_bytes(B.build(3, [], [("r", [33], Q8_0, 0)], b"\0" * 68))
    assert g.tensor("r").data_size() == 68
    g = gguf.GgufModel.from_bytes(B.build(3, [], [("z", [], F32, 0)]))
    assert (g.tensor("z").n_elements(), g.tensor("z").data_size()) == (0, 0)


def test_randomized_files_against_independent_parser():
    rng = np.random.default_rng(11)
    scalar_types = [B.U8, B.I8, B.U16, B.I16, B.U32, B.I32, B.BOOL, B.U64, B.I64, B.STRING]
    for trial in range(60):
        version = int(rng.integers(1, 4))
        kvs = []
        for k in range(int(rng.integers(0, 8))):
            vt = scalar_types[int(rng.integers(0, len(scalar_types)))]
            if vt == B.STRING:
                v = "".join(chr(int(c)) for c in rng.integers(32, 127, size=int(rng.integers(0, 20))))
            elif vt == B.BOOL:
                v = int(rng.integers(0, 2))
            else:
                lo, hi = {B.U8: (0, 255), B.I8: (-128, 127), B.U16: (0, 65535), B.I16: (-32768, 32767), B.U32: (0, 2 ** 32 - 1),
                          B.I32: (-2 ** 31, 2 ** 31 - 1), B.U64: (0, 2 ** 63 - 1), B.I64: (-2 ** 62, 2 ** 62)}[vt]
                v = int(rng.integers(lo, hi, endpoint=True))
            kvs.append((f"key.{k}", vt, v))
        alignment = 32
        if rng.integers(0, 3) == 0:
            alignment = int(rng.choice([8, 16, 64, 128]))
            kvs.append(("general.alignment", B.U32, alignment))
        tensors, off = [], 0
        for k in range(int(rng.integers(0, 6))):
            tid = int(rng.choice(sorted(B.LAYOUT)))
            bs, bb = B.LAYOUT[tid]
            dims = [int(rng.integers(1, 5)), bs * int(rng.integers(1, 4))]
            tensors.append((f"blk.{k}.w", dims, tid, off))
            off += B.align_up(dims[0] * dims[1] // bs * bb, alignment)
        data = rng.integers(0, 256, size=off, dtype=np.uint8).tobytes()
        img = B.build(version, kvs, tensors, data, alignment=alignment)
        v, meta, tmap, data_off, al = B.parse(img)
        g = gguf.GgufModel.from_bytes(img)
        assert (g.version, g.alignment, g.data_offset, g.n_tensors, g.n_metadata) == (v, al, data_off, len(tmap), len(meta))
        for k, val in g.metadata_items():
            assert meta[k] == val
        for t in g.tensors():
            dims, tid, o = tmap[t.name]
            assert (t.dimensions, t.tensor_type, t.offset) == (dims, tid, o)
            bs, bb = B.LAYOUT[tid]
            size = dims[0] * dims[1] // bs * bb
            assert bytes(g.tensor_data(t.name)) == img[data_off + o:data_off + o + size]
        # every truncation of the header part fails cleanly (no crash, an EOF-class error)
        cut = int(rng.integers(8, max(9, data_off - 1))) if data_off > 9 else 8
        try:
            gguf.GgufModel.from_bytes(img[:cut]).close()
        except (gguf.UnexpectedEof, gguf.InvalidString):
            pass
        g.close()


def test_mmap_route_matches_bytes_route(tmp_path):
    img = build_test_gguf()
    p = tmp_path / "m.gguf"
    p.write_bytes(img)
    g = gguf.GgufModel.load(p)  # GgufModel::load_mmap, loader.rs:54-69
    assert (g.version, g.n_tensors, g.architecture(), g.file_size()) == (3, 1, "llama", len(img))
    assert np.all(g.tensor_data("output.weight") == 0xAB)
    g.close()
    (tmp_path / "empty.gguf").write_bytes(b"")
    with pytest.raises(gguf.UnexpectedEof):
        gguf.GgufModel.load(tmp_path / "empty.gguf")
