"""GGUF container: the reader against hand-built byte strings whose field values are known by construction,
the reference's own known answers (example-cli/src/model/formats/gguf.rs:409-447), and writer -> reader
round trips.  CPU only."""
import struct

import numpy as np
import pytest

from rustorch_amd import gguf
from rustorch_amd.gguf import GGMLType, GGUFError, GGUFLoader, GGUFValue, GGUFWriter


def s(text):                      # GGUF string: u64 length + bytes
    b = text.encode()
    return struct.pack("<Q", len(b)) + b


def kv(key, vt, payload):
    return s(key) + struct.pack("<I", vt) + payload


def tinfo(name, dims, t, off):
    return s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", t, off)


def build(kvs, tensors, data=b"", magic=0x46554747, version=3, align=32):
    head = struct.pack("<IIQQ", magic, version, len(tensors), len(kvs)) + b"".join(kvs) + b"".join(tensors)
    return head + b"\0" * (-len(head) % align) + data


@pytest.fixture
def tmpfile(tmp_path):
    def put(blob):
        p = tmp_path / "m.gguf"
        p.write_bytes(blob)
        return p
    return put


# ---- the reference's own known answers
def test_reference_type_ids_and_sizes():
    assert GGMLType.from_u32(0) == GGMLType.F32 and GGMLType.from_u32(1) == GGMLType.F16 and GGMLType.from_u32(2) == GGMLType.Q4_0
    with pytest.raises(ValueError):
        GGMLType.from_u32(999)
    assert GGMLType.F32.type_size() == 4 and GGMLType.F16.type_size() == 2 and GGMLType.I8.type_size() == 1


def test_reference_value_accessors():
    assert GGUFValue(gguf.VT_STRING, "test").as_str() == "test"
    assert GGUFValue(gguf.VT_UINT32, 42).as_str() is None
    assert GGUFValue(gguf.VT_UINT32, 42).as_u32() == 42
    assert GGUFValue(gguf.VT_UINT64, 42).as_u32() == 42 and GGUFValue(gguf.VT_UINT32, 7).as_u64() == 7
    assert GGUFValue(gguf.VT_STRING, "x").as_u32() is None


# ---- every value type, from bytes written by hand
def test_all_thirteen_value_types(tmpfile):
    nested = struct.pack("<IQ", gguf.VT_ARRAY, 2) + struct.pack("<IQ", gguf.VT_UINT8, 2) + b"\x01\x02" + struct.pack("<IQ", gguf.VT_UINT8, 1) + b"\x09"
    kvs = [kv("u8", 0, b"\xfe"), kv("i8", 1, b"\xfe"), kv("u16", 2, b"\x34\x12"), kv("i16", 3, b"\xfe\xff"),
           kv("u32", 4, b"\x78\x56\x34\x12"), kv("i32", 5, b"\xff\xff\xff\xff"), kv("f32", 6, b"\x00\x00\x80\x3f"),
           kv("bool", 7, b"\x01"), kv("str", 8, s("héllo")), kv("arr", 9, struct.pack("<IQ", gguf.VT_STRING, 2) + s("a") + s("bc")),
           kv("u64", 10, struct.pack("<Q", 2**40 + 5)), kv("i64", 11, struct.pack("<q", -2**40)), kv("f64", 12, struct.pack("<d", 0.1)),
           kv("nested", 9, nested)]
    g = GGUFLoader(tmpfile(build(kvs, [])))
    m = {k: v.value for k, v in g.metadata.items() if v.kind != gguf.VT_ARRAY}
    assert m == {"u8": 254, "i8": -2, "u16": 0x1234, "i16": -2, "u32": 0x12345678, "i32": -1, "f32": 1.0, "bool": True,
                 "str": "héllo", "u64": 2**40 + 5, "i64": -2**40, "f64": 0.1}
    assert g.get_metadata("arr").as_list() == ["a", "bc"]
    nest = g.get_metadata("nested")
    assert [x.as_list() for x in nest.value] == [[1, 2], [9]]
    assert g.header.tensor_count == 0 and g.header.metadata_kv_count == 14 and g.header.version == 3
    assert g.get_metadata("absent") is None


def test_tensor_table_alignment_and_payload(tmpfile):
    a = np.arange(6, dtype="<f4").tobytes()                          # 24 bytes -> next tensor at 32
    b = bytes(range(34)) * 2                                         # two Q8_0 blocks = one row of 64
    c = np.array([1, -1, 300], dtype="<i2").tobytes()
    data = a + b"\0" * 8 + b + b"\0" * (96 - 68) + c
    blob = build([kv("general.architecture", 8, s("llama"))],
                 [tinfo("a", (3, 2), 0, 0), tinfo("blk.0.w", (64, 1), 8, 32), tinfo("c", (3,), 17, 128)], data)
    g = GGUFLoader(tmpfile(blob))
    assert g.tensor_names() == ["a", "blk.0.w", "c"]
    assert g.tensor_data_offset % 32 == 0 and g.tensor_data_offset == len(blob) - len(data)
    ta = g.find_tensor("a")
    assert (ta.n_dims, ta.dims, ta.ggml_type, ta.offset, ta.n_cols, ta.n_rows, ta.n_bytes) == (2, (3, 2), GGMLType.F32, 0, 3, 2, 24)
    assert g.get_tensor("blk.0.w").n_bytes == 68 and g.find_tensor("nope") is None
    assert np.array_equal(g.load_f32("a"), np.arange(6, dtype=np.float32))
    assert g.load_tensor_data("blk.0.w").tobytes() == b
    assert np.array_equal(g.load_f32("c"), np.array([1, -1, 300], dtype=np.float32))
    with pytest.raises(GGUFError):
        g.load_f32("blk.0.w")
    with pytest.raises(GGUFError):
        g.load_tensor_data("nope")
    # data section accounts for the rest of the file
    last = g.tensors[-1]
    assert g.tensor_data_offset + last.offset + last.n_bytes == g.file_size


def test_reference_scalar_decode_vectors(tmpfile):
    """The reference loader's own known-answer vectors for the unquantized element types
    (example-cli/src/model/formats/tensor_loader.rs:323-356): F32 `00 00 80 3F` -> 1.0, I8 `00 7F FF` -> 0, 127, -1,
    I16 `00 00 01 00` -> 0, 1, I32 `00 00 00 00 01 00 00 00` -> 0, 1, and a payload whose length is no multiple of the
    element size is an error."""
    f32, i8, i16, i32 = b"\x00\x00\x80\x3f", b"\x00\x7f\xff", b"\x00\x00\x01\x00", b"\x00\x00\x00\x00\x01\x00\x00\x00"
    data = f32 + b"\0" * 28 + i8 + b"\0" * 29 + i16 + b"\0" * 28 + i32
    blob = build([], [tinfo("f", (1,), 0, 0), tinfo("b", (3,), 16, 32), tinfo("h", (2,), 17, 64), tinfo("w", (2,), 18, 96)], data)
    g = GGUFLoader(tmpfile(blob))
    assert g.load_f32("f").tolist() == [1.0]
    assert g.load_f32("b").tolist() == [0.0, 127.0, -1.0]
    assert g.load_f32("h").tolist() == [0.0, 1.0]
    assert g.load_f32("w").tolist() == [0.0, 1.0]
    assert all(g.load_f32(n).dtype == np.float32 for n in "fbhw")
    # three bytes where an f32 tensor of one element is declared: the read runs past the end of the file
    short = build([], [tinfo("f", (1,), 0, 0)], b"\x00\x00\x00")
    with pytest.raises(GGUFError):
        GGUFLoader(tmpfile(short)).load_f32("f")


def test_stated_alignment_is_honoured(tmpfile):
    data = b"\x00\x00\x80\x3f"
    blob = build([kv("general.alignment", 4, struct.pack("<I", 64))], [tinfo("x", (1,), 0, 0)], data, align=64)
    g = GGUFLoader(tmpfile(blob))
    assert g.alignment == 64 and g.tensor_data_offset % 64 == 0
    assert g.load_f32("x")[0] == 1.0


def test_malformed_files(tmpfile):
    with pytest.raises(GGUFError, match="magic"):
        GGUFLoader(tmpfile(build([], [], magic=0x46554746)))
    with pytest.raises(GGUFError, match="Unknown value type"):
        GGUFLoader(tmpfile(build([kv("k", 13, b"\0")], [])))
    with pytest.raises(GGUFError, match="Unknown GGML type"):
        GGUFLoader(tmpfile(build([], [tinfo("t", (4,), 999, 0)])))
    with pytest.raises(GGUFError, match="end of file"):
        GGUFLoader(tmpfile(build([kv("k", 4, b"\x01\x02\x03\x04")], [])[:-30]))
    with pytest.raises(GGUFError, match="UTF-8"):
        GGUFLoader(tmpfile(build([kv("k", 8, struct.pack("<Q", 2) + b"\xff\xfe")], [])))
    g = GGUFLoader(tmpfile(build([], [tinfo("t", (8,), 0, 0)], b"\0" * 16)))      # 32 bytes promised, 16 present
    with pytest.raises(GGUFError, match="past the end"):
        g.load_tensor_data("t")
    with pytest.raises(GGUFError, match="Failed to open"):
        GGUFLoader("/nonexistent/dir/m.gguf")
    v2 = GGUFLoader(tmpfile(build([], [], version=2)))                              # the reference only warns
    assert v2.version_mismatch and v2.header.version == 2


def test_writer_reader_round_trip(tmp_path):
    rng = np.random.default_rng(5)
    w = GGUFWriter()
    w.add_kv("general.architecture", gguf.VT_STRING, "llama")
    w.add_kv("llama.block_count", gguf.VT_UINT32, 2)
    w.add_kv("llama.rope.freq_base", gguf.VT_FLOAT32, 10000.0)
    w.add_kv("tokenizer.ggml.tokens", gguf.VT_ARRAY, (gguf.VT_STRING, ["<s>", "a", "b"]))
    payload = {}
    for name, t, dims in (("q4k", GGMLType.Q4_K, (512, 3)), ("q6k", GGMLType.Q6_K, (256, 5)), ("q80", GGMLType.Q8_0, (64, 7)),
                          ("q40", GGMLType.Q4_0, (32, 1)), ("norm", GGMLType.F32, (17,)), ("half", GGMLType.F16, (5, 3))):
        n = int(np.prod(dims[1:])) * t.row_bytes(dims[0])
        payload[name] = rng.integers(0, 256, n, dtype=np.uint8)
        w.add_tensor(name, t, dims, payload[name])
    with pytest.raises(GGUFError):
        w.add_tensor("bad", GGMLType.Q4_K, (256, 2), np.zeros(100, np.uint8))
    p = tmp_path / "rt.gguf"
    w.write(p)
    with GGUFLoader(p) as g:
        assert g.get_metadata("llama.block_count").as_u32() == 2 and g.get_metadata("llama.rope.freq_base").as_f32() == 10000.0
        assert g.get_metadata("tokenizer.ggml.tokens").as_list() == ["<s>", "a", "b"]
        for t in g.tensors:
            assert t.offset % 32 == 0
            assert np.array_equal(g.load_tensor_data(t.name), payload[t.name])
        assert g.tensor_data_offset + g.tensors[-1].offset + g.tensors[-1].n_bytes == g.file_size


def test_synthetic_llama_file_layout(tmp_path):
    from rustorch_amd import llama
    p = tmp_path / "tiny.gguf"
    llama.write_synthetic_gguf(p, 3, n_layers=2, hidden=256, n_heads=2, ffn=512, vocab=64, context=32)
    with GGUFLoader(p) as g:
        assert g.header.tensor_count == 2 * 9 + 3
        assert g.get_metadata("general.architecture").as_str() == "llama"
        assert g.find_tensor("blk.1.ffn_down.weight").dims == (512, 256) and g.find_tensor("blk.1.ffn_down.weight").ggml_type == GGMLType.Q6_K
        assert g.find_tensor("token_embd.weight").dims == (256, 64)
        want = {n: raw for n, raw in ((llama.gguf_tensor_name(s_, l), raw) for s_, l, t, r, c, raw in llama.synthetic_tensors(3, 2, 256, 512, 64))}
        for t in g.tensors:
            assert g.load_tensor_data(t.name).tobytes() == np.ascontiguousarray(want[t.name]).tobytes()
