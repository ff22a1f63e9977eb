"""The GGUF reader (ogm_gguf_*) against the behaviour src/gguf.rs and engine/loader.rs pin in their own
tests: header, metadata value types, tensor table, alignment, data offset, matrix validation.
Parsing needs no GPU."""
import struct

import numpy as np
import pytest

from helpers import Q4_K, Q6_K, Q8_0, synth_weights

u32 = lambda v: struct.pack("<I", v)
u64 = lambda v: struct.pack("<Q", v)
gstr = lambda s: u64(len(s.encode())) + s.encode()


def kv(key, vtype, payload):
    return gstr(key) + u32(vtype) + payload


def tensor_info(name, dims, ggml_type, offset):
    return gstr(name) + u32(len(dims)) + b"".join(u64(d) for d in dims) + u32(ggml_type) + u64(offset)


def gguf(kvs, tensors, version=3, data=b"", alignment=32):
    head = b"GGUF" + u32(version) + u64(len(tensors)) + u64(len(kvs)) + b"".join(kvs) + b"".join(tensors)
    pad = (-len(head)) % alignment
    return head + b"\0" * pad + data, len(head)


def minimal():
    """The file src/gguf.rs:543-575 builds for its tests."""
    kvs = [kv("general.architecture", 8, gstr("llama")),
           kv("tokenizer.ggml.tokens", 9, u32(8) + u64(3) + gstr("a") + gstr("b") + gstr("c"))]
    return gguf(kvs, [tensor_info("weight", [2, 4], 0, 0)])


def open_bytes(b):
    from orangu_amd.gguf import GgufFile
    return GgufFile(data=b)


def test_parses_header_metadata_and_tensors():
    """src/gguf.rs:582-610."""
    b, head_len = minimal()
    g = open_bytes(b)
    assert g.version == 3 and g.n_tensors == 1 and g.n_metadata == 2
    assert g.meta_string("general.architecture") == "llama"
    assert g.meta_array("tokenizer.ggml.tokens") == (8, 3)
    assert g.tensor(0) == ("weight", [2, 4], 0, 0)
    assert g.find_tensor("weight") == 0 and g.find_tensor("nope") == -1
    assert g.alignment == 32
    assert g.data_offset == (head_len + 31) // 32 * 32
    g.close()


def test_the_parser_stops_at_the_end_of_the_tensor_table():
    """src/gguf.rs:624-640: nothing behind the table is needed to parse it."""
    b, head_len = minimal()
    g = open_bytes(b[:head_len])          # not even the alignment padding
    assert g.n_tensors == 1
    g.close()


def test_rejects_bad_magic_truncation_and_old_versions():
    """src/gguf.rs:685-698 and :223-227."""
    from orangu_amd import OgmError
    b, head_len = minimal()
    with pytest.raises(OgmError, match="bad magic"):
        open_bytes(b"X" + b[1:])
    with pytest.raises(OgmError, match="unexpected end of file"):
        open_bytes(b[:head_len - 10])
    v1, _ = gguf([], [], version=1)
    with pytest.raises(OgmError, match="not supported"):
        open_bytes(v1)
    with pytest.raises(OgmError, match="unknown GGUF metadata value type"):
        open_bytes(gguf([kv("k", 13, b"")], [])[0])
    with pytest.raises(OgmError, match="exceeds the limit"):
        open_bytes(gguf([kv("k", 8, u64(1 << 40))], [])[0])


def test_every_value_type_and_the_alignment_key():
    """Value type ids 0..12 (src/gguf.rs:386-415); as_u64 takes unsigned, non-negative signed and bool
    (:70-83); general.alignment replaces 32 only when positive (:258-263)."""
    kvs = [kv("u8", 0, struct.pack("<B", 200)), kv("i8", 1, struct.pack("<b", -3)),
           kv("u16", 2, struct.pack("<H", 60000)), kv("i16", 3, struct.pack("<h", 123)),
           kv("u32", 4, u32(4096)), kv("i32", 5, struct.pack("<i", -7)),
           kv("f32", 6, struct.pack("<f", 500000.0)), kv("bool", 7, b"\x01"),
           kv("str", 8, gstr("héllo")), kv("arr", 9, u32(4) + u64(3) + u32(1) + u32(2) + u32(3)),
           kv("nested", 9, u32(9) + u64(2) + (u32(0) + u64(2) + b"\x01\x02") + (u32(8) + u64(1) + gstr("x"))),
           kv("u64", 10, u64(1 << 40)), kv("i64", 11, struct.pack("<q", 9)), kv("f64", 12, struct.pack("<d", 1e-5)),
           kv("general.alignment", 4, u32(64))]
    b, head_len = gguf(kvs, [tensor_info("t", [32], 8, 0)], alignment=64)
    g = open_bytes(b)
    assert g.meta_u64("u8") == 200 and g.meta_u64("u16") == 60000 and g.meta_u64("u32") == 4096
    assert g.meta_u64("i16") == 123 and g.meta_u64("i64") == 9 and g.meta_u64("u64") == 1 << 40
    assert g.meta_u64("bool") == 1
    assert g.meta_u64("i8") is None and g.meta_u64("i32") is None and g.meta_u64("f32") is None
    assert g.meta_f64("f32") == 500000.0 and g.meta_f64("f64") == 1e-5 and g.meta_f64("i32") == -7.0
    assert g.meta_string("str") == "héllo" and g.meta_string("u8") is None
    assert g.meta_array("arr") == (4, 3) and g.meta_array("nested") == (9, 2)
    assert g.alignment == 64 and g.data_offset == (head_len + 63) // 64 * 64
    g.close()
    zero, head_len = gguf([kv("general.alignment", 4, u32(0))], [])
    g = open_bytes(zero)
    assert g.alignment == 32
    g.close()


def test_matrix_view_and_its_validation():
    """LoadedModel::matrix (engine/loader.rs:1552-1580): dims[0] is the row length, dims[1] the rows;
    the bytes are exactly the tensor's; wrong shapes and sizes are refused."""
    from orangu_amd import OgmError
    w4 = synth_weights(Q4_K, 512, 5, seed=1)
    w6 = synth_weights(Q6_K, 256, 3, seed=2)
    w8 = synth_weights(Q8_0, 96, 4, seed=3)
    norm = np.arange(8, dtype=np.float32).tobytes()
    blobs, offs, pos = [w4.tobytes(), w6.tobytes(), w8.tobytes(), norm], [], 0
    for bl in blobs:
        offs.append(pos)
        pos += (len(bl) + 31) // 32 * 32
    data = b"".join(bl + b"\0" * ((-len(bl)) % 32) for bl in blobs)
    tensors = [tensor_info("blk.0.ffn_gate.weight", [512, 5], Q4_K, offs[0]),
               tensor_info("blk.0.ffn_down.weight", [256, 3], Q6_K, offs[1]),
               tensor_info("blk.0.attn_q.weight", [96, 4], Q8_0, offs[2]),
               tensor_info("blk.0.attn_norm.weight", [8], 0, offs[3]),
               tensor_info("cube", [256, 2, 2], Q4_K, 0),
               tensor_info("ragged", [100, 2], Q4_K, 0),
               tensor_info("beyond", [256, 1000], Q4_K, offs[3])]
    b, _ = gguf([kv("general.architecture", 8, gstr("llama"))], tensors, data=data)
    g = open_bytes(b)
    t, i, o, rb, raw = g.matrix("blk.0.ffn_gate.weight")
    assert (t, i, o, rb) == (Q4_K, 512, 5, 288) and np.array_equal(raw, w4)
    t, i, o, rb, raw = g.matrix("blk.0.ffn_down.weight")
    assert (t, i, o, rb) == (Q6_K, 256, 3, 210) and np.array_equal(raw, w6)
    t, i, o, rb, raw = g.matrix("blk.0.attn_q.weight")
    assert (t, i, o, rb) == (Q8_0, 96, 4, 102) and np.array_equal(raw, w8)
    assert np.array_equal(g.tensor_data(3).view(np.float32), np.arange(8, dtype=np.float32))
    for name, msg in (("missing", "missing tensor"), ("blk.0.attn_norm.weight", "not a 2D matrix"),
                      ("cube", "not a 2D matrix"), ("ragged", "not a multiple"), ("beyond", "past the end")):
        with pytest.raises(OgmError, match=msg):
            g.matrix(name)
    g.close()


def test_open_from_a_file_at_an_offset(tmp_path):
    """GgufFile::open_at (src/gguf.rs:176-186): the structure may start inside a larger file; offsets
    stay relative to the segment."""
    from orangu_amd import OgmError
    from orangu_amd.gguf import GgufFile
    w = synth_weights(Q4_K, 256, 2, seed=4)
    b, _ = gguf([], [tensor_info("w", [256, 2], Q4_K, 0)], data=w.tobytes())
    p = tmp_path / "bundle.bin"
    p.write_bytes(b"\x7fELF" + b"\0" * 1020 + b)
    g = GgufFile(str(p), offset=1024)
    assert np.array_equal(g.matrix("w")[4], w)
    g.close()
    with pytest.raises(OgmError):
        GgufFile(str(p))                       # no GGUF at offset 0
    with pytest.raises(OgmError):
        GgufFile(str(tmp_path / "absent.gguf"))
