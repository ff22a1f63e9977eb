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


def test_mutated_files_are_refused_or_read_without_leaving_the_buffer():
    """The file is untrusted input: a seeded series of byte flips, truncations and overwritten lengths over a
    file with every value type, nested arrays and three tensors with data.  Whatever the parser makes of one,
    an error or a parse, every accessor afterwards answers from inside the buffer (a read outside it would
    crash the test run); what parses must keep its own invariants."""
    from orangu_amd import OgmError
    rng = np.random.default_rng(20240612)
    kvs = [kv("general.architecture", 8, gstr("llama")), kv("u8", 0, struct.pack("<B", 200)),
           kv("i32", 5, struct.pack("<i", -7)), kv("f32", 6, struct.pack("<f", 1.5)), kv("bool", 7, b"\x01"),
           kv("arr", 9, u32(4) + u64(3) + u32(1) + u32(2) + u32(3)),
           kv("strs", 9, u32(8) + u64(3) + gstr("a") + gstr("bb") + gstr("ccc")),
           kv("nested", 9, u32(9) + u64(2) + (u32(0) + u64(2) + b"\x01\x02") + (u32(8) + u64(1) + gstr("x"))),
           kv("u64", 10, u64(1 << 40)), kv("f64", 12, struct.pack("<d", 1e-5)), kv("general.alignment", 4, u32(32))]
    w8 = synth_weights(Q8_0, 64, 3, seed=1)
    w4 = synth_weights(Q4_K, 256, 2, seed=2)
    data = bytes(w8) + b"\0" * ((-len(w8)) % 32) + bytes(w4) + b"\0" * ((-len(w4)) % 32) + struct.pack("<8f", *range(8))
    off4 = len(w8) + (-len(w8)) % 32
    tensors = [tensor_info("a.weight", [64, 3], Q8_0, 0), tensor_info("b.weight", [256, 2], Q4_K, off4),
               tensor_info("c", [8], 0, off4 + len(w4) + (-len(w4)) % 32)]
    good, head_len = gguf(kvs, tensors, data=data)
    g = open_bytes(good)
    assert g.n_tensors == 3 and g.matrix("b.weight")[:3] == (Q4_K, 256, 2)
    g.close()
    keys = ["general.architecture", "u8", "i32", "f32", "bool", "arr", "strs", "nested", "u64", "f64", "general.alignment"]
    parsed = refused = 0
    for trial in range(12000):
        b = bytearray(good)
        kind = trial % 4
        if kind == 0:      # a few flipped bytes in the header part
            for _ in range(int(rng.integers(1, 6))):
                b[int(rng.integers(0, head_len))] ^= int(rng.integers(1, 256))
        elif kind == 1:    # cut anywhere
            b = b[:int(rng.integers(0, len(b)))]
        elif kind == 2:    # an aligned 8-byte field overwritten with a length that cannot be
            pos = int(rng.integers(1, head_len // 8)) * 8
            vals = [0xFFFFFFFFFFFFFFFF, 1 << 63, 1 << 32, (1 << 31) + 5, len(good), len(good) - 1]
            b[pos:pos + 8] = struct.pack("<Q", vals[int(rng.integers(len(vals)))])
        else:              # the same at an arbitrary position, and a flip in the data part's offsets
            pos = int(rng.integers(4, head_len - 8))
            vals = [0xFFFFFFFFFFFFFFFF, 1 << 62, 1 << 33, 0]
            b[pos:pos + 8] = struct.pack("<Q", vals[int(rng.integers(len(vals)))])
        try:
            g = open_bytes(bytes(b))
        except OgmError:
            refused += 1
            continue
        parsed += 1
        try:
            assert g.n_tensors <= 1 << 20 and g.data_offset % max(g.alignment, 1) == 0
            for k in keys:
                g.meta_u64(k), g.meta_f64(k), g.meta_string(k), g.meta_array(k)
            for i in range(min(g.n_tensors, 8)):
                try:
                    name, dims, t, off = g.tensor(i)
                    d = g.tensor_data(i)
                    assert g.data_offset + off + d.size <= len(b)
                except OgmError:
                    pass
            for name in ("a.weight", "b.weight", "c", "nope"):
                try:
                    t, i_, o_, rb, raw = g.matrix(name)
                    assert raw.size == rb * o_
                except OgmError:
                    pass
        finally:
            g.close()
    assert parsed > 100 and refused > 100, (parsed, refused)


def test_the_model_loader_under_sanitizers_on_mutated_model_files(tmp_path):
    """ogm_gguf_parse + ogm_llama_load_gguf (read_model_config, loader.rs:1652-1714; load_with_backend,
    llama.rs:123-220) over 20 000 seeded mutations of a small model file's header, compiled with AddressSanitizer and
    UBSan beside a driver that stubs the uploads out and reads every byte range the loader hands them: no report,
    and both outcomes -- refused, and parsed as far as the model's creation -- occur."""
    import os
    import shutil
    import subprocess
    import sys
    if not shutil.which("g++"):
        pytest.skip("no host compiler")
    from oracle import llama_ref as R
    from test_gpu_llama import model_gguf
    from orangu_amd.gguf import GgufFile
    f32 = np.float32
    n_embd, n_head, n_kv, hd, n_ff, n_vocab = 256, 4, 2, 64, 256, 64
    mk = lambda i, o, s: (Q8_0, synth_weights(Q8_0, i, o, seed=s), i, o)
    L = R.Layer(mk(n_embd, n_head * hd, 1), mk(n_embd, n_kv * hd, 2), mk(n_embd, n_kv * hd, 3), mk(n_head * hd, n_embd, 4),
                mk(n_embd, n_ff, 5), mk(n_embd, n_ff, 6), mk(n_ff, n_embd, 7), np.ones(n_embd, f32), np.ones(n_embd, f32))
    L.q_bias = np.linspace(-1, 1, n_head * hd).astype(f32)
    L.q_norm = np.ones(hd, f32)
    m = R.Model(n_embd, n_head, n_kv, hd, n_ff, n_vocab, hd, 1e-5, 10000.0, [L], np.ones(n_embd, f32), mk(n_embd, n_vocab, 9),
                rope_freq_factors=np.linspace(1, 2, hd // 2).astype(f32))
    blob = model_gguf(m, "llama", tok_embd=mk(n_embd, n_vocab, 10))
    g = GgufFile(data=blob)
    head = g.data_offset
    g.close()
    path = tmp_path / "model.gguf"
    path.write_bytes(blob)
    here = os.path.dirname(os.path.abspath(__file__))
    exe = str(tmp_path / "gguf_fuzz")
    subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
                    "-o", exe, os.path.join(here, "gguf_fuzz_driver.cpp"),
                    os.path.join(here, "..", "orangu_amd", "csrc", "ogm_gguf.cpp")], check=True)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")   # (a failed load leaves its uploads to ogm_destroy; the stubs' are never freed)
    r = subprocess.run([exe, str(head), "20000", str(path)], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-4000:])
    import re
    mo = re.search(r"parsed (\d+) refused (\d+), loader errors (\d+), uploads (\d+), creates reached (\d+)", r.stdout)
    assert mo, r.stdout
    parsed, refused, _, uploads, creates = map(int, mo.groups())
    assert parsed > 1000 and refused > 1000 and uploads > parsed and creates > 100, r.stdout
