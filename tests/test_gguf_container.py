"""GGUF container parsing (gguf::GgufFile, reference src/gguf.rs:403-561) through the C ABI.
No device is needed: these run in the CPU suite.  The first two cases are the reference's
own (tests/gguf_parity.rs:78-105); the rest pin every metadata type, the tensor directory,
the alignment rule and the behaviour on malformed files."""
import ctypes as C
import os
import struct

import numpy as np
import pytest

import helpers as H


@pytest.fixture(scope="module")
def G():
    from peregrine_amd import gguf
    return gguf


def test_gguf_invalid_magic(G):  # tests/gguf_parity.rs:78-84
    from peregrine_amd._ffi import PeregrineError
    with pytest.raises(PeregrineError, match="invalid GGUF magic"):
        G.GgufFile.parse(bytes(64))


def test_gguf_minimal_valid(G):  # tests/gguf_parity.rs:86-105
    data = struct.pack("<IIQQ", 0x46554747, 3, 0, 0)
    data += bytes(64 - len(data))
    f = G.GgufFile.parse(data)
    assert f.n_metadata == 0 and f.tensors == {} and f.version == 3 and f.data_start == 32


@pytest.mark.parametrize("version,ok", [(1, False), (2, True), (3, True), (4, False)])
def test_gguf_versions(G, version, ok):  # src/gguf.rs:422-428
    from peregrine_amd._ffi import PeregrineError
    data, _, _ = H.build_gguf([], [], version=version)
    if ok:
        assert G.GgufFile.parse(data).version == version
    else:
        with pytest.raises(PeregrineError, match="unsupported GGUF version"):
            G.GgufFile.parse(data)


META = [
    ("a.u8", "u8", 200), ("a.i8", "i8", -5), ("a.u16", "u16", 60000), ("a.i16", "i16", -1234),
    ("llama.block_count", "u32", 32), ("a.i32", "i32", -7), ("llama.rope.freq_base", "f32", 500000.0),
    ("a.bool", "bool", 1), ("general.architecture", "str", "llama"), ("a.u64", "u64", 8192), ("a.i64", "i64", 4096),
    ("a.f64", "f64", 1e-5), ("tokenizer.ggml.tokens", "arr", ("str", ["<s>", "</s>", "héllo", ""])),
    ("tokenizer.ggml.scores", "arr", ("f32", [0.0, -1.5, 2.25])), ("tokenizer.ggml.token_type", "arr", ("i32", [1, -3, 6])),
    ("nested", "arr", ("arr", [("u8", [1, 2]), ("u8", [3])])),
]


def test_gguf_metadata_every_type(G):
    data, _, _ = H.build_gguf(META, [])
    f = G.GgufFile.parse(data)
    assert f.n_metadata == len(META)
    # as_u32: Uint32, Int32 (as u32), Uint64, Int64 only  (src/gguf.rs:77-85)
    assert f.get_u32("llama.block_count") == 32 and f.get_u32("a.u64") == 8192 and f.get_u32("a.i64") == 4096
    assert f.get_u32("a.i32") == (-7) & 0xFFFFFFFF
    assert f.get_u32("a.u8") is None and f.get_u32("a.u16") is None and f.get_u32("missing") is None
    assert f.get_u32("general.architecture") is None
    # as_f32: Float32, Float64 (src/gguf.rs:87-93)
    assert f.get_f32("llama.rope.freq_base") == 500000.0 and f.get_f32("a.f64") == np.float32(1e-5)
    assert f.get_f32("llama.block_count") is None
    assert f.get_str("general.architecture") == "llama" and f.get_str("a.u8") is None
    assert f.get_array("tokenizer.ggml.tokens") == ["<s>", "</s>", "héllo", ""]
    assert f.get_array("tokenizer.ggml.scores") == [0.0, -1.5, 2.25]
    assert f.get_array("tokenizer.ggml.token_type") == [1, -3, 6]
    assert f.get_array("a.u8") is None and f.get_array("missing") is None


def _tensors():
    rng = np.random.default_rng(0)
    f32 = rng.standard_normal(6 * 4).astype(np.float32)
    f16 = rng.standard_normal(10).astype(np.float16)
    w = rng.standard_normal(3 * 64).astype(np.float32)
    return [
        ("token_embd.weight", 0, [4, 6], f32.tobytes()),
        ("norm.weight", 1, [10], f16.tobytes()),
        ("blk.0.attn_q.weight", 8, [64, 3], bytes(H.pack_q8_0(w))),
        ("blk.0.ffn_up.weight", 2, [64, 3], bytes(H.pack_q4_0(w))),
        ("blk.0.q4_1", 3, [32, 2], bytes(range(40))),
    ]


def test_gguf_tensor_directory_and_alignment(G):
    tensors = _tensors()
    for meta, align in (([], 32), ([("general.alignment", "u32", 64)], 64), ([("general.alignment", "u64", 256)], 256)):
        data, data_start, offsets = H.build_gguf(meta, tensors)
        f = G.GgufFile.parse(data)
        assert f.data_start == data_start and data_start % align == 0
        assert f.tensor_names() == [t[0] for t in tensors]  # file order
        for name, typ, shape, raw in tensors:
            t = f.tensors[name]
            assert (t.dtype, t.shape, t.data_offset, t.data_size()) == (typ, shape, offsets[name], len(raw))
            assert f.tensor_shape(name) == list(reversed(shape))  # src/gguf.rs:551-556
            ptr, size = C.c_void_p(), C.c_size_t()
            from peregrine_amd import _ffi
            _ffi.check(_ffi.lib.pg_gguf_file_tensor_info(f._h, name.encode(), None, None, None, 0, None, C.byref(size), C.byref(ptr)))
            assert C.string_at(ptr, size.value) == raw
        assert f.tensors["blk.0.attn_q.weight"].num_elements() == 192
        with pytest.raises(KeyError):
            f.tensor_shape("nope")


def test_gguf_malformed_files_are_errors_not_crashes(G):
    from peregrine_amd._ffi import PeregrineError
    data, data_start, _ = H.build_gguf(META[:6] + META[8:9] + META[12:13], _tensors())
    for cut in list(range(0, 24)) + list(range(24, data_start - 32, 7)):  # (the last < 32 bytes may be padding)
        with pytest.raises(PeregrineError):  # any cut inside the header
            G.GgufFile.parse(data[:cut])
    for cut in range(data_start - 32, data_start):  # header or padding: an error or a clean parse, never a crash
        try:
            G.GgufFile.parse(data[:cut])
        except PeregrineError:
            pass
    f = G.GgufFile.parse(data[: data_start + 8])  # header intact, data section cut short
    from peregrine_amd import _ffi
    size = C.c_size_t()
    assert _ffi.lib.pg_gguf_file_tensor_info(f._h, b"token_embd.weight", None, None, None, 0, None, C.byref(size), None) != 0
    assert "extends past the end" in _ffi.lib.pg_last_error().decode()
    bad_type, _, _ = H.build_gguf([], [("x", 12, [32], bytes(32))])  # Q3_K: not supported (src/gguf.rs:453-455)
    with pytest.raises(PeregrineError, match="unsupported GGML type 12"):
        G.GgufFile.parse(bad_type)
    bad_meta = struct.pack("<IIQQ", 0x46554747, 3, 0, 1) + struct.pack("<Q", 1) + b"k" + struct.pack("<I", 13) + bytes(16)
    with pytest.raises(PeregrineError):  # unknown metadata value type (the reference panics)
        G.GgufFile.parse(bad_meta)
    huge_arr = struct.pack("<IIQQ", 0x46554747, 3, 0, 1) + struct.pack("<Q", 1) + b"k" + struct.pack("<IIQ", 9, 0, 1 << 60)
    with pytest.raises(PeregrineError):  # array length far beyond the file
        G.GgufFile.parse(huge_arr)
    # a large but honest array (1 M empty strings = 8 MB of length fields) parses; the same count with the
    # last length field cut, or a count the file cannot hold, is an error -- and neither reserves
    # room for the claimed count up front
    big = struct.pack("<IIQQ", 0x46554747, 3, 0, 1) + struct.pack("<Q", 1) + b"k" + struct.pack("<IIQ", 9, 8, 1 << 20) + bytes(8 << 20)
    G.GgufFile.parse(big)
    forged = big[:-1]
    with pytest.raises(PeregrineError):
        G.GgufFile.parse(forged)
    # an F32 tensor whose element count times 4 wraps 64 bits: larger than the file, not "0 bytes"
    wrap, _, _ = H.build_gguf([], [("w", 0, [1 << 62], bytes(64))])
    gw = G.GgufFile.parse(wrap)
    assert _ffi.lib.pg_gguf_file_tensor_info(gw._h, b"w", None, None, None, 0, None, C.byref(size), None) != 0
    assert "larger than the file" in _ffi.lib.pg_last_error().decode()
    not_div, _, _ = H.build_gguf([], [("x", 8, [33], bytes(68))])
    g = G.GgufFile.parse(not_div)
    assert _ffi.lib.pg_gguf_file_tensor_info(g._h, b"x", None, None, None, 0, None, C.byref(size), None) != 0
    assert "not divisible by block size" in _ffi.lib.pg_last_error().decode()  # src/gguf.rs:160


def test_gguf_load_maps_the_file(G, tmp_path):
    tensors = _tensors()
    data, data_start, offsets = H.build_gguf(META, tensors)
    path = tmp_path / "tiny.gguf"
    path.write_bytes(data)
    f = G.GgufFile.load(path)
    assert f.tensor_names() == [t[0] for t in tensors] and f.get_str("general.architecture") == "llama"
    f.close()
    from peregrine_amd._ffi import PeregrineError
    with pytest.raises(PeregrineError, match="cannot open"):
        G.GgufFile.load(tmp_path / "missing.gguf")
