"""GPU half of the GGUF container mirror: GgufFile::load_tensor_f32 / load_tensor_q8
(reference src/gguf.rs:485-537) and the keep-quantised upload, against the CPU oracle."""
import sys

import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def build(orc):
    rng = np.random.default_rng(1)
    n_out, k_in = 48, 256
    w = orc.rng_normal(77, n_out * k_in, 0.0, 0.02)
    f32 = orc.rng_normal(78, 5 * 7)
    f16 = np.arange(0, 4096, 7, dtype=np.uint16)  # raw half patterns incl. subnormals
    q41 = rng.integers(0, 256, size=(n_out * k_in // 32, 20), dtype=np.uint8)
    q41[:, 1] = 0x2C  # keep d and m finite
    q41[:, 3] = 0x30
    tensors = [
        ("f32", 0, [7, 5], f32.tobytes()),
        ("f16", 1, [f16.size], f16.tobytes()),
        ("q8", 8, [k_in, n_out], bytes(H.pack_q8_0(w))),
        ("q4", 2, [k_in, n_out], bytes(H.pack_q4_0(w))),
        ("q41", 3, [k_in, n_out], q41.tobytes()),
        ("vec", 8, [64], bytes(H.pack_q8_0(w[:64]))),
    ]
    data, _, _ = H.build_gguf([("general.architecture", "str", "llama")], tensors)
    return data, {t[0]: t for t in tensors}, (n_out, k_in), f32, f16


def test_load_tensor_f32_every_type(ctx, orc):
    from peregrine_amd import gguf
    print("gguf file: load_tensor_f32", flush=True)
    data, T, (n_out, k_in), f32, f16 = build(orc)
    f = gguf.GgufFile.parse(data)
    assert (bits(f.load_tensor_f32("f32", ctx)) == bits(f32)).all()
    want16 = orc.f16_to_f32_bits(f16)
    assert (bits(f.load_tensor_f32("f16", ctx)) == want16).all()
    n = n_out * k_in
    assert (bits(f.load_tensor_f32("q8", ctx)) == bits(orc.dequant_q8_0(T["q8"][3], n))).all()
    assert (bits(f.load_tensor_f32("q4", ctx)) == bits(orc.dequant_q4_0(T["q4"][3], n))).all()
    assert (bits(f.load_tensor_f32("q41", ctx)) == bits(orc.dequant_q4_1(T["q41"][3], n))).all()
    from peregrine_amd._ffi import PeregrineError
    with pytest.raises(PeregrineError, match="not found in GGUF file"):
        f.load_tensor_f32("missing", ctx)


def test_load_tensor_q8_matches_reference_composition(ctx, orc):
    from peregrine_amd import gguf
    print("gguf file: load_tensor_q8", flush=True)
    data, T, (n_out, k_in), _, _ = build(orc)
    f = gguf.GgufFile.parse(data)
    qt = f.load_tensor_q8("q8", ctx)  # (rows, cols) = (shape[1], shape[0])  src/gguf.rs:530-534
    assert (qt.rows, qt.cols) == (n_out, k_in)
    q, q_t, s = orc.quantize_weights(orc.dequant_q8_0(T["q8"][3], n_out * k_in), n_out, k_in)
    assert (qt.data_i8 == q).all() and (qt.data_i8_t == q_t).all() and (bits(qt.scales) == bits(s)).all()
    v = f.load_tensor_q8("vec", ctx)  # 1-D: one row
    assert (v.rows, v.cols) == (1, 64)


def test_upload_tensor_keeps_blocks_quantised(ctx, orc):
    from peregrine_amd import gguf
    print("gguf file: upload_tensor + matmul", flush=True)
    data, T, (n_out, k_in), _, _ = build(orc)
    f = gguf.GgufFile.parse(data)
    for name, typ in (("q8", 8), ("q4", 2)):
        w = f.upload_tensor(name, ctx)
        assert (w.n_out, w.k_in, w.ggml_type) == (n_out, k_in, typ)
        for m in (1, 5):
            x = orc.rng_normal(5 + m, m * k_in)
            H.assert_close_rel(w.matmul(x, m), orc.gguf_matmul(x, m, T[name][3], typ, n_out, k_in), 4e-4, f"{name} m={m}")
        w.free()
    from peregrine_amd._ffi import PeregrineError
    with pytest.raises(PeregrineError):  # f32 tensors have no block form
        f.upload_tensor("f32", ctx)
