"""The int8 wire record of peregrine::serial (reference src/serial.rs:124-222), CPU suite.
test_serialization_roundtrip restates tests/quant_parity.rs:149-173 (the quantised tensor
comes from the CPU oracle here, so no device is needed)."""
import io
import struct

import numpy as np
import pytest


@pytest.fixture(scope="module")
def S():
    from peregrine_amd import serial
    return serial


def make_qt(orc, rows, cols):
    from peregrine_amd.quant import QuantizedTensor
    data = np.array([((i * 11 + 3) % 100) / 50.0 - 1.0 for i in range(rows * cols)], np.float32)
    q, q_t, s = orc.quantize_weights(data, rows, cols)
    return QuantizedTensor(q, q_t, s, rows, cols)


def test_serialization_roundtrip(S, orc):
    rows, cols = 16, 32
    qt = make_qt(orc, rows, cols)
    buf = io.BytesIO()
    S.write_quantized_tensor(buf, "test.weight", qt)
    buf.seek(0)
    name, qt2 = S.read_quantized_tensor(buf)
    assert name == "test.weight" and (qt2.rows, qt2.cols) == (rows, cols)
    assert (qt2.data_i8 == qt.data_i8).all() and (qt2.scales.view(np.uint32) == qt.scales.view(np.uint32)).all()
    assert (qt2.data_i8_t == qt.data_i8_t).all()  # the reader rebuilds the transposed copy  src/serial.rs:202-208
    assert buf.read() == b""


def test_record_bytes_are_the_documented_layout(S, orc):
    qt = make_qt(orc, 3, 5)
    buf = io.BytesIO()
    S.write_quantized_tensor(buf, "blk.0.wq", qt)
    want = struct.pack("<I", 8) + b"blk.0.wq" + b"\x01" + struct.pack("<III", 2, 3, 5)
    want += qt.data_i8.astype(np.int8).tobytes() + qt.scales.astype("<f4").tobytes()
    assert buf.getvalue() == want


def test_several_records_in_one_stream(S, orc):
    buf = io.BytesIO()
    qts = [make_qt(orc, r, c) for r, c in ((4, 8), (1, 1), (7, 3))]
    for i, qt in enumerate(qts):
        S.write_quantized_tensor(buf, f"t{i}" * (i + 1), qt)  # name lengths 2, 4, 6: unaligned scales
    buf.seek(0)
    for i, qt in enumerate(qts):
        name, got = S.read_quantized_tensor(buf)
        assert name == f"t{i}" * (i + 1) and (got.data_i8 == qt.data_i8).all() and (got.scales == qt.scales).all()


def test_bad_records(S, orc):
    from peregrine_amd._ffi import PeregrineError
    qt = make_qt(orc, 4, 4)
    buf = io.BytesIO()
    S.write_quantized_tensor(buf, "w", qt)
    good = buf.getvalue()
    for cut in (0, 3, 5, 10, len(good) - 1):
        with pytest.raises(EOFError):
            S.read_quantized_tensor(io.BytesIO(good[:cut]))
    bad_dtype = bytearray(good)
    bad_dtype[5] = 2  # the 2:4-sparse tag
    with pytest.raises(PeregrineError, match="expected dtype=1"):
        S.read_quantized_tensor(io.BytesIO(bytes(bad_dtype)))
    bad_ndim = bytearray(good)
    bad_ndim[6:10] = struct.pack("<I", 3)
    with pytest.raises(PeregrineError, match="must be 2D"):
        S.read_quantized_tensor(io.BytesIO(bytes(bad_ndim)))
