"""Runs the C++ parity program (tests/cpp/quant_parity.cpp) built on the C++ host mirror
include/peregrine_hip.hpp; its cases follow the reference's tests/quant_parity.rs and
tests/gguf_parity.rs.  The binary is built by __graft_entry__.build() (tests/cpp/Makefile)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "_build", "quant_parity")


@pytest.mark.gpu
def test_cpp_host_mirror_parity():
    if not os.path.exists(BIN):
        pytest.fail(f"{BIN} is not built: run __graft_entry__.build()")
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=110)
    print(r.stdout[-4000:], r.stderr[-2000:])
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "OK: all checks passed" in r.stdout
