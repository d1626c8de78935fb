"""The C ABI from a native program: tests/native/engine_roundtrip.cpp runs the
save -> query -> load cycle in C++ against libpegahip.so and checks every byte
itself.  The binary is built with the library (make -C pegaflow_amd/csrc)."""

import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "tests", "native", "engine_roundtrip")


def test_native_binary_is_built():
    assert os.path.exists(BINARY), \
        f"{BINARY} is missing: build it with `make -C pegaflow_amd/csrc`"


@pytest.mark.gpu
def test_engine_roundtrip_from_cpp():
    proc = subprocess.run([BINARY], capture_output=True, text=True, timeout=300)
    tail = "\n".join(proc.stdout.splitlines()[-12:])
    assert proc.returncode == 0, f"exit {proc.returncode}\n{tail}\n{proc.stderr[-2000:]}"
    assert proc.stdout.strip().endswith("all ok"), tail
