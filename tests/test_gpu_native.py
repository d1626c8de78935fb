"""The C ABI from native programs, built with the library (make -C
pegaflow_amd/csrc): tests/native/engine_roundtrip.cpp runs the save -> query ->
load cycle in C++ against libpegahip.so; tests/native/engine_threads.cpp drives
one engine from several threads under pool pressure.  Both check every byte
themselves."""

import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARIES = {name: os.path.join(ROOT, "tests", "native", name)
            for name in ("engine_roundtrip", "engine_threads")}


@pytest.mark.parametrize("name", sorted(BINARIES))
def test_native_binary_is_built(name):
    assert os.path.exists(BINARIES[name]), \
        f"{BINARIES[name]} is missing: build it with `make -C pegaflow_amd/csrc`"


def _run(name):
    proc = subprocess.run([BINARIES[name]], capture_output=True, text=True, timeout=300)
    tail = "\n".join(proc.stdout.splitlines()[-12:])
    assert proc.returncode == 0, f"exit {proc.returncode}\n{tail}\n{proc.stderr[-2000:]}"
    assert proc.stdout.strip().endswith("all ok"), tail
    return proc.stdout


@pytest.mark.gpu
def test_engine_roundtrip_from_cpp():
    _run("engine_roundtrip")


@pytest.mark.gpu
def test_engine_shared_by_threads_under_pool_pressure():
    out = _run("engine_threads")
    summary = [line for line in out.splitlines() if line.startswith("threads=")][-1]
    fields = dict(item.split("=") for item in summary.split())
    # loads really happened (how many queries miss depends on thread timing)
    assert int(fields["loaded"]) > 1000, summary
