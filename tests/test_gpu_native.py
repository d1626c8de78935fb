"""The C ABI from native programs, built with the library (make -C
pegaflow_amd/csrc): tests/native/engine_roundtrip.cpp runs the save -> query ->
load cycle in C++ against libpegahip.so; tests/native/engine_threads.cpp drives
one engine from several threads under pool pressure; tests/native/
small_transfers.cpp times and checks small transfers; tests/native/cpu_path.cpp
runs the engine-level groups of the reference's cpu_path bench.  All check every
byte themselves."""

import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARIES = {name: os.path.join(ROOT, "tests", "native", name)
            for name in ("engine_roundtrip", "engine_threads", "small_transfers", "cpu_path")}


@pytest.mark.parametrize("name", sorted(BINARIES))
def test_native_binary_is_built(name):
    assert os.path.exists(BINARIES[name]), \
        f"{BINARIES[name]} is missing: build it with `make -C pegaflow_amd/csrc`"


def _run(name, *argv):
    proc = subprocess.run([BINARIES[name], *argv], capture_output=True, text=True, timeout=300)
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


@pytest.mark.gpu
def test_small_transfers_from_cpp():
    """tests/native/small_transfers.cpp: every small case moves the right bytes;
    the timings it prints are reported by bench.py --workload ref_transfer_bench."""
    import json
    out = _run("small_transfers")
    rows = json.loads([ln for ln in out.splitlines() if ln.startswith("{")][-1])["rows"]
    cases = {r["case"] for r in rows}
    assert {"block_ids_save_4MiB", "block_ids_load_4MiB", "kernel_backend_d2h_1024x4KiB",
            "noalloc_h2d_1024x4KiB"} <= cases
    assert all(r["us"] > 0 for r in rows)


@pytest.mark.gpu
def test_cpu_path_groups_from_cpp():
    """tests/native/cpu_path.cpp at its two smaller block counts: every group of
    the reference's benches/cpu_path.rs that is on the path runs, every load
    brings back the saved bytes; bench.py --workload ref_cpu_path reports the
    full table."""
    import json
    out = _run("cpu_path", "quick")
    rows = json.loads([ln for ln in out.splitlines() if ln.startswith("{")][-1])["rows"]
    groups = {r["group"] for r in rows}
    assert groups == {"save_flush_unique", "save_flush_cpu_multilayer_61",
                      "save_flush_dtoh_multilayer_61", "save_flush_transfer_fragmentation",
                      "load_transfer_fragmentation", "query_prefetch_lease", "load_submit_wait"}
    assert all(r["mean_us"] > 0 for r in rows)
