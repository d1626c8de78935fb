"""The worker pool's two directions at once, in a process that holds only
engine worker pools (tests/duplex_child.py): what GpuWorkerPool does at spawn
to keep its streams on hardware queues of their own and to make the link copies
of the two directions overlap (pf_worker.cpp: separate_worker_queues,
prime_copy_overlap) is checked here by its outcome.  Bytes, stream counts and
"both tasks were in flight at the same time" are assertions; rates and the
placement of streams on hardware queues depend on the box and on what else the
runtime has mapped, so a miss there is a recorded warning, not a failure (the
figures with their yardstick are in bench.py's `duplex` and `engine` keys)."""

import json
import os
import subprocess
import sys
import warnings

import pytest

pytestmark = pytest.mark.gpu

CHILD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "duplex_child.py")


@pytest.mark.parametrize("copies", ["in_order", "side"])
def test_two_pools_overlap_and_move_both_directions_at_once(gpu, copies):
    """`side`: the same with pf_engine_config.side_copy_streams, a second
    stream per worker for the link copies (worker_stream_report counts the
    worker streams in both forms)."""
    proc = subprocess.run([sys.executable, "-u", CHILD, "32", copies], capture_output=True,
                          text=True, timeout=170)
    assert proc.returncode == 0, proc.stderr[-3000:]
    out = json.loads([ln for ln in proc.stdout.splitlines() if ln.startswith("{")][-1])
    print(json.dumps(out))
    # the bytes: what the load delivered while a save was running beside it
    assert out["problems"] == []
    # two instances = two pools = four worker streams, all of them probed
    assert out["two_pools"]["streams"] == 4 and out["two_pools"]["skipped"] == 0
    # a third pool makes six worker streams
    assert out["three_pools"]["streams"] == 6
    # the save and the load of every repetition were in flight at the same time
    assert all(r["in_flight_together"] for r in out["concurrent_save_and_load"])
    # Box-dependent outcomes, recorded but not gating: each of the four streams on a
    # hardware queue of its own; six streams on four queues reported as sharing; one
    # direction alone moves ~56 GB/s and two plain hipMemcpyAsync streams ~97 together.
    notes = []
    if out["two_pools"]["clashing_pairs"] != 0:
        notes.append(f"two pools: {out['two_pools']['clashing_pairs']} worker-stream pairs share a "
                     "hardware queue")
    if out["three_pools"]["clashing_pairs"] < 2:
        notes.append("three pools: fewer than 2 clashing pairs reported for 6 streams")
    worst = min(r["aggregate_gbps"] for r in out["concurrent_save_and_load"])
    if worst < 75.0:
        notes.append(f"save and load together moved {worst} GB/s in the slowest repetition")
    for note in notes:
        warnings.warn("duplex outcome below what was measured on MI355X: " + note)
