"""The worker pool's two directions at once, in a process that holds only
engine worker pools (tests/duplex_child.py): what GpuWorkerPool does at spawn
to keep its streams on hardware queues of their own and to make the link copies
of the two directions overlap (pf_worker.cpp: separate_worker_queues,
prime_copy_overlap) is asserted here by its outcome."""

import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

CHILD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "duplex_child.py")


def test_two_pools_overlap_and_move_both_directions_at_once(gpu):
    proc = subprocess.run([sys.executable, "-u", CHILD, "32"], capture_output=True, text=True,
                          timeout=170)
    assert proc.returncode == 0, proc.stderr[-3000:]
    out = json.loads([ln for ln in proc.stdout.splitlines() if ln.startswith("{")][-1])
    print(json.dumps(out))
    # two instances = two pools = four worker streams, each on a queue of its own
    assert out["two_pools"] == {"streams": 4, "clashing_pairs": 0, "skipped": 0}
    assert out["problems"] == []
    best = max(r["aggregate_gbps"] for r in out["concurrent_save_and_load"])
    worst = min(r["aggregate_gbps"] for r in out["concurrent_save_and_load"])
    # one direction alone moves ~56 GB/s; two plain hipMemcpyAsync streams ~97 together
    assert best >= 85.0, out["concurrent_save_and_load"]
    assert worst >= 75.0, out["concurrent_save_and_load"]
    # a third pool makes six worker streams on four hardware queues: some must share,
    # and the report says so instead of hiding it
    assert out["three_pools"]["streams"] == 6
    assert out["three_pools"]["clashing_pairs"] >= 2
