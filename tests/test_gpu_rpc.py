"""The gRPC boundary end to end: this process is the engine server
(pegaflow-server/src/service.rs:205-809 over PegaEngine + TensorRegistry), a
fresh child process (tests/rpc_worker_child.py) is the worker that owns the KV
caches and drives RegisterContextBatch / Save / QueryPrefetch / Load / Release /
UnregisterContext through the client, then verifies its own memory."""

import json
import os
import subprocess
import sys

import pytest

from pegaflow_amd.engine import PegaEngine

pytestmark = pytest.mark.gpu

CHILD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "rpc_worker_child.py")


@pytest.mark.parametrize("backend", ["direct", "kernel"])
def test_worker_process_saves_and_loads_through_grpc(gpu, backend):
    from pegaflow_amd import rpc
    layers, nb, seg, nseg, n = 4, 512, 32768, 2, 120
    engine = PegaEngine(pool_size=layers * nseg * n * seg + (64 << 20))
    server, service, port = rpc.serve(engine, "127.0.0.1:0")
    try:
        proc = subprocess.run(
            [sys.executable, "-u", CHILD, str(port), str(layers), str(nb), str(seg), str(nseg), str(n),
             backend], capture_output=True, text=True, timeout=150)
        assert proc.returncode == 0, proc.stderr[-3000:]
        out = json.loads([ln for ln in proc.stdout.splitlines() if ln.startswith("{")][-1])
        assert out["health"] == [True, ""]
        assert out["register"] == [True, ""] and out["save"] == [True, ""]
        assert "already registered" in out["second_register"]
        assert out["bad_save"].startswith("block_ids length 2 does not match block_hashes 1 for layer")
        assert out["query"] == ["QueryReady", n, 16, []]          # the trailing miss ends the prefix
        assert out["load"] == [True, ""] and out["load_state"] == 1
        assert out["problems"] == []
        assert out["release_consumed"] == "query lease is unknown or expired"
        assert out["released"] == ["QueryReady", 3]
        assert out["bad_lease"] == "query lease id must be 16 bytes, got 5"
        assert out["unregister"] == [True, ""]
        assert len(service.registry) == 0
    finally:
        server.stop(grace=None)
        service.close()
        service.registry.close()
        engine.close()


def test_reference_rpc_scenarios(gpu):
    """The cases of pegaflow-server/tests/mock_vllm_rpc_e2e.rs (line numbers
    below), run by tests/rpc_scenarios_child.py against this process's server."""
    from pegaflow_amd import rpc
    scenarios = os.path.join(os.path.dirname(os.path.abspath(__file__)), "rpc_scenarios_child.py")
    engine = PegaEngine(pool_size=64 << 20)
    server, service, port = rpc.serve(engine, "127.0.0.1:0")
    try:
        proc = subprocess.run([sys.executable, "-u", scenarios, str(port)], capture_output=True,
                              text=True, timeout=150)
        assert proc.returncode == 0, proc.stderr[-3000:]
        out = json.loads([ln for ln in proc.stdout.splitlines() if ln.startswith("{")][-1])
        ok = [True, ""]
        # :26-77 save / query / load round trip
        assert out["register"] == ok and out["save"] == ok
        assert out["cold_query"] == ["QueryReady", 0, 0]
        assert out["empty_query"] == ["QueryReady", 0, True]
        assert out["hit_query"] == ["QueryReady", 4, 16]
        assert out["load"] == [ok, 1] and out["roundtrip_matches"]
        # :79-96
        assert out["empty_req_id"] == ["INVALID_ARGUMENT", "req_id must not be empty"]
        # :98-131 a lease is bound to its instance; the refused load settles its LoadState as an error
        code, message = out["wrong_instance_load"][0]
        assert "query lease belongs to instance" in message and out["wrong_instance_load"][1] < 0
        # :133-171
        assert out["first_release"] == ["accepted", ""]
        assert out["second_release"] == ["FAILED_PRECONDITION", "query lease is unknown or expired"]
        # :173-201 a partial prefix gives a lease over the prefix
        assert out["prefix_save"] == ok and out["prefix_query"] == ["QueryReady", 2, 16]
        assert out["prefix_load"] == [ok, 1] and out["prefix_loaded_suffix_zero"]
        # :203-240
        assert out["mismatch_hits"] == 2
        code, message = out["mismatch_load"][0]
        assert code == "INVALID_ARGUMENT"
        assert "query lease block count 2 does not match destination block count 4" in message
        assert out["mismatch_load"][1] < 0
        # :318-410 (two tensor-parallel workers) needs two GPUs; the reference skips it below two
        # :242-316 the end of the liveness stream drops the instance
        assert out["session_save"] == ok and out["session_hits"] == 4
        for key in ("session_cleanup_probe", "session_save_after_cleanup"):
            assert out[key][0] == "FAILED_PRECONDITION", out[key]
            assert "instance mock-vllm-rpc-e2e-session not found" in out[key][1], out[key]
        code, message = out["session_load_after_cleanup"][0]
        assert code == "FAILED_PRECONDITION" and "not found" in message
        assert out["session_load_after_cleanup"][1] < 0
        assert out["first_instance_still_hits"] == 4
    finally:
        server.stop(grace=None)
        service.close()
        service.registry.close()
        engine.close()


def test_killed_worker_releases_its_tensors(gpu, tmp_path):
    """python/tests/test_session_watcher.py:50-99: a worker that dies without
    unregistering (SIGKILL) closes its liveness stream with its socket; the
    server then drops the instance's mapped tensors and its registration."""
    import signal
    import time
    from pegaflow_amd import _lib, rpc
    child = os.path.join(os.path.dirname(os.path.abspath(__file__)), "rpc_crash_child.py")
    engine = PegaEngine(pool_size=16 << 20)
    server, service, port = rpc.serve(engine, "127.0.0.1:0")
    instance = f"inst-crash-{os.getpid()}"
    ready = tmp_path / "ready"
    worker = subprocess.Popen([sys.executable, "-u", child, str(port), instance, str(ready)],
                              stdout=subprocess.PIPE, stderr=subprocess.PIPE)
    try:
        deadline = time.monotonic() + 60
        while not ready.exists():
            assert worker.poll() is None, worker.stderr.read().decode(errors="replace")[-2000:]
            assert time.monotonic() < deadline, "worker did not become ready"
            time.sleep(0.05)
        assert len(service.registry) == 1
        assert engine.query_prefix(instance, [b"crash-a", b"crash-b"])[0] == 2
        worker.send_signal(signal.SIGKILL)
        worker.wait(timeout=5)
        deadline = time.monotonic() + 10
        while len(service.registry) != 0 and time.monotonic() < deadline:
            time.sleep(0.05)
        assert len(service.registry) == 0, "the dead worker's tensors are still mapped"
        with pytest.raises(_lib.InstanceMissing, match=f"instance {instance} not found"):
            engine.query_prefix(instance, [b"crash-a"])
    finally:
        if worker.poll() is None:
            worker.kill()
            worker.wait(timeout=5)
        server.stop(grace=None)
        service.close()
        service.registry.close()
        engine.close()
