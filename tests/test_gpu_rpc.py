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
        assert out["query"] == ["ready", n, 16, []]          # the trailing miss ends the prefix
        assert out["load"] == [True, ""] and out["load_state"] == 1
        assert out["problems"] == []
        assert out["release_consumed"] == "query lease is unknown or expired"
        assert out["released"] == ["ready", 3]
        assert out["bad_lease"] == "query lease id must be 16 bytes, got 5"
        assert out["unregister"] == [True, ""]
        assert len(service.registry) == 0
    finally:
        server.stop(grace=None)
        service.close()
        service.registry.close()
        engine.close()
