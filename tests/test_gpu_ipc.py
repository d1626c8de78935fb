"""KV cache tensors owned by ANOTHER process: the server-side half of the
reference's RegisterContextBatch / Save / Load flow
(pegaflow-server/src/service.rs:205-540, registry.rs:45-203,
python/pegaflow/ipc_wrapper.py:102-160).

A fresh child process (tests/ipc_worker_child.py) allocates the caches and
exports them; this process opens them, registers the mapped addresses with the
engine, saves the child's blocks into the pinned pool, and, after the child has
zeroed its caches, loads them back into other block ids.  The child verifies
its own memory byte for byte and learns of the completion from the LoadState
shared-memory word it created."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest

from pegaflow_amd import _lib
from pegaflow_amd.engine import LayerSave, LoadState, PegaEngine
from pegaflow_amd.ipc import (HipIPCWrapper, TensorRegistry, context_key, device_from_uuid,
                              device_uuid, register_context_batch)
from pegaflow_amd.runtime import DeviceBuffer
from pegaflow_amd.transfer import TransferMode

pytestmark = pytest.mark.gpu

CHILD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ipc_worker_child.py")


class Worker:
    def __init__(self, layers, num_blocks, seg, nseg, seed=7):
        self.proc = subprocess.Popen(
            [sys.executable, "-u", CHILD, str(layers), str(num_blocks), str(seg), str(nseg), str(seed)],
            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
        self.hello = self.read()
        assert self.hello.get("ready"), self.hello

    def read(self):
        line = self.proc.stdout.readline()
        assert line, f"worker process ended (exit status {self.proc.poll()})"
        return json.loads(line)

    def ask(self, **cmd):
        self.proc.stdin.write(json.dumps(cmd) + "\n")
        self.proc.stdin.flush()
        return self.read()

    def close(self):
        try:
            if self.proc.poll() is None:
                self.ask(op="exit")
                self.proc.wait(timeout=20)
        finally:
            if self.proc.poll() is None:
                self.proc.kill()


def test_device_uuid_round_trip(gpu):
    uuid = device_uuid(0)
    assert len(uuid) == 16 and device_from_uuid(uuid) == 0
    with pytest.raises(_lib.InvalidArgument, match="Device UUID not found"):
        device_from_uuid(bytes(16))


def test_export_describes_the_allocation(gpu):
    buf = DeviceBuffer(3 << 20)
    whole = HipIPCWrapper(data_ptr=buf.ptr, size_bytes=3 << 20)
    inner = HipIPCWrapper(data_ptr=buf.ptr + 4096, size_bytes=1 << 20)
    assert whole.offset == 0 and inner.offset == 4096
    assert whole.handle == inner.handle and whole.alloc_size >= 3 << 20
    assert whole.device_uuid == device_uuid(0)
    assert HipIPCWrapper.from_bytes(inner.to_bytes()) == inner
    with pytest.raises(_lib.InvalidArgument, match="exceed the allocation"):
        HipIPCWrapper(data_ptr=buf.ptr + 4096, size_bytes=whole.alloc_size)
    with pytest.raises(ValueError):
        HipIPCWrapper.from_bytes(b"nonsense")
    buf.close()


@pytest.mark.parametrize("mode", [TransferMode.DIRECT, TransferMode.KERNEL, TransferMode.ZEROCOPY],
                         ids=["direct", "kernel", "zerocopy"])
def test_save_and_load_of_another_process_caches(gpu, mode):
    layers, nb, seg, nseg = 6, 1024, 32768, 2          # 64 MiB per layer, K/V split
    n = 300
    rng = np.random.default_rng(3)
    src_ids = rng.permutation(nb)[:n]
    dst_ids = rng.permutation(nb)[:n]
    names = [f"model.layers.{i}.self_attn.attn" for i in range(layers)]
    worker = Worker(layers, nb, seg, nseg)
    registry = TensorRegistry()
    engine = PegaEngine(pool_size=layers * nseg * n * seg + (64 << 20))
    try:
        wrappers = [bytes.fromhex(h) for h in worker.hello["wrappers"]]
        assert HipIPCWrapper.from_bytes(wrappers[0]).device_uuid.hex() == worker.hello["device_uuid"]
        register_context_batch(engine, registry, "ipc-inst", "ipc-ns", 0, 0, 0, 1, 1, names, wrappers,
                               [nb] * layers, [seg] * layers, [nb * seg] * layers, [nseg] * layers,
                               transfer_mode=mode)
        assert len(registry) == 1
        hashes = [b"ipc" + int(i).to_bytes(4, "little") for i in range(n)]
        engine.batch_save_kv_blocks("ipc-inst", 0, 0, 0,
                                    [LayerSave(nm, src_ids.tolist(), hashes) for nm in names])
        zeroed = worker.ask(op="zero")
        hits, lease = engine.query_prefix("ipc-inst", hashes)
        assert hits == n
        state = LoadState(attach_to=zeroed["shm"])
        engine.batch_load_kv_blocks_multi_layer("ipc-inst", 0, 0, [names], lease,
                                                [dst_ids.tolist()], state).wait()
        answer = worker.ask(op="await", src_ids=src_ids.tolist(), dst_ids=dst_ids.tolist())
        assert answer["state"] == 1, answer
        assert answer["ok"], answer["problems"]
        state.close()

        # registry.rs:73-77: the same context cannot be registered twice
        with pytest.raises(_lib.InvalidArgument,
                           match=f"context {context_key('ipc-inst', 0, 0, 0)} is already registered"):
            register_context_batch(engine, registry, "ipc-inst", "ipc-ns", 0, 0, 0, 1, 1, names,
                                   wrappers, [nb] * layers, [seg] * layers, [nb * seg] * layers,
                                   [nseg] * layers, transfer_mode=mode)
        # service.rs:326-336: a registration the engine refuses leaves no mapping behind
        with pytest.raises(_lib.PegaHipError):
            register_context_batch(engine, registry, "ipc-other", "ipc-ns", 0, 0, 0, 1, 1, names,
                                   wrappers, [nb * 4] * layers, [seg] * layers, [nb * seg] * layers,
                                   [nseg] * layers, transfer_mode=mode)
        assert len(registry) == 1
        engine.unregister_instance("ipc-inst")
        assert registry.drop_instance("ipc-inst") == layers
        assert len(registry) == 0 and registry.drop_instance("ipc-inst") == 0
    finally:
        engine.close()
        registry.close()
        worker.close()


def test_registry_rejections(gpu):
    """registry.rs:73-101 without a second process: duplicate layer names and a
    record whose GPU this process does not have."""
    buf = DeviceBuffer(1 << 20)
    w = HipIPCWrapper(data_ptr=buf.ptr, size_bytes=1 << 20)
    registry = TensorRegistry()
    with pytest.raises(_lib.InvalidArgument, match="layer a appears more than once in context k"):
        registry.register_layers("k", 0, [("a", w), ("a", w)])
    stranger = HipIPCWrapper.from_bytes(w.to_bytes())
    stranger.device_uuid = bytes(range(16))
    with pytest.raises(_lib.InvalidArgument, match="Device UUID not found"):
        registry.register_layers("k", 0, [("a", stranger)])
    assert len(registry) == 0
    registry.close()
    buf.close()
