"""A worker that registers a KV cache, opens its liveness session and then
waits to be killed (tests/test_gpu_rpc.py::test_killed_worker_releases_its_tensors,
after the reference's python/tests/test_session_watcher.py:50-99 and
session_crash_helper.py)."""

import os
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def main():
    port, instance_id, ready_file = int(sys.argv[1]), sys.argv[2], sys.argv[3]
    from pegaflow_amd import runtime
    from pegaflow_amd.ipc import HipIPCWrapper
    from pegaflow_amd.rpc import EngineRpcClient
    from pegaflow_amd.runtime import DeviceBuffer

    runtime.set_device(0)
    buf = DeviceBuffer(4 * 1024)
    client = EngineRpcClient(f"http://127.0.0.1:{port}")
    ok, message = client.register_context_batch(
        instance_id, "crash-ns", 0, 0, 1, 1, 0, ["layer_0"],
        [HipIPCWrapper(data_ptr=buf.ptr, size_bytes=4 * 1024).to_bytes()], [4], [1024], [0], [1],
        "direct", False)
    assert ok, message
    client.start_session_watcher(instance_id, "crash-ns", 1, 1)
    client.save(instance_id, 0, 0, 0, [("layer_0", [0, 1], [b"crash-a", b"crash-b"])])
    with open(ready_file, "w") as f:
        f.write("ready")
    time.sleep(600)


if __name__ == "__main__":
    main()
