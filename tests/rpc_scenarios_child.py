"""Worker-process half of tests/test_gpu_rpc.py::test_reference_rpc_scenarios:
the cases of the reference's pegaflow-server/tests/mock_vllm_rpc_e2e.rs, driven
through EngineRpcClient against the server in the parent process.  A "mock
vLLM" here is what it is there: one layer `layer_0` of 4 blocks x 1024 bytes,
block i filled with byte (i % 251) + 1, hashes salt || u32le(i).  Every scenario
uses an instance of its own; the outcome of each goes into one JSON line."""

import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

BLOCKS, BLOCK_BYTES, LAYER = 4, 1024, "layer_0"


def hashes(salt, n=BLOCKS):
    return [bytes([salt]) + int(i).to_bytes(4, "little") for i in range(n)]


def main():
    port = int(sys.argv[1])
    import numpy as np
    from pegaflow_amd import runtime
    from pegaflow_amd.engine import LoadState
    from pegaflow_amd.ipc import HipIPCWrapper
    from pegaflow_amd.rpc import EngineRpcClient, PegaFlowError, RpcRejected
    from pegaflow_amd.runtime import DeviceBuffer

    runtime.set_device(0)
    expected = np.repeat(((np.arange(BLOCKS) % 251) + 1).astype(np.uint8), BLOCK_BYTES)
    client = EngineRpcClient(f"http://127.0.0.1:{port}")

    class Gpu:
        def __init__(self):
            self.buf = DeviceBuffer(BLOCKS * BLOCK_BYTES)
            self.buf.copy_from_host(expected)
            self.wrapper = HipIPCWrapper(data_ptr=self.buf.ptr, size_bytes=BLOCKS * BLOCK_BYTES).to_bytes()

        def zero(self):
            self.buf.fill(0)

        def matches_expected(self):
            return bool(np.array_equal(self.buf.copy_to_host(), expected))

        def prefix_loaded_suffix_zero(self, n):
            got = self.buf.copy_to_host()
            return bool(np.array_equal(got[:n * BLOCK_BYTES], expected[:n * BLOCK_BYTES])
                        and not got[n * BLOCK_BYTES:].any())

    def register(instance, gpu, tp_rank=0, tp_size=1, world_size=1):
        return client.register_context_batch(instance, "mock-vllm", tp_rank, 0, tp_size, world_size, 0,
                                             [LAYER], [gpu.wrapper], [BLOCKS], [BLOCK_BYTES], [0], [1],
                                             "direct", False)

    def save(instance, hs, tp_rank=0):
        return client.save(instance, tp_rank, 0, 0, [(LAYER, list(range(len(hs))), hs)])

    def load(instance, lease, n, tp_rank=0):
        """-> (outcome, LoadState value after waiting up to 5 s)."""
        state = LoadState()
        try:
            outcome = list(client.load(instance, tp_rank, 0, state.shm_name, [[LAYER]],
                                       [(lease, [list(range(n))])]))
        except (RpcRejected, PegaFlowError) as exc:
            outcome = [exc.code, str(exc)]
        deadline = time.time() + 5
        while state.get() == 0 and time.time() < deadline:
            time.sleep(0.0005)
        value = state.get()
        state.close()
        return outcome, value

    def rejected(fn):
        try:
            fn()
        except (RpcRejected, PegaFlowError) as exc:
            return [exc.code, str(exc)]
        return ["accepted", ""]

    out = {}

    # mock_vllm_save_query_load_roundtrip_over_rpc
    gpu = Gpu()
    inst = "mock-vllm-rpc-e2e"
    out["register"] = list(register(inst, gpu))
    hs = hashes(17)
    def query(instance, hs_, req_id):
        r = client.query_prefetch(instance, hs_, req_id)
        return type(r).__name__, r.num_hit_blocks, r.lease, r.hit_positions

    cold = query(inst, hs, "mock-vllm-cold-query")
    out["cold_query"] = [cold[0], cold[1], len(cold[2])]
    # python/tests/test_engine_client.py:20-44: a query without hashes is Ready(0) with no lease as well
    empty = query(inst, [], "query-contract-empty_query")
    out["empty_query"] = [empty[0], empty[1], empty[2] == b""]
    out["save"] = list(save(inst, hs))
    kind, hits, lease, _ = query(inst, hs, "mock-vllm-hit-query")
    out["hit_query"] = [kind, hits, len(lease)]
    gpu.zero()
    out["load"] = load(inst, lease, len(hs))
    out["roundtrip_matches"] = gpu.matches_expected()

    # mock_vllm_empty_req_id_query_returns_invalid_argument
    out["empty_req_id"] = rejected(lambda: client.query_prefetch(inst, hs, ""))

    # mock_vllm_query_lease_is_bound_to_instance_id
    hs = hashes(37)
    save(inst, hs)
    _k, _h, lease, _ = query(inst, hs, "mock-vllm-instance-bound")
    second = Gpu()
    register("mock-vllm-rpc-e2e-second", second)
    out["wrong_instance_load"] = load("mock-vllm-rpc-e2e-second", lease, len(hs))
    client.release(lease)

    # mock_vllm_release_unknown_lease_returns_error
    hs = hashes(39)
    save(inst, hs)
    _k, _h, lease, _ = query(inst, hs, "mock-vllm-release-once")
    out["first_release"] = rejected(lambda: client.release(lease))
    out["second_release"] = rejected(lambda: client.release(lease))

    # mock_vllm_prefix_partial_query_returns_prefix_lease
    hs = hashes(41)
    out["prefix_save"] = list(save(inst, hs[:2]))
    kind, hits, lease, _ = query(inst, hs, "mock-vllm-prefix-partial")
    out["prefix_query"] = [kind, hits, len(lease)]
    gpu.zero()
    out["prefix_load"] = load(inst, lease, 2)
    out["prefix_loaded_suffix_zero"] = gpu.prefix_loaded_suffix_zero(2)

    # mock_vllm_load_rejects_lease_block_count_mismatch
    hs = hashes(43)
    save(inst, hs[:2])
    _k, hits, lease, _ = query(inst, hs, "mock-vllm-load-count-mismatch")
    out["mismatch_hits"] = hits
    out["mismatch_load"] = load(inst, lease, len(hs))

    # mock_vllm_naive_tp2_load_roundtrip_over_rpc needs two GPUs (one context per device and
    # instance, as in the reference, which skips the case below two devices): not run here.

    # mock_vllm_session_disconnect_cleans_instance
    sess = Gpu()
    si = "mock-vllm-rpc-e2e-session"
    register(si, sess)
    client.start_session_watcher(si, "mock-vllm", 1, 1)
    hs = hashes(47)
    out["session_save"] = list(save(si, hs))
    _k, hits, lease, _ = query(si, hs, "mock-vllm-session-cleanup-hit")
    out["session_hits"] = hits
    client.stop_session_watcher()              # the stream ends: the server cleans the instance up
    deadline = time.time() + 10
    probe = ["accepted", ""]
    while time.time() < deadline:
        probe = rejected(lambda: client.query_prefetch(si, hs, "cleanup-probe"))
        if probe[0] != "accepted":
            break
        time.sleep(0.02)
    out["session_cleanup_probe"] = probe
    out["session_save_after_cleanup"] = rejected(lambda: save(si, hs))
    out["session_load_after_cleanup"] = load(si, lease, len(hs))

    # the first instance is still served after all of that
    hs = hashes(17)
    _k, hits, lease, _ = query(inst, hs, "still-there")
    out["first_instance_still_hits"] = hits
    client.release(lease)
    client.close()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
