"""Child process of tests/test_gpu_duplex.py: a process that holds nothing but
engine worker pools (as the engine server does), so the hardware queues of the
device are shared by the worker streams alone.

Reports, as one JSON line: the worker-stream report after two instances (two
pools, four worker streams) and after a third; and the rate of a save and a
load in flight together through the engine on the Llama-3.1-8B shape
(BASELINE configs[1] + configs[2] at once: the reference's pool runs a load
thread and a save thread per GPU, pegaflow-core/src/gpu_worker.rs:131-201),
with the loaded blocks of two layers checked."""

import json
import os
import sys
import threading
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def main():
    layers = int(sys.argv[1]) if len(sys.argv) > 1 else 32
    side_copy_streams = len(sys.argv) > 2 and sys.argv[2] == "side"
    import numpy as np
    from pegaflow_amd import runtime
    from pegaflow_amd.engine import LayerSave, PackedSaves, PegaEngine, worker_stream_report
    from pegaflow_amd.runtime import DeviceBuffer
    from pegaflow_amd.transfer import TransferMode

    runtime.set_device(0)
    nb, seg, nseg, n = 8192, 32768, 2, 5000
    layer_bytes = nseg * nb * seg
    payload = layers * nseg * n * seg
    rng = np.random.default_rng(0)
    base = rng.integers(0, 256, size=layer_bytes, dtype=np.uint8)
    src = [DeviceBuffer(layer_bytes) for _ in range(layers)]
    dst = [DeviceBuffer(layer_bytes) for _ in range(layers)]
    for s_, d_ in zip(src, dst):
        s_.copy_from_host(base)
        d_.fill(0)
    names = [f"model.layers.{i}.self_attn.attn" for i in range(layers)]
    eng = PegaEngine(pool_size=int(payload * 2.3) + (256 << 20),
                     side_copy_streams=side_copy_streams)
    out = {}

    def register(inst, caches):
        eng.register_context_layer_batch(
            inst, "duplex", 0, 0, 0, 1, 1, names, [c.ptr for c in caches], [layer_bytes] * layers,
            [nb] * layers, [seg] * layers, [nb * seg] * layers, [nseg] * layers,
            transfer_mode=TransferMode.DIRECT)

    register("src", src)
    register("dst", dst)
    streams, pairs, skipped = worker_stream_report(0)
    out["two_pools"] = {"streams": streams, "clashing_pairs": pairs, "skipped": skipped}

    save_ids = rng.permutation(nb)[:n]
    load_ids = rng.permutation(nb)[:n]
    hashes_a = [b"A" + int(i).to_bytes(4, "little") for i in range(n)]
    hashes_b = [b"B" + int(i).to_bytes(4, "little") for i in range(n)]
    packed_a = PackedSaves([LayerSave(nm, save_ids, hashes_a) for nm in names])
    packed_b = PackedSaves([LayerSave(nm, save_ids, hashes_b) for nm in names])
    eng.batch_save_kv_blocks("src", 0, 0, 0, packed_a)
    rates = []
    for rep in range(3):
        hits, lease = eng.query_prefix("dst", hashes_a)
        assert hits == n
        times = {}

        def do_save():
            t0 = time.perf_counter()
            eng.batch_save_kv_blocks("src", 0, 0, 0, packed_b)
            times["save"] = time.perf_counter() - t0
            times["save_span"] = (t0, time.perf_counter())

        def do_load():
            t0 = time.perf_counter()
            task = eng.batch_load_kv_blocks_multi_layer("dst", 0, 0, [names], lease,
                                                        [load_ids.tolist()])
            task.wait()
            times["load"] = time.perf_counter() - t0
            times["load_span"] = (t0, time.perf_counter())
            task.close()

        threads = [threading.Thread(target=do_save), threading.Thread(target=do_load)]
        t0 = time.perf_counter()
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        span = time.perf_counter() - t0
        (s0, s1), (l0, l1) = times["save_span"], times["load_span"]
        rates.append({"in_flight_together": bool(s0 < l1 and l0 < s1),
                      "save_gbps": round(payload / times["save"] / 1e9, 2),
                      "load_gbps": round(payload / times["load"] / 1e9, 2),
                      "aggregate_gbps": round(2 * payload / span / 1e9, 2)})
        # drop batch B so the next repetition stores it again
        eng.evict_all()
        eng.batch_save_kv_blocks("src", 0, 0, 0, packed_a)
    out["concurrent_save_and_load"] = rates
    problems = []
    base3 = base.reshape(nseg, nb, seg)
    for li in (0, layers - 1):
        got = dst[li].copy_to_host().reshape(nseg, nb, seg)
        if not np.array_equal(got[:, load_ids], base3[:, save_ids]):
            problems.append(f"layer {li}: loaded blocks differ")
        rest = np.ones(nb, dtype=bool)
        rest[load_ids] = False
        if got[:, rest].any():
            problems.append(f"layer {li}: a block outside the list changed")
    out["problems"] = problems
    third = [DeviceBuffer(1 << 20) for _ in range(2)]
    eng.register_context_layer_batch(
        "third", "duplex", 0, 0, 0, 1, 1, ["a", "b"], [c.ptr for c in third], [1 << 20] * 2, [16] * 2,
        [32768] * 2, [16 * 32768] * 2, [2] * 2, transfer_mode=TransferMode.DIRECT)
    streams, pairs, skipped = worker_stream_report(0)
    out["three_pools"] = {"streams": streams, "clashing_pairs": pairs, "skipped": skipped}
    eng.close()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
