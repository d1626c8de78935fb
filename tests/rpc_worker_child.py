"""Worker-process half of tests/test_gpu_rpc.py: a stand-in for the vLLM worker
of the reference's deployment.  It owns the KV caches, talks to the engine
server only through EngineRpcClient (the reference client's method names,
python/pegaflow/pegaflow.pyi:69-300), and checks its own memory after the load
it asked for has been reported complete through its LoadState.  Prints one
JSON line with the outcome."""

import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def main():
    port, layers, num_blocks, seg, nseg, n, backend = sys.argv[1:8]
    port, layers, num_blocks, seg, nseg, n = (int(x) for x in (port, layers, num_blocks, seg, nseg, n))
    import numpy as np
    import torch
    from pegaflow_amd import runtime
    from pegaflow_amd.engine import LoadState
    from pegaflow_amd.ipc import HipIPCWrapper
    from pegaflow_amd.rpc import EngineRpcClient

    torch.cuda.set_device(0)
    runtime.set_device(0)
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(11)
    layer_bytes = nseg * num_blocks * seg
    caches = [torch.empty(layer_bytes, device=dev, dtype=torch.uint8).random_(0, 256, generator=gen)
              for _ in range(layers)]
    originals = [c.clone() for c in caches]
    torch.cuda.synchronize()
    names = [f"model.layers.{i}.self_attn.attn" for i in range(layers)]
    rng = np.random.default_rng(5)
    src = rng.permutation(num_blocks)[:n]
    dst = rng.permutation(num_blocks)[:n]
    hashes = [b"rpc" + int(i).to_bytes(4, "little") for i in range(n)]
    out = {}
    client = EngineRpcClient(f"http://127.0.0.1:{port}")
    out["health"] = client.health()
    out["register"] = client.register_context_batch(
        "rpc-inst", "rpc-ns", 0, 0, 1, 1, 0, names, [HipIPCWrapper(c).to_bytes() for c in caches],
        [num_blocks] * layers, [seg] * layers, [num_blocks * seg if nseg == 2 else 0] * layers,
        [nseg] * layers, backend, False)
    try:
        client.register_context_batch(
            "rpc-inst", "rpc-ns", 0, 0, 1, 1, 0, names, [HipIPCWrapper(c).to_bytes() for c in caches],
            [num_blocks] * layers, [seg] * layers, [num_blocks * seg if nseg == 2 else 0] * layers,
            [nseg] * layers, backend, False)
        out["second_register"] = "accepted"
    except Exception as exc:
        out["second_register"] = f"{type(exc).__name__}: {exc}"
    out["save"] = client.save("rpc-inst", 0, 0, 0, [(nm, src.tolist(), hashes) for nm in names])
    try:
        client.save("rpc-inst", 0, 0, 0, [(names[0], [1, 2], [b"x"])])
        out["bad_save"] = "accepted"
    except ValueError as exc:
        out["bad_save"] = str(exc)
    for c in caches:
        c.zero_()
    torch.cuda.synchronize()
    ready = client.query_prefetch("rpc-inst", hashes + [b"missing"], "req-1")
    hits, lease = ready.num_hit_blocks, ready.lease
    out["query"] = [type(ready).__name__, hits, len(lease), ready.hit_positions]
    state = LoadState()
    # every second block of the lease goes nowhere (an absent target)
    targets = [int(b) if i % 2 == 0 else None for i, b in enumerate(dst)]
    out["load"] = client.load("rpc-inst", 0, 0, state.shm_name, [names], [(lease, [targets])])
    deadline = time.time() + 30
    while state.get() == 0 and time.time() < deadline:
        time.sleep(0.0005)
    out["load_state"] = state.get()
    torch.cuda.synchronize()
    keep = torch.tensor([i for i in range(n) if i % 2 == 0], device=dev)
    s_ids = torch.from_numpy(src).to(dev)[keep]
    d_ids = torch.from_numpy(dst).to(dev)[keep]
    rest = torch.ones(num_blocks, dtype=torch.bool, device=dev)
    rest[d_ids] = False
    rest = torch.nonzero(rest).reshape(-1)
    problems = []
    for li, (c, o) in enumerate(zip(caches, originals)):
        c3, o3 = c.view(nseg, num_blocks, seg), o.view(nseg, num_blocks, seg)
        if not torch.equal(c3[:, d_ids], o3[:, s_ids]):
            problems.append(f"layer {li}: loaded blocks differ")
        if bool(c3[:, rest].any()):
            problems.append(f"layer {li}: a block outside the targets changed")
    out["problems"] = problems[:4]
    # the lease was consumed by the load: releasing it now is refused
    try:
        client.release(lease)
        out["release_consumed"] = "accepted"
    except ValueError as exc:
        out["release_consumed"] = str(exc)
    again = client.query_prefetch("rpc-inst", hashes[:3], "req-2")
    client.release(again.lease)
    out["released"] = [type(again).__name__, again.num_hit_blocks]
    try:
        client.release(b"short")
        out["bad_lease"] = "accepted"
    except ValueError as exc:
        out["bad_lease"] = str(exc)
    out["unregister"] = client.unregister_context("rpc-inst")
    state.close()
    client.close()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
