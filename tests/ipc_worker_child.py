"""Worker-process half of tests/test_gpu_ipc.py.

Plays the vLLM worker of the reference's deployment: it owns the KV cache
tensors on the GPU, exports them (HipIPCWrapper, the stand-in for
python/pegaflow/ipc_wrapper.py), and later checks what the server process
loaded back into them, polling a LoadState it created itself
(pegaflow-core/src/sync_state.rs:23-188).  Commands arrive as JSON lines on
stdin, answers leave as JSON lines on stdout.
"""

import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def say(**kw):
    sys.stdout.write(json.dumps(kw) + "\n")
    sys.stdout.flush()


def hear():
    line = sys.stdin.readline()
    if not line:
        sys.exit(0)
    return json.loads(line)


def main():
    layers, num_blocks, seg, nseg, seed = (int(x) for x in sys.argv[1:6])
    import torch
    from pegaflow_amd import runtime
    from pegaflow_amd.engine import LoadState
    from pegaflow_amd.ipc import HipIPCWrapper, device_uuid

    torch.cuda.set_device(0)
    runtime.set_device(0)
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    layer_bytes = nseg * num_blocks * seg
    caches = [torch.empty(layer_bytes, device=dev, dtype=torch.uint8).random_(0, 256, generator=gen)
              for _ in range(layers)]
    originals = [c.clone() for c in caches]
    torch.cuda.synchronize()
    wrappers = [HipIPCWrapper(c) for c in caches]
    for w in wrappers:
        assert HipIPCWrapper.from_bytes(w.to_bytes()) == w
    say(ready=True, pid=os.getpid(), wrappers=[w.to_bytes().hex() for w in wrappers],
        device_uuid=device_uuid(0).hex(), layer_bytes=layer_bytes)
    state = None
    while True:
        cmd = hear()
        if cmd["op"] == "zero":
            for c in caches:
                c.zero_()
            torch.cuda.synchronize()
            if state is not None:
                state.close()
            state = LoadState()
            say(zeroed=True, shm=state.shm_name)
        elif cmd["op"] == "await":
            deadline = time.time() + 30
            while state.get() == 0 and time.time() < deadline:
                time.sleep(0.0005)
            result = state.get()
            torch.cuda.synchronize()
            src = torch.tensor(cmd["src_ids"], device=dev, dtype=torch.int64)
            dst = torch.tensor(cmd["dst_ids"], device=dev, dtype=torch.int64)
            rest = torch.ones(num_blocks, dtype=torch.bool, device=dev)
            rest[dst] = False
            rest = torch.nonzero(rest).reshape(-1)
            bad = []
            for li, (c, o) in enumerate(zip(caches, originals)):
                c3, o3 = c.view(nseg, num_blocks, seg), o.view(nseg, num_blocks, seg)
                if not torch.equal(c3[:, dst], o3[:, src]):
                    bad.append(f"layer {li}: loaded blocks differ")
                if bool(c3[:, rest].any()):
                    bad.append(f"layer {li}: a block outside the list changed")
            say(state=result, ok=not bad, problems=bad[:4])
        elif cmd["op"] == "checksum":
            say(sums=[int(c.to(torch.int64).sum().item()) for c in caches])
        elif cmd["op"] == "exit":
            say(bye=True)
            return
        else:
            say(error=f"unknown op {cmd['op']}")


if __name__ == "__main__":
    main()
