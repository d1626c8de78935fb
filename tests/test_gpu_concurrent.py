"""Transfers that run next to other work on the device, with every byte checked.

BASELINE configs[2] is a load of the 5,000 saved Llama-3.1-8B blocks "concurrently
with a synthetic 4096x4096x4096 bf16 GEMM stream"; the reference's worker pool
runs a load thread and a save thread per GPU at once
(pegaflow-core/src/gpu_worker.rs:131-201).  These tests run exactly those
combinations at full size and then check, on every layer, that block
save_ids[i] of the source arrived at list position i of the host image and at
block load_ids[i] of the destination, that no other destination block changed,
and that the GEMM stream computed what it computes alone."""

import time
import warnings

import numpy as np
import pytest

from bench import make_ids
from pegaflow_amd import runtime
from pegaflow_amd.layout import KVCacheLayout
from pegaflow_amd.runtime import PinnedMemory, Stream
from pegaflow_amd.transfer import BlockTransfer, LayerBlocks, TransferPath

pytestmark = pytest.mark.gpu

LAYERS, NB, SEG, NSEG, N = 32, 8192, 32768, 2, 5000
LAYER_BYTES = NSEG * NB * SEG
LAYER_PAYLOAD = NSEG * N * SEG
PAYLOAD = LAYERS * LAYER_PAYLOAD

# (path, copy_stream of the engine)
FORMS = [(TransferPath.STAGED, 0), (TransferPath.STAGED, 1), (TransferPath.STAGED, 2),
         (TransferPath.ZEROCOPY, 0)]
FORM_IDS = ["staged-default", "staged-side-stream", "staged-in-order", "zerocopy"]


class World:
    def __init__(self, torch):
        self.torch = torch
        self.dev = torch.device("cuda:0")
        gen = torch.Generator(device=self.dev)
        gen.manual_seed(4321)
        self.src = [torch.empty(LAYER_BYTES, device=self.dev, dtype=torch.uint8)
                    .random_(0, 256, generator=gen) for _ in range(LAYERS)]
        self.dst = [torch.zeros(LAYER_BYTES, device=self.dev, dtype=torch.uint8)
                    for _ in range(LAYERS)]
        self.pool_a = PinnedMemory(PAYLOAD)
        self.pool_b = PinnedMemory(PAYLOAD)
        self.scratch = torch.empty(LAYER_PAYLOAD, device=self.dev, dtype=torch.uint8)
        self.zeros = torch.zeros(LAYER_PAYLOAD, device=self.dev, dtype=torch.uint8)
        # One stream serves the checks and the transfers of the GEMM test: a process's
        # streams share GPU_MAX_HW_QUEUES (4) hardware queues, and a stream that lands on
        # the queue of the saturated GEMM stream would wait behind it.  torch's default
        # stream, the GEMM stream, this one and the engine's side stream make four.
        self.util = Stream()
        m = 4096
        self.a = torch.randn(m, m, device=self.dev, dtype=torch.bfloat16, generator=gen)
        self.b = [torch.randn(m, m, device=self.dev, dtype=torch.bfloat16, generator=gen)
                  for _ in range(4)]
        self.c = [torch.empty(m, m, device=self.dev, dtype=torch.bfloat16) for _ in range(4)]
        self.gemm_stream = torch.cuda.Stream()
        # The GEMM stream alone: reference results and time per GEMM.
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        self.run_gemms(8)
        torch.cuda.synchronize()
        with torch.cuda.stream(self.gemm_stream):
            t0.record()
        host0 = time.perf_counter()
        self.run_gemms(200)
        self.enqueue_ms = (time.perf_counter() - host0) * 1e3 / 200   # host time per launch
        with torch.cuda.stream(self.gemm_stream):
            t1.record()
        torch.cuda.synchronize()
        self.gemm_ms = t0.elapsed_time(t1) / 200
        self.c_alone = [c.clone() for c in self.c]
        self.run_gemms(8)
        torch.cuda.synchronize()
        self.gemm_is_deterministic = all(torch.equal(x, y) for x, y in zip(self.c, self.c_alone))

    def run_gemms(self, count):
        torch = self.torch
        with torch.cuda.stream(self.gemm_stream):
            for i in range(count):
                torch.matmul(self.a, self.b[i % 4], out=self.c[i % 4])

    def check_gemms(self):
        torch = self.torch
        for got, want in zip(self.c, self.c_alone):
            if self.gemm_is_deterministic:
                assert torch.equal(got, want), "GEMM next to a transfer differs from the GEMM alone"
            else:
                assert torch.allclose(got.float(), want.float(), rtol=2e-2, atol=1.0)

    def layouts(self, caches):
        return [KVCacheLayout(t.data_ptr(), LAYER_BYTES, NB, SEG, NB * SEG, NSEG) for t in caches]

    def layers(self, caches, ids, pool):
        buf = N * SEG
        out = []
        for li, lay in enumerate(self.layouts(caches)):
            off = li * LAYER_PAYLOAD
            out.append(LayerBlocks(
                layout=lay, block_ids=ids,
                host=tuple(pool.host_ptr + off + s * buf for s in range(NSEG)),
                host_device=tuple(pool.device_ptr + off + s * buf for s in range(NSEG)),
                host_len=(buf, buf), host_stride=SEG, layer_name=f"layer{li}"))
        return out

    def clear_pool(self, pool):
        for li in range(LAYERS):
            runtime.memcpy_d2h_async(pool.host_ptr + li * LAYER_PAYLOAD, self.zeros.data_ptr(),
                                     LAYER_PAYLOAD, self.util)
        self.util.synchronize()

    def clear_dst(self):
        for t in self.dst:
            t.zero_()
        self.torch.cuda.synchronize()

    def check_image(self, pool, ids, what):
        """Every layer of the host image holds the source blocks in list order."""
        torch = self.torch
        sid = torch.from_numpy(ids.astype(np.int64)).to(self.dev)
        for li in range(LAYERS):
            runtime.memcpy_h2d_async(self.scratch.data_ptr(), pool.host_ptr + li * LAYER_PAYLOAD,
                                     LAYER_PAYLOAD, self.util)
            self.util.synchronize()
            want = self.src[li].view(NSEG, NB, SEG)[:, sid]
            assert torch.equal(self.scratch.view(NSEG, N, SEG), want), \
                f"{what}: host image of layer {li} differs"

    def check_dst(self, save_ids, load_ids, what):
        """Block save_ids[i] of the source is block load_ids[i] of the destination on
        every layer, and every other destination block is still zero."""
        torch = self.torch
        sid = torch.from_numpy(save_ids.astype(np.int64)).to(self.dev)
        lid = torch.from_numpy(load_ids.astype(np.int64)).to(self.dev)
        untouched = torch.ones(NB, dtype=torch.bool, device=self.dev)
        untouched[lid] = False
        rest = torch.nonzero(untouched).reshape(-1)
        for li in range(LAYERS):
            s = self.src[li].view(NSEG, NB, SEG)
            d = self.dst[li].view(NSEG, NB, SEG)
            assert torch.equal(d[:, lid], s[:, sid]), f"{what}: layer {li}: loaded blocks differ"
            assert not bool(d[:, rest].any()), f"{what}: layer {li}: a block outside the list changed"

    def close(self):
        self.util.close()
        self.pool_a.close()
        self.pool_b.close()


@pytest.fixture(scope="module")
def world(gpu):
    import torch
    torch.cuda.set_device(0)
    w = World(torch)
    yield w
    w.close()
    del w
    torch.cuda.empty_cache()


@pytest.mark.parametrize("path,copy_stream", FORMS, ids=FORM_IDS)
def test_save_then_load_next_to_gemm_stream(world, path, copy_stream):
    """configs[1] + configs[2] with the GEMM stream busy for the whole transfer."""
    torch = world.torch
    save_ids = make_ids(np, "permutation", NB, N, 0)
    load_ids = make_ids(np, "permutation", NB, N, 1)
    world.clear_pool(world.pool_a)
    world.clear_dst()
    for c in world.c:
        c.zero_()
    torch.cuda.synchronize()
    xfer = BlockTransfer(copy_stream=copy_stream)
    stream = world.util
    try:
        # allocate staging before the contended run (an allocation synchronises the device)
        xfer.save(world.layers(world.src, save_ids, world.pool_a)[:1], stream, path)
        stream.synchronize()
        world.clear_pool(world.pool_a)
        # A backlog of GEMMs first, so that the stream is busy when the transfer starts;
        # then the transfer is enqueued (the calls only enqueue), and the host keeps feeding
        # the GEMM stream until the transfer's last event has completed.
        gemm_native = Stream.wrap(world.gemm_stream.cuda_stream)
        marks = [runtime.Event(timing=True) for _ in range(4)]
        marks[0].record(gemm_native)
        count = 1500
        world.run_gemms(count)
        marks[2].record(stream)
        xfer.save(world.layers(world.src, save_ids, world.pool_a), stream, path)
        xfer.load(world.layers(world.dst, load_ids, world.pool_a), stream, path)
        marks[3].record(stream)
        while not marks[3].query():
            world.run_gemms(32)
            count += 32
            assert count < 40000, "the transfer does not finish"
        marks[1].record(gemm_native)
        stream.synchronize()
        torch.cuda.synchronize()
        gemm_ms = marks[0].elapsed_ms(marks[1])
        xfer_begin, xfer_end = marks[0].elapsed_ms(marks[2]), marks[0].elapsed_ms(marks[3])
        together = min(gemm_ms, xfer_end) - max(0.0, xfer_begin)
        print(f"GEMM stream {gemm_ms:.0f} ms ({count} GEMMs, {world.gemm_ms * 1e3:.0f} us each alone); "
              f"transfer from {xfer_begin:.0f} to {xfer_end:.0f} ms; together {together:.0f} ms",
              flush=True)
        # The GEMM stream and the transfer were in flight at the same time (order of
        # events); for how much of the transfer depends on how fast the host feeds
        # the GEMM stream on this box, so a low share is a warning, not a failure.
        assert together > 0.0, "the GEMM stream and the transfer never ran at the same time"
        if together < 0.9 * (xfer_end - xfer_begin):
            warnings.warn(f"the GEMM stream ran beside the transfer for only {together:.0f} of "
                          f"{xfer_end - xfer_begin:.0f} ms")
        assert xfer.last_path == path
        torch.cuda.synchronize()
        world.check_image(world.pool_a, save_ids, "save next to GEMMs")
        world.check_dst(save_ids, load_ids, "load next to GEMMs")
        world.check_gemms()
    finally:
        xfer.close()


@pytest.mark.parametrize("path,copy_stream", FORMS[1:], ids=FORM_IDS[1:])
def test_save_and_load_at_once(world, path, copy_stream):
    """A save (cache -> pool B) and a load (pool A -> second cache) in flight
    together on two engines and two streams, as the pool's two workers issue them."""
    torch = world.torch
    ids_a = make_ids(np, "permutation", NB, N, 10)     # what pool A holds
    ids_b = make_ids(np, "permutation", NB, N, 11)     # what the concurrent save gathers
    load_ids = make_ids(np, "permutation", NB, N, 12)
    xa, xb = BlockTransfer(copy_stream=copy_stream), BlockTransfer(copy_stream=copy_stream)
    sa, sb = Stream(), Stream()
    try:
        xa.save(world.layers(world.src, ids_a, world.pool_a), sa, path)
        sa.synchronize()
        xb.load(world.layers(world.dst, load_ids, world.pool_a)[:1], sb, path)  # staging of xb
        sb.synchronize()
        world.clear_pool(world.pool_b)
        world.clear_dst()
        done = [runtime.Event(timing=True) for _ in range(4)]
        done[0].record(sa)
        done[2].record(sb)
        xa.save(world.layers(world.src, ids_b, world.pool_b), sa, path)
        xb.load(world.layers(world.dst, load_ids, world.pool_a), sb, path)
        done[1].record(sa)
        done[3].record(sb)
        sa.synchronize()
        sb.synchronize()
        # the two really were in flight together: each started before the other ended
        assert done[0].elapsed_ms(done[3]) > 0 and done[2].elapsed_ms(done[1]) > 0
        overlap_ms = min(done[0].elapsed_ms(done[1]), done[0].elapsed_ms(done[3])) - \
            max(0.0, done[0].elapsed_ms(done[2]))
        if overlap_ms < 50.0:   # how long is a matter of rates: recorded, not gating
            warnings.warn(f"save and load overlapped for only {overlap_ms:.1f} ms")
        world.check_image(world.pool_b, ids_b, "save next to a load")
        world.check_image(world.pool_a, ids_a, "pool read by the load")
        world.check_dst(ids_a, load_ids, "load next to a save")
    finally:
        for o in (xa, xb, sa, sb):
            o.close()
