"""Pinned pool on a real device: the reference's pool vectors
(pinned_pool.rs:722-795), sharding, exhaustion, reuse, and that the memory is
really device-mapped (a kernel copy through the pool's device pointers)."""

import numpy as np
import pytest

from pegaflow_amd import _lib
from pegaflow_amd.pool import PinnedAllocator
from pegaflow_amd.runtime import DeviceBuffer, PinnedMemory, Stream
from pegaflow_amd.transfer import CopyDesc, KernelBackend

pytestmark = pytest.mark.gpu


def test_pool_kat_largest_free_per_node(gpu, kats):
    case = kats["pool"][0]
    pool = PinnedAllocator(case["pool_bytes"], unit_size_hint=case["unit_hint"])
    other = PinnedAllocator(case["pool_bytes"], unit_size_hint=case["unit_hint"])
    held = pool.allocate(case["alloc"])
    assert held is not None and held.size == case["alloc"]
    assert pool.largest_free_allocation_for_node() == case["expect"]["largest_after"]
    assert other.largest_free_allocation_for_node() == case["expect"]["largest_untouched"]
    assert pool.usage() == (case["alloc"], case["pool_bytes"])
    assert not pool.is_numa
    held.free()
    assert pool.usage() == (0, case["pool_bytes"])
    pool.close()
    other.close()


def test_allocations_are_unit_rounded_disjoint_and_reusable(gpu):
    pool = PinnedAllocator(1 << 20)
    a = pool.allocate(1)
    b = pool.allocate(513)
    assert (a.size, b.size) == (512, 1024)
    assert a.host_ptr + a.size <= b.host_ptr or b.host_ptr + b.size <= a.host_ptr
    assert pool.usage() == (1536, 1 << 20)
    first = a.host_ptr
    a.free()
    c = pool.allocate(512)
    assert c.host_ptr == first  # the freed unit is handed out again
    assert pool.allocate(2 << 20) is None  # larger than the pool: None, not an error
    big = pool.allocate((1 << 20) - 1536 - 512)
    assert big is None or big.size <= (1 << 20)
    for x in (b, c, big):
        if x is not None:
            x.free()
    whole = pool.allocate(1 << 20)
    assert whole is not None and whole.size == 1 << 20
    assert pool.allocate(1) is None
    whole.free()
    pool.close()


def test_sharded_pool_round_robin_with_fallback(gpu):
    pool = PinnedAllocator(4 * 65536, num_shards=4)
    # Each shard holds 64 KiB: four 64 KiB allocations must land one per shard.
    allocs = [pool.allocate(65536) for _ in range(4)]
    assert all(a is not None for a in allocs)
    assert len({a.host_ptr for a in allocs}) == 4
    assert pool.allocate(1) is None
    allocs[2].free()
    again = pool.allocate(512)  # cursor points elsewhere: falls back to the shard with room
    assert again is not None
    assert pool.usage() == (3 * 65536 + 512, 4 * 65536)
    for a in allocs + [again]:
        a.free()
    pool.close()


def test_pool_memory_is_device_mapped(gpu):
    """A kernel-backend copy through the pool's (host, device-visible) pair."""
    pool = PinnedAllocator(1 << 20)
    a = pool.allocate(256 * 1024)
    data = np.random.default_rng(1).integers(0, 256, size=a.size, dtype=np.uint8)
    a.as_numpy()[:] = data
    dev = DeviceBuffer(a.size)
    dev.fill(0)
    s = Stream()
    k = KernelBackend()
    k.h2d([CopyDesc(dev.ptr, a.host_ptr, a.device_ptr, a.size)], s)
    s.synchronize()
    assert np.array_equal(dev.copy_to_host(), data)
    a.as_numpy()[:] = 0
    k.d2h([CopyDesc(dev.ptr, a.host_ptr, a.device_ptr, a.size)], s)
    s.synchronize()
    assert np.array_equal(a.as_numpy(), data)
    k.close()
    s.close()
    dev.close()
    a.free()
    pool.close()


def test_numa_pool_allocates_on_the_requested_node(gpu):
    pool = PinnedAllocator(2 << 20, numa_nodes=[0])
    assert pool.is_numa
    assert pool.allocate(4096, numa_node=-1) is None  # UNKNOWN node: no fallback
    assert pool.allocate(4096, numa_node=7) is None   # node without a pool
    a = pool.allocate(4096, numa_node=0)
    assert a is not None
    assert pool.largest_free_allocation_for_node(-1) == 0
    assert pool.largest_free_allocation_for_node(0) > 0
    a.free()
    pool.close()


def test_zero_size_and_bad_strategy(gpu):
    with pytest.raises(_lib.InvalidArgument, match="greater than zero"):
        PinnedMemory(0)
    with pytest.raises(_lib.InvalidArgument, match="greater than zero"):
        PinnedAllocator(0)


def test_stream_concurrency_probe(gpu):
    """A stream cannot overlap with itself: the waiting kernel gives up after
    its 2 ms and the answer is no.  For two streams the answer depends on the
    runtime's queue assignment; whichever it is, the call returns, twice the
    same, and leaves both streams idle.  A pool's two workers do overlap."""
    import time
    from pegaflow_amd.runtime import Stream
    a, b = Stream(), Stream()
    t0 = time.perf_counter()
    assert a.runs_concurrently_with(a) is False
    assert time.perf_counter() - t0 < 1.0
    first = a.runs_concurrently_with(b)
    assert a.runs_concurrently_with(b) is first
    a.synchronize()
    b.synchronize()
    a.close()
    b.close()
