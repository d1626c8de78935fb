"""GPU parity of pf_desc_copy_noalloc, the descriptor copy that allocates
nothing, against the kernel backend's pf_backend_h2d / pf_backend_d2h on the
same descriptors: byte-exact, two calls in a row (the second smaller, so a
table that kept rows of the first call would show), both directions, aligned
and unaligned fragments; and the refusals (too many descriptors, null
addresses)."""

import numpy as np
import pytest

from pegaflow_amd import _lib
from pegaflow_amd.runtime import DeviceBuffer, PinnedMemory, Stream
from pegaflow_amd.transfer import (KernelBackend, desc_array, desc_copy_noalloc,
                                   desc_copy_noalloc_max)
from tests.helpers import random_bytes

pytestmark = pytest.mark.gpu


def _fragments(rng, n, slot, odd):
    """n fragments in shuffled host order, device side strided by two slots."""
    order = rng.permutation(n)
    if odd:
        sizes = rng.integers(1, slot - 32, size=n)
        d_off = rng.integers(0, 16, size=n)
        h_off = rng.integers(0, 16, size=n)
    else:
        sizes = np.full(n, slot)
        d_off = np.zeros(n, dtype=np.int64)
        h_off = np.zeros(n, dtype=np.int64)
    dev_off = np.arange(n) * 2 * slot + d_off
    host_off = order * slot + h_off
    return dev_off.astype(np.uint64), host_off.astype(np.uint64), sizes.astype(np.uint64)


@pytest.mark.parametrize("direction", ["d2h", "h2d"])
@pytest.mark.parametrize("odd", [False, True], ids=["aligned4k", "unaligned"])
def test_noalloc_matches_kernel_backend_twice(gpu, direction, odd):
    rng = np.random.default_rng(77 + odd)
    slot = 4096
    n_first, n_second = 3000, 700
    dev_bytes, host_bytes = n_first * 2 * slot, n_first * slot
    dev0, host0 = random_bytes(rng, dev_bytes), random_bytes(rng, host_bytes)
    stream = Stream()
    backend = KernelBackend()
    host = PinnedMemory(host_bytes)
    dev = DeviceBuffer(dev_bytes)
    host_is_src = direction == "h2d"
    for n in (n_first, n_second):
        d, h, size = _fragments(rng, n, slot, odd)
        descs = desc_array(dev.ptr + d, host.host_ptr + h, host.device_ptr + h, size)
        results = []
        for call in ("backend", "noalloc"):
            host.as_numpy()[:] = host0
            dev.copy_from_host(dev0)
            if call == "backend":
                getattr(backend, direction)(descs, stream)
            else:
                keep = desc_copy_noalloc(descs, stream, host_is_src)
            stream.synchronize()
            results.append((dev.copy_to_host().copy(), host.as_numpy().copy()))
        del keep
        assert np.array_equal(results[0][0], results[1][0]), f"device bytes differ, n={n}"
        assert np.array_equal(results[0][1], results[1][1]), f"host bytes differ, n={n}"
        # and the copy did something: the written side changed
        changed = results[1][0] if host_is_src else results[1][1]
        before = dev0 if host_is_src else host0
        assert not np.array_equal(changed, before)
    backend.close()
    stream.close()
    dev.close()
    host.close()


def test_noalloc_two_calls_without_a_synchronise_between(gpu):
    """Two calls on one stream with no synchronise between them: the second
    call's table upload is ordered behind the first call's kernel."""
    rng = np.random.default_rng(5)
    slot, n = 8192, 512
    src = random_bytes(rng, 2 * n * slot)
    stream = Stream()
    host = PinnedMemory(2 * n * slot)
    dev = DeviceBuffer(2 * n * slot)
    dev.copy_from_host(src)
    host.as_numpy()[:] = 0
    perm = rng.permutation(2 * n).astype(np.uint64)
    first = desc_array(dev.ptr + np.arange(n, dtype=np.uint64) * slot,
                       host.host_ptr + perm[:n] * slot, host.device_ptr + perm[:n] * slot, slot)
    second = desc_array(dev.ptr + (n + np.arange(n // 4, dtype=np.uint64)) * slot,
                        host.host_ptr + perm[n:n + n // 4] * slot,
                        host.device_ptr + perm[n:n + n // 4] * slot, slot)
    keep = [desc_copy_noalloc(first, stream, False), desc_copy_noalloc(second, stream, False)]
    stream.synchronize()
    del keep
    img = host.as_numpy().reshape(2 * n, slot)
    srcv = src.reshape(2 * n, slot)
    expect = np.zeros_like(img)
    expect[perm[:n].astype(np.int64)] = srcv[:n]
    expect[perm[n:n + n // 4].astype(np.int64)] = srcv[n:n + n // 4]
    assert np.array_equal(img, expect)
    stream.close()
    dev.close()
    host.close()


def test_noalloc_calls_on_two_streams_share_the_table_safely(gpu):
    """A long call on one stream, then a short one on another stream with no
    host synchronise between them: the second call's upload overwrites the rows
    the first call's kernel reads, so the library makes it wait on the device
    for that kernel.  Both results must be whole."""
    rng = np.random.default_rng(11)
    slot, n = 4096, 24576
    src = random_bytes(rng, n * slot)
    sa, sb = Stream(), Stream()
    host = PinnedMemory(n * slot)
    host2 = PinnedMemory(64 * slot)
    dev = DeviceBuffer(n * slot)
    dev.copy_from_host(src)
    host.as_numpy()[:] = 0
    host2.as_numpy()[:] = 0
    perm = rng.permutation(n).astype(np.uint64)
    first = desc_array(dev.ptr + np.arange(n, dtype=np.uint64) * slot,
                       host.host_ptr + perm * slot, host.device_ptr + perm * slot, slot)
    pick = rng.permutation(n)[:64].astype(np.uint64)
    second = desc_array(dev.ptr + pick * slot,
                        host2.host_ptr + np.arange(64, dtype=np.uint64) * slot,
                        host2.device_ptr + np.arange(64, dtype=np.uint64) * slot, slot)
    for _ in range(3):
        keep = [desc_copy_noalloc(first, sa, False), desc_copy_noalloc(second, sb, False)]
        sa.synchronize()
        sb.synchronize()
        del keep
        srcv = src.reshape(n, slot)
        assert np.array_equal(host.as_numpy().reshape(n, slot)[perm.astype(np.int64)], srcv)
        assert np.array_equal(host2.as_numpy().reshape(64, slot), srcv[pick.astype(np.int64)])
        host.as_numpy()[:] = 0
        host2.as_numpy()[:] = 0
    for o in (sa, sb, dev, host, host2):
        o.close()


def test_noalloc_refusals(gpu):
    stream = Stream()
    host = PinnedMemory(4096)
    dev = DeviceBuffer(4096)
    limit = desc_copy_noalloc_max()
    assert limit == 32768
    too_many = desc_array(np.full(limit + 1, dev.ptr, dtype=np.uint64), host.host_ptr,
                          host.device_ptr, 16)
    with pytest.raises(_lib.InvalidArgument, match="at most 32768 descriptors"):
        desc_copy_noalloc(too_many, stream, False)
    with pytest.raises(_lib.InvalidArgument, match="descriptor 1: the copy kernel needs"):
        desc_copy_noalloc(desc_array([dev.ptr, 0], host.host_ptr, host.device_ptr, 64), stream, True)
    desc_copy_noalloc(desc_array([], [], [], []), stream, True)
    desc_copy_noalloc(desc_array([0], [0], [0], [0]), stream, True)
    stream.synchronize()
    stream.close()
    dev.close()
    host.close()


def test_noalloc_full_table(gpu):
    """The largest batch the call takes (every row of the table in use)."""
    rng = np.random.default_rng(9)
    n = desc_copy_noalloc_max()
    slot = 1024
    src = random_bytes(rng, n * slot)
    stream = Stream()
    host = PinnedMemory(n * slot)
    dev = DeviceBuffer(n * slot)
    host.as_numpy()[:] = src
    dev.fill(0)
    perm = rng.permutation(n).astype(np.uint64)
    descs = desc_array(dev.ptr + perm * slot, host.host_ptr + np.arange(n, dtype=np.uint64) * slot,
                       host.device_ptr + np.arange(n, dtype=np.uint64) * slot, slot)
    keep = desc_copy_noalloc(descs, stream, True)
    stream.synchronize()
    del keep
    out = dev.copy_to_host().reshape(n, slot)
    assert np.array_equal(out[perm.astype(np.int64)], src.reshape(n, slot))
    stream.close()
    dev.close()
    host.close()
