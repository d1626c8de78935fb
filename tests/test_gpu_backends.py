"""GPU parity of the two reference-compatible transfer backends ("direct",
"kernel") through the C ABI, against the CPU oracle and the reference's own
GPU test vector (transfer/kernel.rs:203-267)."""

import numpy as np
import pytest

from oracle import oracle as O
from pegaflow_amd.runtime import DeviceBuffer, PinnedMemory, Stream
from pegaflow_amd.transfer import CopyDesc, KernelBackend, MemcpyBackend
from tests.helpers import kernel_test_pattern, random_bytes, xorshift_shuffle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def stream(gpu):
    s = Stream()
    yield s
    s.close()


@pytest.fixture(scope="module")
def backends(gpu):
    bs = [KernelBackend(), MemcpyBackend()]
    assert [b.name for b in bs] == ["kernel", "direct"]
    yield bs
    for b in bs:
        b.close()


def test_kernel_matches_direct_both_directions(backends, stream):
    n, seg = 257, 4096 + 16
    total = n * seg
    pattern = kernel_test_pattern(total)
    host = PinnedMemory(total)
    dev = DeviceBuffer(total)
    hv = host.as_numpy()
    descs = [CopyDesc(dev.ptr + k * seg, host.host_ptr + k * seg, host.device_ptr + k * seg, seg)
             for k in range(n)]
    for b in backends:
        hv[:] = pattern
        dev.fill(0)
        b.h2d(descs, stream)
        stream.synchronize()
        assert np.array_equal(dev.copy_to_host(), pattern), f"h2d mismatch for backend {b.name}"
    for b in backends:
        dev.copy_from_host(pattern)
        hv[:] = 0
        b.d2h(descs, stream)
        stream.synchronize()
        assert np.array_equal(hv, pattern), f"d2h mismatch for backend {b.name}"
    dev.close()
    host.close()


def test_empty_batch_is_a_no_op(backends, stream):
    for b in backends:
        b.h2d([], stream)
        b.d2h([], stream)
    stream.synchronize()


def _oracle_expect(dev0, host0, rows, host_is_src):
    """Run the oracle on host-resident copies; rows hold OFFSETS."""
    dev, host = dev0.copy(), host0.copy()
    orows = [(dev.ctypes.data + d, host.ctypes.data + h, host.ctypes.data + h, s, 0, 0)
             for d, h, s in rows]
    O.exec_descs(orows, host_is_src=host_is_src, backend="kernel")
    return dev, host


@pytest.mark.parametrize("direction", ["h2d", "d2h"])
def test_unaligned_and_odd_sizes_match_oracle(backends, stream, direction):
    """Fragment sizes that are not multiples of 16 and addresses that are not
    16-byte aligned on either side (the reference kernel's byte-loop cases,
    transfer/kernel.rs:31-43); bytes outside the fragments stay untouched."""
    rng = np.random.default_rng(31)
    slot = 8192
    cases = [(0, 0, 4112), (16, 32, 33), (5, 0, 100), (0, 3, 17), (1, 1, 4097), (4, 8, 1000),
             (8, 4, 15), (0, 0, 1), (7, 9, 1), (16, 16, 4096), (2, 2, 6000), (0, 0, 16), (12, 12, 20)]
    rows = [(i * slot + do, i * slot + ho, size) for i, (do, ho, size) in enumerate(cases)]
    total = slot * len(cases)
    dev0, host0 = random_bytes(rng, total), random_bytes(rng, total)
    exp_dev, exp_host = _oracle_expect(dev0, host0, rows, host_is_src=(direction == "h2d"))
    host = PinnedMemory(total)
    dev = DeviceBuffer(total)
    for b in backends:
        host.as_numpy()[:] = host0
        dev.copy_from_host(dev0)
        descs = [CopyDesc(dev.ptr + d, host.host_ptr + h, host.device_ptr + h, s) for d, h, s in rows]
        getattr(b, direction)(descs, stream)
        stream.synchronize()
        assert np.array_equal(dev.copy_to_host(), exp_dev), b.name
        assert np.array_equal(host.as_numpy(), exp_host), b.name
    dev.close()
    host.close()


def test_shuffled_4k_fragments(backends, stream):
    """Shape of the reference's transfer bench (benches/transfer_h2d.rs):
    4096-byte fragments in a seeded shuffled order, device strided by two."""
    seg, n = 4096, 4096
    perm = xorshift_shuffle(n)
    assert sorted(perm) == list(range(n))
    rng = np.random.default_rng(3)
    host0 = random_bytes(rng, n * seg)
    dev_bytes = ((n - 1) * 2 + 1) * seg
    host = PinnedMemory(n * seg)
    dev = DeviceBuffer(dev_bytes)
    descs = [CopyDesc(dev.ptr + slot * 2 * seg, host.host_ptr + slot * seg,
                      host.device_ptr + slot * seg, seg) for slot in perm]
    expect = np.full(dev_bytes, 0xA5, dtype=np.uint8)
    ev = expect[: (n - 1) * 2 * seg + seg]
    for slot in range(n):
        ev[slot * 2 * seg: slot * 2 * seg + seg] = host0[slot * seg: (slot + 1) * seg]
    for b in backends:
        host.as_numpy()[:] = host0
        dev.fill(0xA5)
        b.h2d(descs, stream)
        stream.synchronize()
        assert np.array_equal(dev.copy_to_host(), expect), b.name
        host.as_numpy()[:] = 0
        b.d2h(descs, stream)
        stream.synchronize()
        assert np.array_equal(host.as_numpy(), host0), b.name
    dev.close()
    host.close()


def test_few_large_descriptors_spread_over_tiles(backends, stream):
    """A batch of two large copies (one with a 48-byte tail): the kernel
    backend splits each descriptor over many workgroups."""
    rng = np.random.default_rng(8)
    sizes = [8 * 1024 * 1024 + 48, 3 * 1024 * 1024]
    total = sum(sizes) + 4096
    data = random_bytes(rng, total)
    host = PinnedMemory(total)
    dev = DeviceBuffer(total)
    offs = [0, sizes[0] + 4096 - 48]
    descs = [CopyDesc(dev.ptr + o, host.host_ptr + o, host.device_ptr + o, s)
             for o, s in zip(offs, sizes)]
    expect = np.zeros(total, dtype=np.uint8)
    for o, s in zip(offs, sizes):
        expect[o:o + s] = data[o:o + s]
    for b in backends:
        host.as_numpy()[:] = data
        dev.fill(0)
        b.h2d(descs, stream)
        stream.synchronize()
        assert np.array_equal(dev.copy_to_host(), expect), b.name
    dev.close()
    host.close()


def test_two_batches_without_sync_between(backends, stream):
    """Backends only enqueue: two batches on one stream, one synchronise."""
    rng = np.random.default_rng(4)
    seg, n = 4096, 64
    data = random_bytes(rng, 2 * n * seg)
    host = PinnedMemory(2 * n * seg)
    dev = DeviceBuffer(2 * n * seg)
    for b in backends:
        host.as_numpy()[:] = data
        dev.fill(0)
        first = [CopyDesc(dev.ptr + k * seg, host.host_ptr + k * seg, host.device_ptr + k * seg, seg)
                 for k in range(n)]
        second = [CopyDesc(dev.ptr + (n + k) * seg, host.host_ptr + (n + k) * seg,
                           host.device_ptr + (n + k) * seg, seg) for k in range(n)]
        b.h2d(first, stream)
        b.h2d(second, stream)
        stream.synchronize()
        assert np.array_equal(dev.copy_to_host(), data), b.name
    dev.close()
    host.close()
