"""GPU parity of the two reference-compatible transfer backends ("direct",
"kernel") through the C ABI, against the CPU oracle and the reference's own
GPU test vector (transfer/kernel.rs:203-267)."""

import numpy as np
import pytest

from oracle import oracle as O
from pegaflow_amd import _lib
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


def test_kernel_backend_refuses_null_addresses(stream, gpu):
    """A descriptor the kernel would dereference at address 0 is refused on the
    host; zero-size descriptors carry no addresses worth checking."""
    b = KernelBackend()
    host = PinnedMemory(4096)
    dev = DeviceBuffer(4096)
    for desc in (CopyDesc(0, host.host_ptr, host.device_ptr, 64, 0, 1),
                 CopyDesc(dev.ptr, host.host_ptr, 0, 64, 0, 1)):
        with pytest.raises(_lib.InvalidArgument, match="descriptor 1: the kernel backend needs"):
            b.d2h([CopyDesc(dev.ptr, host.host_ptr, host.device_ptr, 64, 0, 1), desc], stream)
    b.d2h([CopyDesc(0, 0, 0, 0, 0, 0)], stream)
    stream.synchronize()
    b.close()
    host.close()
    dev.close()


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


@pytest.mark.parametrize("n", [4096, 16385, 40001])
def test_shuffled_4k_fragments(backends, stream, n):
    """Shape of the reference's transfer bench (benches/transfer_h2d.rs):
    4096-byte fragments in a seeded shuffled order, device strided by two.
    The larger, odd count makes the direct backend's packing launch take two
    fragments per workgroup with one left over; the largest goes through the
    direct backend in pieces (lists that do not merge are submitted 16 384
    descriptors at a time)."""
    seg = 4096
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


def test_direct_backend_batches_on_two_streams_share_its_staging(gpu):
    """Two host-dense batches through ONE direct backend on two different
    streams with no synchronise between them: both are packed through the
    backend's one staging buffer, so the second has to wait (on the device) for
    the first one's use of it."""
    from pegaflow_amd.transfer import desc_array
    rng = np.random.default_rng(21)
    seg, n = 4096, 6000
    data = random_bytes(rng, 2 * n * seg)
    host = PinnedMemory(2 * n * seg)
    dev = DeviceBuffer(2 * n * seg)
    s1, s2 = Stream(), Stream()
    b = MemcpyBackend()
    perm1 = rng.permutation(n).astype(np.uint64)
    perm2 = rng.permutation(n).astype(np.uint64) + n
    pos = np.arange(n, dtype=np.uint64)
    first = desc_array(dev.ptr + perm1 * seg, host.host_ptr + pos * seg, host.device_ptr + pos * seg,
                       seg, 0, 1)
    second = desc_array(dev.ptr + perm2 * seg, host.host_ptr + (n + pos) * seg,
                        host.device_ptr + (n + pos) * seg, seg, 0, 1)
    try:
        for _ in range(3):
            host.as_numpy()[:] = data
            dev.fill(0)
            b.h2d(first, s1)
            b.h2d(second, s2)
            s1.synchronize()
            s2.synchronize()
            got = dev.copy_to_host().reshape(2 * n, seg)
            want = data.reshape(2 * n, seg)
            assert np.array_equal(got[perm1.astype(np.int64)], want[:n])
            assert np.array_equal(got[perm2.astype(np.int64)], want[n:])
            host.as_numpy()[:] = 0
            b.d2h(first, s2)
            b.d2h(second, s1)
            s1.synchronize()
            s2.synchronize()
            assert np.array_equal(host.as_numpy(), data)
    finally:
        b.close()
        s1.close()
        s2.close()
        dev.close()
        host.close()


def _run_both_directions(backend, stream, descs_fn, dev_bytes, host_bytes, rows, seed):
    """rows: (device offset, host offset, size).  Checks h2d and d2h of one
    backend against the oracle, including the bytes outside the fragments."""
    rng = np.random.default_rng(seed)
    dev0, host0 = random_bytes(rng, dev_bytes), random_bytes(rng, host_bytes)
    host = PinnedMemory(host_bytes)
    dev = DeviceBuffer(dev_bytes)
    try:
        for direction in ("h2d", "d2h"):
            exp_dev, exp_host = _oracle_expect(dev0, host0, rows, host_is_src=(direction == "h2d"))
            host.as_numpy()[:] = host0
            dev.copy_from_host(dev0)
            getattr(backend, direction)(descs_fn(dev, host), stream)
            stream.synchronize()
            assert np.array_equal(dev.copy_to_host(), exp_dev), direction
            assert np.array_equal(host.as_numpy(), exp_host), direction
    finally:
        dev.close()
        host.close()


@pytest.mark.parametrize("n", [3000, 21000])
def test_direct_backend_packs_host_dense_runs(stream, gpu, n):
    """Many small ranges whose host sides follow one another (the batch image
    of a save): the direct backend stages them instead of one copy each.  K/V
    style interleave over two host allocations, device side shuffled.  The
    larger list (42 000 descriptors) is submitted in pieces, each with its own
    runs through the one staging buffer."""
    from pegaflow_amd.transfer import desc_array
    seg = 4096
    perm = np.array(xorshift_shuffle(n), dtype=np.uint64)
    k_dev = perm * 2 * seg                       # K region: every other slot
    v_dev = (2 * n + perm * 2) * seg             # V region behind it
    k_host = np.arange(n, dtype=np.uint64) * seg
    v_host = (n + np.arange(n, dtype=np.uint64)) * seg + 4096   # second allocation, after a gap
    dev_off = np.stack([k_dev, v_dev], axis=1).reshape(-1)      # K0 V0 K1 V1 ...
    host_off = np.stack([k_host, v_host], axis=1).reshape(-1)
    alloc = np.tile(np.array([1, 2], dtype=np.uint64), n)
    rows = [(int(d), int(h), seg) for d, h in zip(dev_off, host_off)]

    def descs(dev, host):
        return desc_array(dev.ptr + dev_off, host.host_ptr + host_off, host.device_ptr + host_off,
                          seg, 0, alloc)

    b = MemcpyBackend()
    try:
        _run_both_directions(b, stream, descs, 4 * n * seg, (2 * n + 1) * seg, rows, seed=11)
    finally:
        b.close()


def test_direct_backend_mixed_batch(stream, gpu):
    """One batch holding a large range, a host-dense run of odd-sized unaligned
    pieces, isolated small ranges without a device-visible host address (so
    they must be copied one by one), and an empty range."""
    from pegaflow_amd.transfer import desc_array
    big = 5 * 1024 * 1024 + 48
    piece, n_dense = 1000, 300
    rows = [(0, 64, big)]
    dense_host0 = big + 4096 + 3
    rows += [(big + 8192 + i * 2048 + 1, dense_host0 + i * piece, piece) for i in range(n_dense)]
    iso_dev0 = big + 8192 + n_dense * 2048 + 4096
    iso_host0 = dense_host0 + n_dense * piece + 777
    rows += [(iso_dev0 + i * 4096, iso_host0 + i * 8192, 333 + i) for i in range(12)]
    rows.append((0, 0, 0))
    dev_bytes = iso_dev0 + 12 * 4096 + 4096
    host_bytes = iso_host0 + 12 * 8192 + 4096
    d = np.array([r[0] for r in rows], dtype=np.uint64)
    h = np.array([r[1] for r in rows], dtype=np.uint64)
    sz = np.array([r[2] for r in rows], dtype=np.uint64)
    mapped = np.ones(len(rows), dtype=np.uint64)
    mapped[1 + n_dense:1 + n_dense + 12] = 0       # isolated ranges: no mapping given

    def descs(dev, host):
        return desc_array(dev.ptr + d, host.host_ptr + h, (host.device_ptr + h) * mapped, sz, 0, 7)

    b = MemcpyBackend()
    try:
        _run_both_directions(b, stream, descs, dev_bytes, host_bytes, rows, seed=12)
    finally:
        b.close()


def test_direct_backend_run_longer_than_the_staging_buffer(stream, gpu):
    """A host-dense run of 273 MiB is split over several passes of the 256 MiB
    staging buffer; verified by value on the device (too large for the oracle)."""
    from pegaflow_amd.transfer import desc_array
    seg, n = 4096, 70000
    host = PinnedMemory(n * seg)
    dev = DeviceBuffer(2 * n * seg)
    hv = host.as_numpy().view(np.uint32)
    hv[:] = np.arange(hv.size, dtype=np.uint32) * np.uint32(2654435761)
    want = host.as_numpy().copy()
    pos = np.arange(n, dtype=np.uint64)
    slot = (pos * 7919) % n                       # 7919 is coprime to 70000: a permutation
    descs = desc_array(dev.ptr + slot * 2 * seg, host.host_ptr + pos * seg,
                       host.device_ptr + pos * seg, seg, 0, 1)
    b = MemcpyBackend()
    try:
        dev.fill(0)
        b.h2d(descs, stream)
        stream.synchronize()
        got = dev.copy_to_host().reshape(2 * n, seg)
        assert np.array_equal(got[slot.astype(np.int64) * 2], want.reshape(n, seg))
        assert not got[1::2].any()
        host.as_numpy()[:] = 0
        b.d2h(descs, stream)
        stream.synchronize()
        assert np.array_equal(host.as_numpy(), want)
    finally:
        b.close()
        dev.close()
        host.close()


def _random_batch(rng):
    """Rows (device offset, host offset, size, host allocation) of a random
    batch: host-dense runs of small pieces, isolated pieces, now and then a
    large range; device slots are disjoint and visited in shuffled order."""
    pieces = []           # (size, host_off, alloc)
    host_cursor = int(rng.integers(0, 64))
    alloc = 1
    for _ in range(int(rng.integers(1, 6))):
        kind = int(rng.integers(0, 3))
        if kind == 0:     # a dense run
            count = int(rng.integers(2, 400))
            unit = int(rng.choice([16, 64, 1000, 4096, 4112]))
            for _ in range(count):
                size = unit if rng.integers(0, 4) else int(rng.integers(1, unit + 1))
                pieces.append((size, host_cursor, alloc))
                host_cursor += size
        elif kind == 1:   # isolated pieces with gaps between them
            for _ in range(int(rng.integers(1, 40))):
                size = int(rng.integers(1, 6000))
                host_cursor += int(rng.integers(1, 300))
                pieces.append((size, host_cursor, alloc))
                host_cursor += size
        else:             # one large range
            size = (4 << 20) + int(rng.integers(0, 4096))
            host_cursor += int(rng.integers(0, 64))
            pieces.append((size, host_cursor, alloc))
            host_cursor += size
        host_cursor += int(rng.integers(1, 5000))
        alloc += int(rng.integers(0, 2))
    # disjoint device slots, assigned in shuffled order
    order = rng.permutation(len(pieces))
    dev_cursor = int(rng.integers(0, 64))
    dev_off = [0] * len(pieces)
    for idx in order:
        dev_off[idx] = dev_cursor
        dev_cursor += pieces[idx][0] + int(rng.integers(0, 128))
    rows = [(dev_off[i], p[1], p[0], p[2]) for i, p in enumerate(pieces)]
    return rows, dev_cursor + 64, host_cursor + 64


@pytest.mark.parametrize("seed", range(12))
def test_random_descriptor_batches_match_oracle(backends, stream, seed):
    """Both backends, both directions, on seeded random batches; bytes outside
    the fragments must stay as they were."""
    from pegaflow_amd.transfer import desc_array
    rng = np.random.default_rng(7000 + seed)
    rows4, dev_bytes, host_bytes = _random_batch(rng)
    rows = [(d, h, s) for d, h, s, _a in rows4]
    d = np.array([r[0] for r in rows4], dtype=np.uint64)
    h = np.array([r[1] for r in rows4], dtype=np.uint64)
    sz = np.array([r[2] for r in rows4], dtype=np.uint64)
    al = np.array([r[3] for r in rows4], dtype=np.uint64)

    def descs(dev, host):
        return desc_array(dev.ptr + d, host.host_ptr + h, host.device_ptr + h, sz, 0, al)

    for b in backends:
        _run_both_directions(b, stream, descs, dev_bytes, host_bytes, rows, seed=seed)
