"""The offset allocator under interleaved allocate / free, offset by offset.

The reference's ScaledOffsetAllocator (allocator.rs:63-142) wraps the
third-party crate offset-allocator 0.2.0 (Cargo.lock:1703-1704), whose source
is not in the reference tree.  oracle/offset_allocator.py restates the published
algorithm the crate ports; it is pinned here by the known answers of that
algorithm's own test suite (small-float table, merge / reuse cases, zero
fragmentation), and the product's allocator (pf_allocator_*, through the C ABI)
must then give the same offsets as the restatement on the same cases and on
random sequences."""

import numpy as np
import pytest

from oracle import offset_allocator as OA
from pegaflow_amd.pool import ScaledOffsetAllocator

MiB = 1 << 20
SIZE = 256 * MiB


# ---- the restatement against the algorithm's published known answers --------

def test_small_float_known_answers():
    # every value below 17 is its own bin, rounding either way
    for i in range(17):
        assert OA.uint_to_float_round_up(i) == i and OA.uint_to_float_round_down(i) == i
    for number, up, down in [(17, 17, 16), (118, 39, 38), (1024, 64, 64), (65536, 112, 112),
                             (529445, 137, 136), (1048575, 144, 143)]:
        assert OA.uint_to_float_round_up(number) == up, number
        assert OA.uint_to_float_round_down(number) == down, number


def test_small_float_round_trip():
    # every bin's lower bound maps back to the bin, both ways
    for i in range(240):
        v = OA.float_to_uint(i)
        assert OA.uint_to_float_round_up(v) == i and OA.uint_to_float_round_down(v) == i
    rng = np.random.default_rng(5)
    for v in rng.integers(1, 2**32 - 1, size=5000):
        v = int(v)
        lo, hi = OA.uint_to_float_round_down(v), OA.uint_to_float_round_up(v)
        assert OA.float_to_uint(lo) <= v <= OA.float_to_uint(hi) and hi - lo in (0, 1)


class _Oracle:
    """The restatement behind the interface of the product's wrapper (unit 1)."""

    def __init__(self, size, max_allocs=128 * 1024):
        self.a = OA.OffsetAllocator(size, max_allocs)

    def allocate(self, n):
        r = self.a.allocate(n)
        return None if r is None else r

    def offset(self, r):
        return r[0]

    def free(self, r):
        self.a.free(r[1])

    def report(self):
        return self.a.report()


class _Product:
    def __init__(self, size, max_allocs=128 * 1024):
        self.a = ScaledOffsetAllocator(size, 1, max_allocs)

    def allocate(self, n):
        return self.a.allocate(n)

    def offset(self, r):
        return r.offset_bytes

    def free(self, r):
        self.a.free(r)

    def report(self):
        rep = self.a.report()
        return rep["total_free_bytes"], rep["largest_free_allocation_bytes"]


@pytest.fixture(params=["restatement", "product"])
def make(request):
    return _Oracle if request.param == "restatement" else _Product


def test_basic_and_simple(make):
    a = make(SIZE)
    r = a.allocate(1337)
    assert a.offset(r) == 0
    a.free(r)
    b, c, d = a.allocate(1), a.allocate(123), a.allocate(1234)
    assert [a.offset(x) for x in (b, c, d)] == [0, 1, 124]
    for x in (b, c, d):
        a.free(x)
    # everything merged back: the whole range is one region again
    whole = a.allocate(SIZE)
    assert a.offset(whole) == 0


def test_merge_and_reuse_trivial(make):
    a = make(SIZE)
    x = a.allocate(1337)
    assert a.offset(x) == 0
    a.free(x)
    y = a.allocate(1337)
    assert a.offset(y) == 0            # the merged region is reused from its start
    a.free(y)
    p, q = a.allocate(1024), a.allocate(3456)
    assert (a.offset(p), a.offset(q)) == (0, 1024)
    a.free(p)
    r = a.allocate(1024)
    assert a.offset(r) == 0            # the hole fits exactly
    a.free(r)
    a.free(q)
    assert a.offset(a.allocate(SIZE)) == 0


def test_reuse_complex(make):
    a = make(SIZE)
    p, q = a.allocate(1024), a.allocate(3456)
    assert (a.offset(p), a.offset(q)) == (0, 1024)
    a.free(p)
    c = a.allocate(2345)               # too large for the 1024 hole: behind q
    assert a.offset(c) == 1024 + 3456
    d = a.allocate(456)                # the hole's head
    assert a.offset(d) == 0
    e = a.allocate(512)                # the hole's rest (568) takes it
    assert a.offset(e) == 456
    free, largest = a.report()
    assert free == SIZE - 3456 - 2345 - 456 - 512
    assert largest != free
    for x in (c, d, q, e):
        a.free(x)
    assert a.offset(a.allocate(SIZE)) == 0


def test_zero_fragmentation(make):
    a = make(SIZE)
    regions = [a.allocate(MiB) for _ in range(256)]
    assert [a.offset(r) for r in regions] == [i * MiB for i in range(256)]
    assert a.report() == (0, 0)
    for i in (243, 5, 123, 95):
        a.free(regions[i])
    for i in (151, 152, 153, 154):     # four in a row merge into one 4 MiB hole
        a.free(regions[i])
    for i in (243, 5, 123, 95):
        regions[i] = a.allocate(MiB)
        assert regions[i] is not None
    regions[151] = a.allocate(4 * MiB)
    assert regions[151] is not None and a.offset(regions[151]) == 151 * MiB
    for i, r in enumerate(regions):
        if i not in (152, 153, 154):
            a.free(r)
    assert a.report() == (SIZE, SIZE)
    assert a.offset(a.allocate(SIZE)) == 0


# ---- the product against the restatement, offset by offset -------------------

@pytest.mark.parametrize("unit,units,max_allocs,sizes,seed", [
    (1, 1 << 20, 1 << 16, [1, 7, 8, 9, 100, 1000, 4096, 65536], 1),
    (512, 1 << 16, 1 << 16, [1, 511, 512, 513, 4096, 32768, 100000, 1 << 20], 2),
    (4096, 1 << 14, 1 << 12, [4096, 8192, 65536, 73728, 1 << 20], 3),
    (512, 4096, 64, [512, 1024, 4096, 65536], 4),   # few bookkeeping nodes: runs out of them
])
def test_product_gives_the_offsets_of_the_restatement(unit, units, max_allocs, sizes, seed):
    rng = np.random.default_rng(seed)
    product = ScaledOffsetAllocator(unit * units, unit, max_allocs)
    oracle = OA.OffsetAllocator(units, max_allocs)
    live = []
    refused = 0
    for step in range(20000):
        if live and rng.random() < 0.48:
            pr, node = live.pop(int(rng.integers(len(live))))
            product.free(pr)
            oracle.free(node)
        else:
            want = int(rng.choice(sizes))
            n_units = -(-want // unit)
            got = product.allocate(want)
            expect = oracle.allocate(n_units)
            if expect is None:
                assert got is None, (step, want)
                refused += 1
                continue
            assert got is not None, (step, want)
            assert got.offset_bytes == expect[0] * unit, (step, want)
            assert got.size_bytes == n_units * unit
            live.append((got, expect[1]))
        if step % 64 == 0:
            rep = product.report()
            free, largest = oracle.report()
            assert rep["total_free_bytes"] == free * unit
            assert rep["largest_free_allocation_bytes"] == largest * unit
    assert len(live) > 0
    if max_allocs == 64:
        assert refused > 0
    product.close()
