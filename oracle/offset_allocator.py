"""CPU restatement of the offset allocator behind the reference's
``ScaledOffsetAllocator`` (pegaflow-core/src/allocator.rs:63-142 wraps the
third-party crate ``offset-allocator`` 0.2.0, Cargo.lock:1703-1704, whose source
is not in the reference tree).  The crate is a port of the published
OffsetAllocator algorithm (S. Aaltonen): free regions sit in 32 x 8 bins indexed
by a small float of their size (3 mantissa bits), an allocation takes the head
of the lowest bin whose every member is large enough, the remainder goes back to
the bin of its own size, and a freed region merges with free neighbours.  This
file restates that algorithm from its published description; the tests pin it
with the known answers of the algorithm's own test suite (small-float table,
trivial / complex reuse, zero fragmentation) and then compare the product's
allocator with it offset by offset on random sequences.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``; the product never imports it.
"""

from __future__ import annotations

NUM_TOP_BINS = 32
BINS_PER_LEAF = 8
TOP_BINS_INDEX_SHIFT = 3
LEAF_BINS_INDEX_MASK = 7
NUM_LEAF_BINS = NUM_TOP_BINS * BINS_PER_LEAF
MANTISSA_BITS = 3
MANTISSA_VALUE = 1 << MANTISSA_BITS
MANTISSA_MASK = MANTISSA_VALUE - 1
NO_SPACE = 0xFFFFFFFF
UNUSED = 0xFFFFFFFF


def uint_to_float_round_up(size: int) -> int:
    """Bin whose every member is >= size."""
    exp = mantissa = 0
    if size < MANTISSA_VALUE:
        mantissa = size
    else:
        highest = size.bit_length() - 1
        start = highest - MANTISSA_BITS
        exp = start + 1
        mantissa = (size >> start) & MANTISSA_MASK
        if size & ((1 << start) - 1):
            mantissa += 1
    return (exp << MANTISSA_BITS) + mantissa  # '+': a mantissa overflow carries into the exponent


def uint_to_float_round_down(size: int) -> int:
    """Bin a free region of `size` belongs to."""
    exp = mantissa = 0
    if size < MANTISSA_VALUE:
        mantissa = size
    else:
        highest = size.bit_length() - 1
        start = highest - MANTISSA_BITS
        exp = start + 1
        mantissa = (size >> start) & MANTISSA_MASK
    return (exp << MANTISSA_BITS) | mantissa


def float_to_uint(value: int) -> int:
    exp, mantissa = value >> MANTISSA_BITS, value & MANTISSA_MASK
    if exp == 0:
        return mantissa
    return (mantissa | MANTISSA_VALUE) << (exp - 1)


def _lowest_set_bit_from(mask: int, start: int) -> int:
    bits = mask & ~((1 << start) - 1) & 0xFFFFFFFF
    if bits == 0:
        return NO_SPACE
    return (bits & -bits).bit_length() - 1


class _Node:
    __slots__ = ("offset", "size", "bin_prev", "bin_next", "nb_prev", "nb_next", "used")

    def __init__(self):
        self.offset = self.size = 0
        self.bin_prev = self.bin_next = self.nb_prev = self.nb_next = UNUSED
        self.used = False


class OffsetAllocator:
    """Offsets and sizes in units; allocate() -> (offset, node) or None."""

    def __init__(self, size: int, max_allocs: int = 128 * 1024):
        self.size = size
        self.max_allocs = max_allocs
        self.free_storage = 0
        self.used_bins_top = 0
        self.used_bins = [0] * NUM_TOP_BINS
        self.bin_heads = [UNUSED] * NUM_LEAF_BINS
        self.nodes = [_Node() for _ in range(max_allocs)]
        # a stack; node 0 is handed out first
        self.free_nodes = [max_allocs - i - 1 for i in range(max_allocs)]
        self.free_offset = max_allocs - 1
        self._insert(size, 0)

    def _insert(self, size: int, offset: int) -> int:
        b = uint_to_float_round_down(size)
        top, leaf = b >> TOP_BINS_INDEX_SHIFT, b & LEAF_BINS_INDEX_MASK
        if self.bin_heads[b] == UNUSED:
            self.used_bins[top] |= 1 << leaf
            self.used_bins_top |= 1 << top
        head = self.bin_heads[b]
        idx = self.free_nodes[self.free_offset]
        self.free_offset -= 1
        n = self.nodes[idx]
        n.offset, n.size, n.bin_next, n.bin_prev = offset, size, head, UNUSED
        n.nb_prev = n.nb_next = UNUSED
        n.used = False
        if head != UNUSED:
            self.nodes[head].bin_prev = idx
        self.bin_heads[b] = idx
        self.free_storage += size
        return idx

    def _remove(self, idx: int) -> None:
        n = self.nodes[idx]
        if n.bin_prev != UNUSED:
            self.nodes[n.bin_prev].bin_next = n.bin_next
            if n.bin_next != UNUSED:
                self.nodes[n.bin_next].bin_prev = n.bin_prev
        else:
            b = uint_to_float_round_down(n.size)
            top, leaf = b >> TOP_BINS_INDEX_SHIFT, b & LEAF_BINS_INDEX_MASK
            self.bin_heads[b] = n.bin_next
            if n.bin_next != UNUSED:
                self.nodes[n.bin_next].bin_prev = UNUSED
            if self.bin_heads[b] == UNUSED:
                self.used_bins[top] &= ~(1 << leaf)
                if self.used_bins[top] == 0:
                    self.used_bins_top &= ~(1 << top)
        self.free_offset += 1
        self.free_nodes[self.free_offset] = idx
        self.free_storage -= n.size

    def allocate(self, size: int):
        if self.free_offset == 0:  # out of bookkeeping nodes
            return None
        min_bin = uint_to_float_round_up(size)
        min_top, min_leaf = min_bin >> TOP_BINS_INDEX_SHIFT, min_bin & LEAF_BINS_INDEX_MASK
        top, leaf = min_top, NO_SPACE
        if min_top < NUM_TOP_BINS and self.used_bins_top & (1 << top):
            leaf = _lowest_set_bit_from(self.used_bins[top], min_leaf)
        if leaf == NO_SPACE:
            top = _lowest_set_bit_from(self.used_bins_top, min_top + 1) \
                if min_top + 1 < NUM_TOP_BINS else NO_SPACE
            if top == NO_SPACE:
                return None
            m = self.used_bins[top]
            leaf = (m & -m).bit_length() - 1
        b = (top << TOP_BINS_INDEX_SHIFT) | leaf
        idx = self.bin_heads[b]
        n = self.nodes[idx]
        total = n.size
        n.size = size
        n.used = True
        self.bin_heads[b] = n.bin_next
        if n.bin_next != UNUSED:
            self.nodes[n.bin_next].bin_prev = UNUSED
        self.free_storage -= total
        if self.bin_heads[b] == UNUSED:
            self.used_bins[top] &= ~(1 << leaf)
            if self.used_bins[top] == 0:
                self.used_bins_top &= ~(1 << top)
        rest = total - size
        if rest > 0:
            new = self._insert(rest, n.offset + size)
            if n.nb_next != UNUSED:
                self.nodes[n.nb_next].nb_prev = new
            self.nodes[new].nb_prev = idx
            self.nodes[new].nb_next = n.nb_next
            n.nb_next = new
        return n.offset, idx

    def free(self, idx: int) -> None:
        n = self.nodes[idx]
        assert n.used
        offset, size = n.offset, n.size
        if n.nb_prev != UNUSED and not self.nodes[n.nb_prev].used:
            p = self.nodes[n.nb_prev]
            offset = p.offset
            size += p.size
            self._remove(n.nb_prev)
            n.nb_prev = p.nb_prev
        if n.nb_next != UNUSED and not self.nodes[n.nb_next].used:
            q = self.nodes[n.nb_next]
            size += q.size
            self._remove(n.nb_next)
            n.nb_next = q.nb_next
        nb_next, nb_prev = n.nb_next, n.nb_prev
        self.free_offset += 1
        self.free_nodes[self.free_offset] = idx
        n.used = False
        merged = self._insert(size, offset)
        if nb_next != UNUSED:
            self.nodes[merged].nb_next = nb_next
            self.nodes[nb_next].nb_prev = merged
        if nb_prev != UNUSED:
            self.nodes[merged].nb_prev = nb_prev
            self.nodes[nb_prev].nb_next = merged

    def report(self):
        """(total free, lower bound of the largest free region's bin)."""
        if self.free_offset == 0:
            return 0, 0
        largest = 0
        if self.used_bins_top:
            top = self.used_bins_top.bit_length() - 1
            leaf = self.used_bins[top].bit_length() - 1
            largest = float_to_uint((top << TOP_BINS_INDEX_SHIFT) | leaf)
        return self.free_storage, largest
