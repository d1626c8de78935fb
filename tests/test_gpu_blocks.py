"""GPU parity of the block-ID gather/scatter path (pf_xfer_save / pf_xfer_load)
against the CPU oracle, for both link paths (zero-copy and staged) and every
layout the reference supports: K/V split, contiguous (MLA), adjacent K/V,
strided fused buffer, padded host strides, page-first pages."""

import zlib

import numpy as np
import pytest

from oracle import oracle as O
from pegaflow_amd import _lib
from pegaflow_amd.layout import KVCacheLayout
from pegaflow_amd.runtime import DeviceBuffer, Event, PinnedMemory, Stream
from pegaflow_amd.transfer import BlockTransfer, LayerBlocks, TransferPath
from tests.helpers import random_bytes

pytestmark = pytest.mark.gpu

ZC, ST = TransferPath.ZEROCOPY, TransferPath.STAGED
SENT = 0xC3


@pytest.fixture(scope="module")
def stream(gpu):
    s = Stream()
    yield s
    s.close()


@pytest.fixture(scope="module")
def xfer(gpu):
    # Small staging slots so that modest test sizes already span several
    # units and reuse slots.
    x = BlockTransfer(staging_slot_bytes=1 << 20, staging_slots=2, auto_staged_min_bytes=4 << 20)
    yield x
    x.close()


class Case:
    """One layer: device cache + host image, mirrored for product and oracle."""

    def __init__(self, rng, num_blocks, seg, segments, kv_stride=None, block_stride=None,
                 pad_to=None, n_ids=None, base_off=0):
        self.seg, self.segments, self.num_blocks = seg, segments, num_blocks
        if segments == 2 and kv_stride is None:
            kv_stride = num_blocks * (block_stride or seg)
        kv = kv_stride or 0
        probe = O.Layout(0x1000, 1 << 40, num_blocks, seg, kv, segments)
        if block_stride:
            probe.with_block_stride(block_stride)
        stride = probe.c.block_stride_bytes
        frag = probe.fragment_bytes
        self.size = (num_blocks - 1) * stride + frag + (kv if probe.is_split else 0)
        self.base_off = base_off
        self.cache0 = random_bytes(rng, self.size + base_off)
        self.dev = DeviceBuffer(self.size + base_off)
        self.args = (self.size, num_blocks, seg, kv, segments)
        self.block_stride = block_stride
        self.pad_to = pad_to
        n_ids = n_ids if n_ids is not None else max(1, num_blocks // 2)
        self.ids = rng.choice(num_blocks, n_ids, replace=False).astype(np.uint32)

    def product_layout(self):
        L = KVCacheLayout(self.dev.ptr + self.base_off, *self.args)
        if self.block_stride:
            L.with_block_stride(self.block_stride)
        if self.pad_to:
            L.with_ssd_padding(self.pad_to)
        return L

    def oracle_layout(self, cache):
        L = O.Layout(cache.ctypes.data + self.base_off, *self.args)
        if self.block_stride:
            L.with_block_stride(self.block_stride)
        if self.pad_to:
            L.with_ssd_padding(self.pad_to)
        return L

    def close(self):
        self.dev.close()


def _dense_layer(case, L, host, ids):
    """LayerBlocks over the layer-first batch image: K buffer then V buffer."""
    n = len(ids)
    stride = L.host_stride
    nseg = 2 if L.is_split else 1
    buf = n * stride
    return LayerBlocks(
        layout=L, block_ids=ids,
        host=tuple(host.host_ptr + s * buf for s in range(nseg)),
        host_device=tuple(host.device_ptr + s * buf for s in range(nseg)),
        host_len=tuple(buf for _ in range(nseg)), host_stride=stride, layer_name="layer_0")


def _roundtrip(case, xfer, stream, path):
    L = case.product_layout()
    n = len(case.ids)
    stride = L.host_stride
    nseg = 2 if L.is_split else 1
    buf = n * stride
    host = PinnedMemory(nseg * buf)
    hv = host.as_numpy()

    # ---- save: device -> host image, compare with the oracle ------------
    case.dev.copy_from_host(case.cache0)
    hv[:] = SENT
    xfer.save([_dense_layer(case, L, host, case.ids)], stream, path)
    stream.synchronize()
    assert xfer.last_path == path
    ocache = case.cache0.copy()
    oL = case.oracle_layout(ocache)
    ok = np.full(buf, SENT, dtype=np.uint8)
    ov = np.full(buf, SENT, dtype=np.uint8) if nseg == 2 else None
    O.transfer_layer(oL, case.ids, ok, ov, host_is_src=False)
    assert np.array_equal(hv[:buf], ok), "saved K/contiguous image differs from the oracle"
    if nseg == 2:
        assert np.array_equal(hv[buf:], ov), "saved V image differs from the oracle"
    assert np.array_equal(case.dev.copy_to_host(), case.cache0), "save modified device memory"

    # ---- load: host image -> other device slots, compare whole cache ----
    rng = np.random.default_rng(int(case.ids.sum()) + 1)
    dest = rng.choice(case.num_blocks, n, replace=False).astype(np.uint32)
    case.dev.fill(SENT)
    xfer.load([_dense_layer(case, L, host, dest)], stream, path)
    stream.synchronize()
    ocache2 = np.full_like(case.cache0, SENT)
    oL2 = case.oracle_layout(ocache2)
    O.transfer_layer(oL2, dest, ok, ov, host_is_src=True)
    assert np.array_equal(case.dev.copy_to_host(), ocache2), "loaded cache differs from the oracle"
    host.close()


LAYOUTS = {
    # name: kwargs of Case
    "llama_split_32k": dict(num_blocks=96, seg=32768, segments=2),
    "fp8_split_16k": dict(num_blocks=128, seg=16384, segments=2),
    "mla_contiguous_72k": dict(num_blocks=48, seg=73728, segments=1),
    "adjacent_kv": dict(num_blocks=64, seg=8192, segments=2, kv_stride=8192),
    "fused_strided": dict(num_blocks=40, seg=8192, segments=1, block_stride=16384),
    # V segments interleaved between the K segments of a strided buffer
    "sparse_split": dict(num_blocks=32, seg=4096, segments=2, kv_stride=139264, block_stride=16384),
    "tail_4112": dict(num_blocks=70, seg=4112, segments=2),
    "tiny_528": dict(num_blocks=300, seg=528, segments=1, n_ids=300),
    "odd_size_1000": dict(num_blocks=50, seg=1000, segments=2),
    "misaligned_base": dict(num_blocks=50, seg=4096, segments=2, base_off=4),
    # more list positions than one tile launch can index (65535): the staged path splits units
    "many_tiny_64": dict(num_blocks=70000, seg=64, segments=1, n_ids=70000),
    # zero-copy lists short enough to travel in the launch's arguments: as 32-bit ids
    # (850 fill the argument slab to the last byte), as 16-bit ids (an odd count, so
    # the last word is half used), and too long or too large for either form
    "args_ids32_850": dict(num_blocks=4096, seg=2048, segments=2, n_ids=850),
    "args_ids16_1001": dict(num_blocks=4096, seg=2048, segments=2, n_ids=1001),
    "args_ids16_1791": dict(num_blocks=4096, seg=1024, segments=1, n_ids=1791),
    "slab_ids16_too_many_1800": dict(num_blocks=4096, seg=1024, segments=1, n_ids=1800),
    "slab_ids_over_65535": dict(num_blocks=70000, seg=256, segments=1, n_ids=1001),
}


@pytest.mark.parametrize("path", [ZC, ST], ids=["zerocopy", "staged"])
@pytest.mark.parametrize("name", sorted(LAYOUTS))
def test_save_load_matches_oracle(name, path, xfer, stream):
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    case = Case(rng, **LAYOUTS[name])
    try:
        _roundtrip(case, xfer, stream, path)
    finally:
        case.close()


def _random_case_kwargs(rng):
    """A valid layout drawn at random: contiguous or split, dense / strided /
    interleaved, aligned or not, fragment sizes with and without a 16-byte
    tail, sometimes padded host strides and a misaligned base."""
    segments = int(rng.integers(1, 3))
    seg = int(rng.choice([64, 528, 1000, 4096, 4112, 12288, 40000]))
    num_blocks = int(rng.integers(2, 120))
    kw = dict(num_blocks=num_blocks, seg=seg, segments=segments)
    shape = int(rng.integers(0, 4))
    if segments == 2 and shape == 1:
        kw["kv_stride"] = seg                       # adjacent K/V: collapses to contiguous
    elif segments == 2 and shape == 2:
        stride = seg * 4                            # V between the K segments of a strided buffer
        kw["block_stride"] = stride
        kw["kv_stride"] = stride * num_blocks + 2 * seg
    elif segments == 1 and shape in (1, 2):
        kw["block_stride"] = seg * int(rng.integers(2, 4))
    if rng.integers(0, 4) == 0:
        kw["pad_to"] = 512
    if rng.integers(0, 5) == 0:
        kw["base_off"] = int(rng.choice([4, 16, 3]))
    kw["n_ids"] = int(rng.integers(1, num_blocks + 1))
    return kw


@pytest.mark.parametrize("seed", range(24))
def test_random_layouts_match_oracle(seed, xfer, stream):
    """Seeded random layouts and id lists through both link paths against the
    oracle (save image, untouched device memory, load into other slots)."""
    rng = np.random.default_rng(1000 + seed)
    kw = _random_case_kwargs(rng)
    case = Case(rng, **kw)
    try:
        L = case.product_layout()
        dense = L.host_stride == L.fragment_bytes     # the staged path needs a dense host image
        for path in (ZC, ST) if dense else (ZC,):
            _roundtrip(case, xfer, stream, path)
    except AssertionError as exc:
        raise AssertionError(f"{kw}: {exc}") from exc
    finally:
        case.close()


@pytest.mark.parametrize("kw", [
    dict(num_blocks=60, seg=8848, segments=2, pad_to=512),
    # fragment size not a multiple of 16 while every fragment START is aligned:
    # the 16-byte vector path with a bytewise tail
    dict(num_blocks=40, seg=1000, segments=1, block_stride=1024, pad_to=512),
], ids=["split_8848_to_9216", "contiguous_1000_to_1024"])
def test_padded_host_stride_leaves_padding_untouched(kw, xfer, stream):
    """SSD padding: the host stride is the segment size rounded up to 512;
    copies use the unpadded size and the pad tail is never written
    (layout.rs:157-160, offload.rs:472-474).  The staged path needs a dense
    image and must refuse; zero-copy and AUTO must work."""
    rng = np.random.default_rng(77)
    case = Case(rng, **kw)
    L = case.product_layout()
    seg, stride = L.fragment_bytes, L.host_stride
    assert stride > seg and stride % 512 == 0
    nseg = 2 if L.is_split else 1
    host = PinnedMemory(nseg * len(case.ids) * stride)
    with pytest.raises(_lib.InvalidArgument, match="dense host image"):
        xfer.save([_dense_layer(case, L, host, case.ids)], stream, ST)
    _roundtrip(case, xfer, stream, ZC)
    # AUTO picks zero-copy for a non-dense image
    host.as_numpy()[:] = SENT
    case.dev.copy_from_host(case.cache0)
    xfer.save([_dense_layer(case, L, host, case.ids)], stream, TransferPath.AUTO)
    stream.synchronize()
    assert xfer.last_path == ZC
    img = host.as_numpy().reshape(nseg, len(case.ids), stride)
    assert (img[:, :, seg:] == SENT).all()
    assert not (img[:, :, :seg] == SENT).all()
    host.close()
    case.close()


def test_page_first_pages(xfer, stream):
    """Page-first host layout: one page per block, each layer at its own byte
    offset (instance.rs:107-162, offload.rs:182-282).  Three layers of
    distinct sizes 512/1024/1536 -> offsets 0/512/1536 as in the reference's
    page_first_multi_layer_roundtrip."""
    rng = np.random.default_rng(5)
    sizes = [512, 1024, 1536]
    placement = O.build_page_layout([[0, 1, 2]], 3, sizes)
    assert placement["layer_offsets"] == [0, 512, 1536]
    page = placement["shard_page_sizes"][0]
    num_blocks, n = 16, 11
    ids = rng.choice(num_blocks, n, replace=False).astype(np.uint32)
    # pages deliberately not in address order and not evenly spaced
    slots = rng.permutation(2 * n)[:n]
    pool = PinnedMemory(2 * n * page)
    pool.as_numpy()[:] = SENT
    page_host = np.array([pool.host_ptr + int(s) * page for s in slots], dtype=np.uint64)
    page_dev = np.array([pool.device_ptr + int(s) * page for s in slots], dtype=np.uint64)
    cases = [Case(rng, num_blocks=num_blocks, seg=sz, segments=1) for sz in sizes]
    layers = []
    for li, c in enumerate(cases):
        c.dev.copy_from_host(c.cache0)
        layers.append(LayerBlocks(layout=c.product_layout(), block_ids=ids, page_host=page_host,
                                  page_host_device=page_dev,
                                  page_offset=placement["layer_offsets"][li], page_len=page,
                                  layer_name=f"layer_{li}"))
    xfer.save(layers, stream, TransferPath.AUTO)
    stream.synchronize()
    assert xfer.last_path == ZC
    # oracle on a host-resident pool image
    opool = np.full(2 * n * page, SENT, dtype=np.uint8)
    opages = np.array([opool.ctypes.data + int(s) * page for s in slots], dtype=np.uint64)
    for li, c in enumerate(cases):
        oc = c.cache0.copy()
        O.transfer_layer_paged(c.oracle_layout(oc), ids, opages, placement["layer_offsets"][li],
                               host_is_src=False)
    assert np.array_equal(pool.as_numpy(), opool)
    # load back into permuted slots
    dest = rng.choice(num_blocks, n, replace=False).astype(np.uint32)
    for li, c in enumerate(cases):
        c.dev.fill(SENT)
        layers[li].block_ids = dest
    xfer.load(layers, stream, TransferPath.AUTO)
    stream.synchronize()
    for li, c in enumerate(cases):
        oc = np.full_like(c.cache0, SENT)
        O.transfer_layer_paged(c.oracle_layout(oc), dest, opages, placement["layer_offsets"][li],
                               host_is_src=True)
        assert np.array_equal(c.dev.copy_to_host(), oc), li
        c.close()
    pool.close()


def test_multi_layer_batch_with_layer_events_and_empty_layer(xfer, stream):
    """Several layers in one call, one of them empty; per-layer events all
    fire; mixed paths in one call."""
    rng = np.random.default_rng(13)
    cases = [Case(rng, num_blocks=64, seg=32768, segments=2, n_ids=40),
             Case(rng, num_blocks=64, seg=4096, segments=2, n_ids=1),
             Case(rng, num_blocks=64, seg=16384, segments=1, n_ids=30)]
    cases[1].ids = np.zeros(0, dtype=np.uint32)  # empty layer
    hosts, layers, Ls = [], [], []
    for c in cases:
        L = c.product_layout()
        Ls.append(L)
        nseg = 2 if L.is_split else 1
        h = PinnedMemory(max(1, nseg * len(c.ids) * L.host_stride))
        h.as_numpy()[:] = SENT
        hosts.append(h)
        c.dev.copy_from_host(c.cache0)
        layers.append(_dense_layer(c, L, h, c.ids))
    events = [Event() for _ in cases]
    big = BlockTransfer(staging_slot_bytes=1 << 20, staging_slots=2, auto_staged_min_bytes=1 << 20)
    big.set_layer_events(events)
    big.save(layers, stream, TransferPath.AUTO)
    for e in events:
        e.synchronize()
    stream.synchronize()
    assert all(e.query() for e in events)
    for c, L, h in zip(cases, Ls, hosts):
        if len(c.ids) == 0:
            continue
        n, stride = len(c.ids), L.host_stride
        oc = c.cache0.copy()
        ok = np.full(n * stride, SENT, dtype=np.uint8)
        ov = np.full(n * stride, SENT, dtype=np.uint8) if L.is_split else None
        O.transfer_layer(c.oracle_layout(oc), c.ids, ok, ov, host_is_src=False)
        hv = h.as_numpy()
        assert np.array_equal(hv[: n * stride], ok)
        if ov is not None:
            assert np.array_equal(hv[n * stride: 2 * n * stride], ov)
    big.set_layer_events(None)
    big.close()
    for c, h in zip(cases, hosts):
        c.close()
        h.close()


def test_errors_are_reported_before_anything_is_enqueued(xfer, stream):
    rng = np.random.default_rng(2)
    case = Case(rng, num_blocks=16, seg=4096, segments=2, n_ids=4)
    L = case.product_layout()
    host = PinnedMemory(2 * 4 * 4096)
    host.as_numpy()[:] = SENT
    bad = _dense_layer(case, L, host, np.array([1, 2, 16, 3], dtype=np.uint32))
    bad.layer_name = "model.layers.7"
    with pytest.raises(_lib.StorageError,
                       match=r"layer model.layers.7: block 16 out of range \(16 blocks\)"):
        xfer.save([bad], stream)
    short = _dense_layer(case, L, host, case.ids)
    short.host_len = (4 * 4096 - 1, 4 * 4096)
    with pytest.raises(_lib.InvalidArgument, match="needs 16384 bytes, has 16383"):
        xfer.save([short], stream)
    stream.synchronize()
    assert (host.as_numpy() == SENT).all()
    # zero layers / zero blocks are fine
    xfer.save([], stream)
    xfer.load([_dense_layer(case, L, host, np.zeros(0, dtype=np.uint32))], stream)
    stream.synchronize()
    host.close()
    case.close()


def test_duplicate_source_ids_get_their_own_host_image(xfer, stream):
    """Duplicate block ids in one save list are not rejected; each occurrence
    gets its own host image (offload.rs:348-360)."""
    rng = np.random.default_rng(21)
    case = Case(rng, num_blocks=8, seg=4096, segments=2, n_ids=1)
    case.ids = np.array([3, 3, 5, 3], dtype=np.uint32)
    L = case.product_layout()
    host = PinnedMemory(2 * 4 * 4096)
    case.dev.copy_from_host(case.cache0)
    for path in (ZC, ST):
        host.as_numpy()[:] = SENT
        xfer.save([_dense_layer(case, L, host, case.ids)], stream, path)
        stream.synchronize()
        ek, ev = O.np_save_split(case.cache0, 8, 4096, case.ids)
        img = host.as_numpy().reshape(2, 4, 4096)
        assert np.array_equal(img[0], ek) and np.array_equal(img[1], ev)
    host.close()
    case.close()


def _paged_setup(rng, sizes, num_blocks, n, page_gap_after=None, stride_extra=0):
    """Layers of `sizes` bytes per block over pages laid back to back (with an
    optional hole after position `page_gap_after`)."""
    offsets = np.concatenate([[0], np.cumsum(sizes)[:-1]]).astype(int)
    page = int(sum(sizes)) + stride_extra
    hole = 3 if page_gap_after is not None else 0
    pool = PinnedMemory((n + hole) * page)
    pool.as_numpy()[:] = SENT
    idx = np.arange(n)
    if page_gap_after is not None:
        idx = np.where(idx > page_gap_after, idx + hole, idx)
    page_host = (pool.host_ptr + idx * page).astype(np.uint64)
    page_dev = (pool.device_ptr + idx * page).astype(np.uint64)
    ids = rng.choice(num_blocks, n, replace=False).astype(np.uint32)
    cases = [Case(rng, num_blocks=num_blocks, seg=int(sz), segments=1) for sz in sizes]
    return offsets, page, pool, idx, page_host, page_dev, ids, cases


@pytest.mark.parametrize("variant", ["aligned", "two_runs", "unaligned_slices", "unlike_slices"])
def test_page_first_whole_page_packing(variant, xfer, stream):
    """Page-first layers that tile contiguous pages go through staging as whole
    pages (several staging units, slot reuse), byte-exact against the oracle;
    AUTO picks that path, ZEROCOPY must give the same bytes.  `unlike_slices`:
    72 KiB and 8 KiB slices in one page, which go out as two launches per
    chunk, the large slices and the small ones."""
    rng = np.random.default_rng(61)
    sizes = {"aligned": [512, 1024, 1536, 4096], "two_runs": [4096, 2048, 1024],
             "unaligned_slices": [1000, 520, 24, 3000],
             "unlike_slices": [73728, 8192, 73728, 8192, 8192]}[variant]
    n = 1000  # x page bytes >= 4 MiB, the AUTO threshold for staging
    gap = 400 if variant == "two_runs" else None
    offsets, page, pool, idx, page_host, page_dev, ids, cases = _paged_setup(
        rng, sizes, num_blocks=1024, n=n, page_gap_after=gap)
    layers = []
    for li, c in enumerate(cases):
        c.dev.copy_from_host(c.cache0)
        layers.append(LayerBlocks(layout=c.product_layout(), block_ids=ids, page_host=page_host,
                                  page_host_device=page_dev, page_offset=int(offsets[li]),
                                  page_len=page, layer_name=f"layer_{li}"))
    opool = np.full(pool.size, SENT, dtype=np.uint8)
    opages = (opool.ctypes.data + idx * page).astype(np.uint64)
    for li, c in enumerate(cases):
        oc = c.cache0.copy()  # keep the oracle's "device" image alive across the call
        O.transfer_layer_paged(c.oracle_layout(oc), ids, opages, int(offsets[li]),
                               host_is_src=False)
    for path, expect_path in ((TransferPath.AUTO, ST), (ST, ST), (ZC, ZC)):
        pool.as_numpy()[:] = SENT
        xfer.save(layers, stream, path)
        stream.synchronize()
        assert xfer.last_path == expect_path
        assert np.array_equal(pool.as_numpy(), opool), (variant, path)
    dest = rng.choice(1024, n, replace=False).astype(np.uint32)
    for path in (TransferPath.AUTO, ZC):
        for li, c in enumerate(cases):
            c.dev.fill(SENT)
            layers[li].block_ids = dest
        xfer.load(layers, stream, path)
        stream.synchronize()
        for li, c in enumerate(cases):
            oc = np.full_like(c.cache0, SENT)
            O.transfer_layer_paged(c.oracle_layout(oc), dest, opages, int(offsets[li]),
                                   host_is_src=True)
            assert np.array_equal(c.dev.copy_to_host(), oc), (variant, path, li)
    for c in cases:
        c.close()
    pool.close()


def test_page_packing_is_refused_when_it_would_touch_foreign_bytes(xfer, stream):
    """A save that covers only part of each page must not drain whole pages
    (the rest of the page belongs to someone else); a load of most of a page may
    read the whole page."""
    rng = np.random.default_rng(62)
    sizes = [4096] * 10
    n = 600
    offsets, page, pool, idx, page_host, page_dev, ids, cases = _paged_setup(
        rng, sizes, num_blocks=700, n=n)

    def layers_for(which, block_ids):
        out = []
        for li in which:
            out.append(LayerBlocks(layout=cases[li].product_layout(), block_ids=block_ids,
                                   page_host=page_host, page_host_device=page_dev,
                                   page_offset=int(offsets[li]), page_len=page,
                                   layer_name=f"layer_{li}"))
        return out

    for c in cases:
        c.dev.copy_from_host(c.cache0)
    subset = [0, 1, 2, 3, 4, 6, 7, 8, 9]  # layer 5 is missing: a hole in every page
    with pytest.raises(_lib.InvalidArgument, match="tile contiguous pages"):
        xfer.save(layers_for(subset, ids), stream, ST)
    xfer.save(layers_for(subset, ids), stream, TransferPath.AUTO)
    stream.synchronize()
    assert xfer.last_path == ZC
    img = pool.as_numpy().reshape(n, page)
    assert (img[:, 5 * 4096: 6 * 4096] == SENT).all(), "bytes of the missing layer were written"
    # fill in layer 5 too, then load the 9-of-10 subset: packing allowed (reads only)
    xfer.save(layers_for([5], ids), stream, TransferPath.AUTO)
    stream.synchronize()
    dest = rng.choice(700, n, replace=False).astype(np.uint32)
    for c in cases:
        c.dev.fill(SENT)
    xfer.load(layers_for(subset, dest), stream, TransferPath.AUTO)
    stream.synchronize()
    assert xfer.last_path == ST
    opages = (pool.host_ptr + idx * page).astype(np.uint64)
    for li, c in enumerate(cases):
        oc = np.full_like(c.cache0, SENT)
        if li in subset:
            O.transfer_layer_paged(c.oracle_layout(oc), dest, opages, int(offsets[li]),
                                   host_is_src=True)
        assert np.array_equal(c.dev.copy_to_host(), oc), li
    for c in cases:
        c.close()
    pool.close()


@pytest.mark.parametrize("copy_stream", [0, 2], ids=["side_stream", "in_order"])
def test_small_staged_layers_share_slots_and_launches(stream, copy_stream):
    """Staged layers that are small share a staging slot and one gather /
    scatter launch per group.  Nine layers of unlike shapes in one call -
    split and contiguous, 4 KiB to 48 KiB fragments, one with a size that is
    no multiple of 16, one empty, counts from 1 to 300 - so that groups close
    on the unit count and on the byte cap; checked against the oracle both
    ways, with per-layer events and untouched bytes."""
    rng = np.random.default_rng(77)
    shapes = [dict(num_blocks=512, seg=32768, segments=2, n_ids=300),   # 18.75 MiB: fills most of a group
              dict(num_blocks=256, seg=16384, segments=2, n_ids=200),   # closes the first group on bytes
              dict(num_blocks=128, seg=4096, segments=2, n_ids=97),
              dict(num_blocks=64, seg=49152, segments=1, n_ids=33),
              dict(num_blocks=64, seg=4104, segments=2, n_ids=20),      # byte tail in every fragment
              dict(num_blocks=64, seg=8192, segments=2, n_ids=1),
              dict(num_blocks=64, seg=8192, segments=1, n_ids=1),
              dict(num_blocks=300, seg=16384, segments=2, n_ids=299),
              dict(num_blocks=128, seg=32768, segments=1, n_ids=128)]
    cases = [Case(rng, **kw) for kw in shapes]
    cases[6].ids = np.zeros(0, dtype=np.uint32)                          # an empty layer inside a group
    # One pinned pool, the layers' images one behind the other as the engine's
    # allocations of one save are: even layers have V right behind K and start
    # right behind the layer before (pieces that cross the link as one copy),
    # odd ones keep a gap before V and after themselves.
    sizes = []
    for li, c in enumerate(cases):
        L = c.product_layout()
        nseg = 2 if L.is_split else 1
        sizes.append(nseg * len(c.ids) * L.host_stride + (0 if li % 2 == 0 else 2 * 4096))
    pool = PinnedMemory(sum(sizes) + 4096)
    pool.as_numpy()[:] = SENT
    hosts, layers, Ls = [], [], []
    cursor = 0
    for li, c in enumerate(cases):
        L = c.product_layout()
        Ls.append(L)
        nseg = 2 if L.is_split else 1
        gap = 0 if li % 2 == 0 else 4096
        n, stride = len(c.ids), L.host_stride
        buf = n * stride
        hosts.append((cursor, gap))
        c.dev.copy_from_host(c.cache0)
        lb = LayerBlocks(
            layout=L, block_ids=c.ids,
            host=tuple(pool.host_ptr + cursor + s_ * (buf + gap) for s_ in range(nseg)),
            host_device=tuple(pool.device_ptr + cursor + s_ * (buf + gap) for s_ in range(nseg)),
            host_len=tuple(buf for _ in range(nseg)), host_stride=stride, layer_name=f"layer_{li}")
        layers.append(lb)
        cursor += sizes[li]
    xfer = BlockTransfer(auto_staged_min_bytes=1, copy_stream=copy_stream)
    events = [Event() for _ in cases]
    xfer.set_layer_events(events)
    xfer.save(layers, stream, TransferPath.AUTO)
    for e in events:
        e.synchronize()
    stream.synchronize()
    assert xfer.last_path == ST
    images = []
    expect_pool = np.full(pool.as_numpy().size, SENT, dtype=np.uint8)
    for c, L, (at, gap) in zip(cases, Ls, hosts):
        n, stride = len(c.ids), L.host_stride
        if n == 0:
            images.append((None, None))
            continue
        oc = c.cache0.copy()
        ok = np.full(n * stride, SENT, dtype=np.uint8)
        ov = np.full(n * stride, SENT, dtype=np.uint8) if L.is_split else None
        O.transfer_layer(c.oracle_layout(oc), c.ids, ok, ov, host_is_src=False)
        expect_pool[at: at + n * stride] = ok
        if ov is not None:
            expect_pool[at + n * stride + gap: at + 2 * n * stride + gap] = ov
        hv = pool.as_numpy()[at:]
        assert np.array_equal(hv[: n * stride], ok), c.args
        if ov is not None:
            assert (hv[n * stride: n * stride + gap] == SENT).all()
            assert np.array_equal(hv[n * stride + gap: 2 * n * stride + gap], ov), c.args
        images.append((ok, ov))
    assert np.array_equal(pool.as_numpy(), expect_pool)      # gaps and the pool's tail untouched
    # load into other slots of sentinel-filled caches
    for li, c in enumerate(cases):
        c.dev.fill(SENT)
        if len(c.ids):
            layers[li].block_ids = rng.choice(c.num_blocks, len(c.ids), replace=False).astype(np.uint32)
    xfer.load(layers, stream, TransferPath.AUTO)
    for e in events:
        e.synchronize()
    stream.synchronize()
    for li, (c, L) in enumerate(zip(cases, Ls)):
        oc = np.full_like(c.cache0, SENT)
        if len(c.ids):
            ok, ov = images[li]
            O.transfer_layer(c.oracle_layout(oc), layers[li].block_ids, ok, ov, host_is_src=True)
        assert np.array_equal(c.dev.copy_to_host(), oc), li
    xfer.set_layer_events(None)
    xfer.close()
    for c in cases:
        c.close()
    pool.close()


@pytest.mark.parametrize("kind", ["mixed", "contiguous"])
@pytest.mark.parametrize("copy_stream", [0, 2], ids=["side_stream", "in_order"])
def test_layers_split_across_staging_slot_fills(stream, copy_stream, kind):
    """Without per-layer events a staging slot is filled to the brim: whole
    layers while they fit, then the head of the next layer, whose tail opens
    the following fill.  Five layers of 40, 40, 24, 52 and 2 MiB in 64 MiB
    slots make three fills per direction - [L0, head of L1], [tail of L1, L2,
    head of L3], [tail of L3, L4] - with split and contiguous layers, unlike
    fragment sizes and unlike row counts inside one launch.  Bytes against the
    oracle both ways, the launch count, and the same call with per-layer
    events (no layer split, one more fill)."""
    rng = np.random.default_rng(4242)
    shapes = [dict(num_blocks=700, seg=32768, segments=2, n_ids=640),     # 40 MiB
              dict(num_blocks=1400, seg=32768, segments=1, n_ids=1280),   # 40 MiB, contiguous
              dict(num_blocks=800, seg=16384, segments=2, n_ids=768),     # 24 MiB
              dict(num_blocks=900, seg=32768, segments=2, n_ids=832),     # 52 MiB
              dict(num_blocks=64, seg=16400, segments=2, n_ids=61)]       # ~2 MiB, fragments with a tail
    if kind == "contiguous":
        # the same sizes with one segment per block everywhere (MLA-like): the
        # one-segment form of the launch
        shapes = [dict(kw, seg=kw["seg"] * kw["segments"], segments=1) for kw in shapes]
    cases = [Case(rng, **kw) for kw in shapes]
    hosts, layers, Ls = [], [], []
    for c in cases:
        L = c.product_layout()
        Ls.append(L)
        nseg = 2 if L.is_split else 1
        h = PinnedMemory(nseg * len(c.ids) * L.host_stride)
        h.as_numpy()[:] = SENT
        hosts.append(h)
        c.dev.copy_from_host(c.cache0)
        layers.append(_dense_layer(c, L, h, c.ids))
    xfer = BlockTransfer(staging_slot_bytes=64 << 20, staging_slots=2, auto_staged_min_bytes=1,
                         copy_stream=copy_stream)
    xfer.set_kernel_timing(1)
    xfer.save(layers, stream, TransferPath.STAGED)
    stream.synchronize()
    assert xfer.last_path == ST
    assert xfer.last_kernel_ms()[1] == 3
    images = []
    for c, L, h in zip(cases, Ls, hosts):
        n, stride = len(c.ids), L.host_stride
        oc = c.cache0.copy()
        ok = np.full(n * stride, SENT, dtype=np.uint8)
        ov = np.full(n * stride, SENT, dtype=np.uint8) if L.is_split else None
        O.transfer_layer(c.oracle_layout(oc), c.ids, ok, ov, host_is_src=False)
        hv = h.as_numpy()
        assert np.array_equal(hv[: n * stride], ok), c.args
        if ov is not None:
            assert np.array_equal(hv[n * stride:], ov), c.args
        images.append((ok, ov))

    def load_and_check(want_launches):
        for li, c in enumerate(cases):
            c.dev.fill(SENT)
            layers[li].block_ids = rng.choice(c.num_blocks, len(c.ids), replace=False).astype(np.uint32)
        xfer.load(layers, stream, TransferPath.STAGED)
        stream.synchronize()
        assert xfer.last_kernel_ms()[1] == want_launches
        for li, c in enumerate(cases):
            oc = np.full_like(c.cache0, SENT)
            ok, ov = images[li]
            O.transfer_layer(c.oracle_layout(oc), layers[li].block_ids, ok, ov, host_is_src=True)
            assert np.array_equal(c.dev.copy_to_host(), oc), li

    load_and_check(3)
    # Per-layer events: a layer's event fires behind the fill that completes it,
    # so layers stay whole and small ones share fills of at most 32 MiB:
    # [L0] [L1] [L2] [L3] [L4].
    events = [Event() for _ in cases]
    xfer.set_layer_events(events)
    load_and_check(5)
    for e in events:
        e.synchronize()
    xfer.set_layer_events(None)
    xfer.close()
    for c, h in zip(cases, hosts):
        c.close()
        h.close()


@pytest.mark.parametrize("seed", range(4))
def test_launches_follow_the_planner_on_random_calls(stream, seed):
    """Random calls of 3-7 layers of 1-50 MiB (split and contiguous, 4-64 KiB
    fragments) in 64 MiB slots: the number of gather and of scatter launches is
    the number of fills pf_plan_staged_fills gives for the call, and the bytes
    are the oracle's."""
    from pegaflow_amd.transfer import plan_staged_fills
    rng = np.random.default_rng(9000 + seed)
    cases = []
    for _ in range(int(rng.integers(3, 8))):
        segments = int(rng.choice([1, 2]))
        seg = int(rng.choice([4096, 16384, 32768, 65536]))
        payload = int(rng.integers(1 << 20, 50 << 20))
        n_ids = max(1, payload // (seg * segments))
        cases.append(Case(rng, num_blocks=n_ids + int(rng.integers(1, 64)), seg=seg, segments=segments,
                          n_ids=n_ids))
    hosts, layers, Ls = [], [], []
    for c in cases:
        L = c.product_layout()
        Ls.append(L)
        nseg = 2 if L.is_split else 1
        h = PinnedMemory(nseg * len(c.ids) * L.host_stride)
        h.as_numpy()[:] = SENT
        hosts.append(h)
        c.dev.copy_from_host(c.cache0)
        layers.append(_dense_layer(c, L, h, c.ids))
    _units, fills = plan_staged_fills([len(c.ids) for c in cases],
                                      [L.host_stride * (2 if L.is_split else 1) for L in Ls],
                                      staging_slot_bytes=64 << 20)
    xfer = BlockTransfer(staging_slot_bytes=64 << 20, staging_slots=2, auto_staged_min_bytes=1)
    xfer.set_kernel_timing(1)
    xfer.save(layers, stream, TransferPath.STAGED)
    stream.synchronize()
    assert xfer.last_kernel_ms()[1] == fills
    images = []
    for c, L, h in zip(cases, Ls, hosts):
        n, stride = len(c.ids), L.host_stride
        oc = c.cache0.copy()
        ok = np.full(n * stride, SENT, dtype=np.uint8)
        ov = np.full(n * stride, SENT, dtype=np.uint8) if L.is_split else None
        O.transfer_layer(c.oracle_layout(oc), c.ids, ok, ov, host_is_src=False)
        hv = h.as_numpy()
        assert np.array_equal(hv[: n * stride], ok), c.args
        if ov is not None:
            assert np.array_equal(hv[n * stride:], ov), c.args
        images.append((ok, ov))
    for li, c in enumerate(cases):
        c.dev.fill(SENT)
        layers[li].block_ids = rng.choice(c.num_blocks, len(c.ids), replace=False).astype(np.uint32)
    xfer.load(layers, stream, TransferPath.STAGED)
    stream.synchronize()
    assert xfer.last_kernel_ms()[1] == fills
    for li, c in enumerate(cases):
        oc = np.full_like(c.cache0, SENT)
        ok, ov = images[li]
        O.transfer_layer(c.oracle_layout(oc), layers[li].block_ids, ok, ov, host_is_src=True)
        assert np.array_equal(c.dev.copy_to_host(), oc), li
    xfer.close()
    for c, h in zip(cases, hosts):
        c.close()
        h.close()


def test_fill_of_many_layers_of_unlike_length(stream):
    """Twelve layers in one fill, two of 600 blocks among ten of 8 (a task over
    cache groups of unlike size): more units than one rows launch takes and
    too unlike for the grid of the units-inner form, so the fill goes out as
    two rows launches (one timed group); bytes against the oracle both ways.
    A second call of twelve equal layers takes the units-inner form; a third
    mixes 72 KiB and 8 KiB fragments in one fill."""
    rng = np.random.default_rng(612)
    # (blocks, fragment bytes) per layer; the third call mixes 72 KiB and 8 KiB
    # fragments of one length (latent and indexer caches of one model), which
    # leaves most workgroups of the small fragments' rows without a tile
    calls = ([(n, 32768) for n in (8, 8, 600, 8, 8, 8, 8, 8, 600, 8, 8, 8)],
             [(40, 32768)] * 12,
             [(512, 73728), (512, 8192)] * 3)
    for call in calls:
        cases = [Case(rng, num_blocks=n + 24, seg=seg, segments=2 if li % 3 else 1, n_ids=n)
                 for li, (n, seg) in enumerate(call)]
        hosts, layers, Ls = [], [], []
        for c in cases:
            L = c.product_layout()
            Ls.append(L)
            nseg = 2 if L.is_split else 1
            h = PinnedMemory(nseg * len(c.ids) * L.host_stride)
            h.as_numpy()[:] = SENT
            hosts.append(h)
            c.dev.copy_from_host(c.cache0)
            layers.append(_dense_layer(c, L, h, c.ids))
        xfer = BlockTransfer(staging_slot_bytes=256 << 20, staging_slots=2, auto_staged_min_bytes=1)
        xfer.set_kernel_timing(1)
        xfer.save(layers, stream, TransferPath.STAGED)
        stream.synchronize()
        assert xfer.last_path == ST and xfer.last_kernel_ms()[1] == 1
        images = []
        for c, L, h in zip(cases, Ls, hosts):
            n, stride = len(c.ids), L.host_stride
            oc = c.cache0.copy()
            ok = np.full(n * stride, SENT, dtype=np.uint8)
            ov = np.full(n * stride, SENT, dtype=np.uint8) if L.is_split else None
            O.transfer_layer(c.oracle_layout(oc), c.ids, ok, ov, host_is_src=False)
            hv = h.as_numpy()
            assert np.array_equal(hv[: n * stride], ok), c.args
            if ov is not None:
                assert np.array_equal(hv[n * stride:], ov), c.args
            images.append((ok, ov))
        for li, c in enumerate(cases):
            c.dev.fill(SENT)
            layers[li].block_ids = rng.choice(c.num_blocks, len(c.ids), replace=False).astype(np.uint32)
        xfer.load(layers, stream, TransferPath.STAGED)
        stream.synchronize()
        assert xfer.last_kernel_ms()[1] == 1
        for li, c in enumerate(cases):
            oc = np.full_like(c.cache0, SENT)
            ok, ov = images[li]
            O.transfer_layer(c.oracle_layout(oc), layers[li].block_ids, ok, ov, host_is_src=True)
            assert np.array_equal(c.dev.copy_to_host(), oc), li
        xfer.close()
        for c, h in zip(cases, hosts):
            c.close()
            h.close()


def test_long_layer_of_small_blocks_behind_another_layer_in_one_fill(stream):
    """A layer of 68 000 blocks of 1 KiB (more rows than one grid extent)
    that fits the room a small layer left in the slot: it becomes two units
    of the same fill, and the bytes are the oracle's both ways."""
    rng = np.random.default_rng(515)
    cases = [Case(rng, num_blocks=128, seg=4096, segments=2, n_ids=100),
             Case(rng, num_blocks=70000, seg=1024, segments=1, n_ids=68000)]
    hosts, layers, Ls = [], [], []
    for c in cases:
        L = c.product_layout()
        Ls.append(L)
        nseg = 2 if L.is_split else 1
        h = PinnedMemory(nseg * len(c.ids) * L.host_stride)
        h.as_numpy()[:] = SENT
        hosts.append(h)
        c.dev.copy_from_host(c.cache0)
        layers.append(_dense_layer(c, L, h, c.ids))
    xfer = BlockTransfer(staging_slot_bytes=128 << 20, staging_slots=2, auto_staged_min_bytes=1)
    xfer.set_kernel_timing(1)
    xfer.save(layers, stream, TransferPath.STAGED)
    stream.synchronize()
    assert xfer.last_path == ST
    assert xfer.last_kernel_ms()[1] == 1
    images = []
    for c, L, h in zip(cases, Ls, hosts):
        n, stride = len(c.ids), L.host_stride
        oc = c.cache0.copy()
        ok = np.full(n * stride, SENT, dtype=np.uint8)
        ov = np.full(n * stride, SENT, dtype=np.uint8) if L.is_split else None
        O.transfer_layer(c.oracle_layout(oc), c.ids, ok, ov, host_is_src=False)
        hv = h.as_numpy()
        assert np.array_equal(hv[: n * stride], ok), c.args
        if ov is not None:
            assert np.array_equal(hv[n * stride:], ov), c.args
        images.append((ok, ov))
    for li, c in enumerate(cases):
        c.dev.fill(SENT)
        layers[li].block_ids = rng.choice(c.num_blocks, len(c.ids), replace=False).astype(np.uint32)
    xfer.load(layers, stream, TransferPath.STAGED)
    stream.synchronize()
    assert xfer.last_kernel_ms()[1] == 1
    for li, c in enumerate(cases):
        oc = np.full_like(c.cache0, SENT)
        ok, ov = images[li]
        O.transfer_layer(c.oracle_layout(oc), layers[li].block_ids, ok, ov, host_is_src=True)
        assert np.array_equal(c.dev.copy_to_host(), oc), li
    xfer.close()
    for c, h in zip(cases, hosts):
        c.close()
        h.close()


def test_auto_takes_zero_copy_when_no_staging_slot_can_be_allocated(stream):
    """A staging slot the device cannot hold (1 TiB): PF_PATH_AUTO moves the
    same bytes over the zero-copy path instead of failing; an explicit
    PF_PATH_STAGED reports the allocation error and touches nothing."""
    rng = np.random.default_rng(808)
    c = Case(rng, num_blocks=256, seg=32768, segments=2, n_ids=200)
    L = c.product_layout()
    n, stride = len(c.ids), L.host_stride
    h = PinnedMemory(2 * n * stride)
    h.as_numpy()[:] = SENT
    c.dev.copy_from_host(c.cache0)
    layer = _dense_layer(c, L, h, c.ids)
    xfer = BlockTransfer(staging_slot_bytes=1 << 40, auto_staged_min_bytes=1)
    with pytest.raises(_lib.PegaHipError, match="staging slot"):
        xfer.save([layer], stream, TransferPath.STAGED)
    stream.synchronize()
    assert (h.as_numpy() == SENT).all()
    for _ in range(2):                       # the second call finds the slots still missing
        h.as_numpy()[:] = SENT
        xfer.save([layer], stream, TransferPath.AUTO)
        stream.synchronize()
        assert xfer.last_path == ZC
        oc = c.cache0.copy()
        ok = np.full(n * stride, SENT, dtype=np.uint8)
        ov = np.full(n * stride, SENT, dtype=np.uint8)
        O.transfer_layer(c.oracle_layout(oc), c.ids, ok, ov, host_is_src=False)
        assert np.array_equal(h.as_numpy()[: n * stride], ok)
        assert np.array_equal(h.as_numpy()[n * stride:], ov)
    c.dev.fill(SENT)
    xfer.load([layer], stream, TransferPath.AUTO)
    stream.synchronize()
    assert xfer.last_path == ZC
    oc = np.full_like(c.cache0, SENT)
    O.transfer_layer(c.oracle_layout(oc), c.ids, ok, ov, host_is_src=True)
    assert np.array_equal(c.dev.copy_to_host(), oc)
    xfer.close()
    c.close()
    h.close()


def test_call_size_rule_stages_small_layers_of_a_long_call(stream):
    """auto_staged_min_call_bytes: PF_PATH_AUTO stages the dense layers of a
    call whose dense bytes reach the threshold even though no layer reaches
    the per-layer threshold; a shorter call stays zero-copy; the bytes are
    the oracle's either way."""
    rng = np.random.default_rng(91)
    xfer = BlockTransfer(auto_staged_min_call_bytes=2 << 20)   # per-layer default: 16 MiB
    for n_ids, want in ((40, ST), (8, ZC)):                       # 4 x 640 KiB = 2.5 MiB | 4 x 128 KiB
        cases = [Case(rng, num_blocks=64, seg=8192, segments=2, n_ids=n_ids) for _ in range(4)]
        hosts, layers = [], []
        for li, c in enumerate(cases):
            L = c.product_layout()
            h = PinnedMemory(2 * n_ids * L.host_stride)
            h.as_numpy()[:] = SENT
            hosts.append(h)
            c.dev.copy_from_host(c.cache0)
            layers.append(_dense_layer(c, L, h, c.ids))
        xfer.save(layers, stream, TransferPath.AUTO)
        stream.synchronize()
        assert xfer.last_path == want
        for c, h in zip(cases, hosts):
            L = c.product_layout()
            n, stride = n_ids, L.host_stride
            oc = c.cache0.copy()
            ok = np.full(n * stride, SENT, dtype=np.uint8)
            ov = np.full(n * stride, SENT, dtype=np.uint8)
            O.transfer_layer(c.oracle_layout(oc), c.ids, ok, ov, host_is_src=False)
            assert np.array_equal(h.as_numpy()[: n * stride], ok)
            assert np.array_equal(h.as_numpy()[n * stride:], ov)
            c.dev.fill(SENT)
        xfer.load(layers, stream, TransferPath.AUTO)
        stream.synchronize()
        assert xfer.last_path == want
        for c, h in zip(cases, hosts):
            L = c.product_layout()
            n, stride = n_ids, L.host_stride
            oc = np.full_like(c.cache0, SENT)
            hv = h.as_numpy()
            O.transfer_layer(c.oracle_layout(oc), c.ids, hv[: n * stride].copy(),
                             hv[n * stride:].copy(), host_is_src=True)
            assert np.array_equal(c.dev.copy_to_host(), oc)
            c.close()
            h.close()
    xfer.close()
