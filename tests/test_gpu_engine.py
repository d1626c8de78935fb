"""Worker pool and save/query/load cycle on a real device, mirroring the
reference's engine integration tests (pegaflow-core/tests/engine_basic.rs,
hybrid_groups.rs, save_validation.rs) with the same closed-form patterns:
block i filled with byte (i % 251) + 1, `overwrite(m)` = wrapping add."""

import numpy as np
import pytest

from oracle import oracle as O
from pegaflow_amd import _lib
from pegaflow_amd.engine import (LOAD_STATE_ERROR, LOAD_STATE_SUCCESS, GpuWorkerPool, LayerSave,
                                 LoadState, PegaEngine)
from pegaflow_amd.layout import KVCacheLayout
from pegaflow_amd.runtime import DeviceBuffer, PinnedMemory
from pegaflow_amd.transfer import HostBlock, LayerTransferData, TransferMode
from tests.helpers import block_fill_pattern, random_bytes, split_fill_pattern

pytestmark = pytest.mark.gpu


def make_block_hashes(n, salt):
    """salt || u32le(idx)  (tests/common/helpers.rs:91-100)."""
    return [bytes([salt]) + int(i).to_bytes(4, "little") for i in range(n)]


class Layer:
    def __init__(self, name, num_blocks, block_bytes, overwrite=0, split_kv_stride=None):
        self.name, self.num_blocks, self.block_bytes = name, num_blocks, block_bytes
        if split_kv_stride:
            self.expected = split_fill_pattern(num_blocks, block_bytes, split_kv_stride)
            self.reg = (block_bytes, split_kv_stride, 2)
        else:
            self.expected = block_fill_pattern(num_blocks, block_bytes)
            self.reg = (block_bytes, 0, 1)
        self.expected = (self.expected.astype(np.uint16) + overwrite).astype(np.uint8)
        self.gpu = DeviceBuffer(self.expected.nbytes)
        self.gpu.copy_from_host(self.expected)

    def zero_gpu(self):
        self.gpu.fill(0)

    def assert_gpu_matches(self, expected):
        assert np.array_equal(self.gpu.copy_to_host(), expected), f"GPU data mismatch in {self.name}"


def register(engine, instance, layers, page_first=False, mode=TransferMode.DIRECT, ns="test-ns",
             groups=None):
    engine.register_context_layer_batch(
        instance, ns, 0, 0, 0, 1, 1, [l.name for l in layers], [l.gpu.ptr for l in layers],
        [l.expected.nbytes for l in layers], [l.num_blocks for l in layers],
        [l.reg[0] for l in layers], [l.reg[1] for l in layers], [l.reg[2] for l in layers],
        transfer_mode=mode, page_first=page_first, layer_group_ids=groups)


@pytest.fixture(params=[False, True], ids=["block_ids", "descriptors"])
def engine(request, gpu):
    e = PegaEngine(pool_size=64 << 20, use_descriptor_backends=request.param)
    yield e
    e.close()


def test_save_query_load_roundtrip(engine):
    """engine_basic.rs:12-25."""
    layer = Layer("layer_0", 4, 1024)
    register(engine, "test-roundtrip", [layer])
    hashes = make_block_hashes(4, 0)
    engine.batch_save_kv_blocks("test-roundtrip", 0, 0, 0, [LayerSave("layer_0", [0, 1, 2, 3], hashes)])
    layer.zero_gpu()
    hits, lease = engine.query_prefix("test-roundtrip", hashes)
    assert hits == 4 and lease != 0
    engine.batch_load_kv_blocks_multi_layer("test-roundtrip", 0, 0, [["layer_0"]], lease,
                                            [[0, 1, 2, 3]]).wait()
    layer.assert_gpu_matches(layer.expected)
    # saving the same hashes again stores nothing new (dedupe against the cache)
    used = engine.pool_usage()[0]
    engine.batch_save_kv_blocks("test-roundtrip", 0, 0, 0, [LayerSave("layer_0", [0, 1, 2, 3], hashes)])
    assert engine.pool_usage()[0] == used and engine.cached_blocks == 4


@pytest.mark.parametrize("mode", [TransferMode.DIRECT, TransferMode.KERNEL, TransferMode.ZEROCOPY],
                         ids=["direct", "kernel", "zerocopy"])
def test_split_layout_roundtrip_both_backends(engine, mode):
    """K/V split registration (tests/common/harness.rs:53-80), both transfer modes."""
    layer = Layer("kv", 16, 4096, split_kv_stride=16 * 4096)
    register(engine, f"split-{mode}", [layer], mode=mode)
    hashes = make_block_hashes(8, 3)
    ids = [1, 3, 5, 7, 9, 11, 13, 15]
    engine.batch_save_kv_blocks(f"split-{mode}", 0, 0, 0, [LayerSave("kv", ids, hashes)])
    layer.zero_gpu()
    hits, lease = engine.query_prefix(f"split-{mode}", hashes)
    assert hits == 8
    dest = [0, 2, 4, 6, 8, 10, 12, 14]
    engine.batch_load_kv_blocks_multi_layer(f"split-{mode}", 0, 0, [["kv"]], lease, [dest]).wait()
    want = np.zeros_like(layer.expected)
    for src, dst in zip(ids, dest):
        for region in (0, 16 * 4096):
            want[region + dst * 4096: region + (dst + 1) * 4096] = \
                layer.expected[region + src * 4096: region + (src + 1) * 4096]
    layer.assert_gpu_matches(want)


def test_page_first_multi_layer_roundtrip(engine, kats):
    """engine_basic.rs:32-58: three layers of distinct sizes and contents in one page."""
    case = next(c for c in kats["engine"] if c["name"] == "page_first_multi_layer_roundtrip")
    layers = [Layer(l["name"], l["num_blocks"], l["block_bytes"], l["overwrite"]) for l in case["layers"]]
    register(engine, "test-page-first", layers, page_first=True, mode=TransferMode.KERNEL)
    hashes = make_block_hashes(4, 0xAB)
    engine.batch_save_kv_blocks("test-page-first", 0, 0, 0,
                                [LayerSave(l.name, [0, 1, 2, 3], hashes) for l in layers])
    used, _total = engine.pool_usage()
    assert used == 4 * case["expect"]["page_size"]  # one 3072-byte page per block
    for l in layers:
        l.zero_gpu()
    hits, lease = engine.query_prefix("test-page-first", hashes)
    assert hits == 4
    engine.batch_load_kv_blocks_multi_layer("test-page-first", 0, 0, [[l.name for l in layers]],
                                            lease, [[0, 1, 2, 3]]).wait()
    for l in layers:
        l.assert_gpu_matches(l.expected)


def test_partial_layer_page_first_save_is_rejected(engine):
    """engine_basic.rs:126-160: a page-first save must carry every layer of the shard."""
    layers = [Layer("layer_a", 4, 512), Layer("layer_b", 4, 1024)]
    register(engine, "test-partial", layers, page_first=True)
    hashes = make_block_hashes(2, 1)
    with pytest.raises(_lib.InvalidArgument, match="must cover all 2 layers of shard 0"):
        engine.batch_save_kv_blocks("test-partial", 0, 0, 0, [LayerSave("layer_a", [0, 1], hashes)])
    assert engine.pool_usage()[0] == 0


def test_hybrid_groups_load_to_distinct_block_ids(engine, kats):
    """engine_basic.rs:62-124: same hashes saved from different block ids per
    layer, loaded into per-group destinations with skips; expected bytes are
    given explicitly by the reference."""
    case = next(c for c in kats["engine"] if c["name"] == "hybrid_groups_load_to_distinct_block_ids")
    layers = [Layer(l["name"], l["num_blocks"], l["block_bytes"], l["overwrite"]) for l in case["layers"]]
    register(engine, "test-hybrid-groups", layers)
    hashes = make_block_hashes(2, 0xAC)
    engine.batch_save_kv_blocks("test-hybrid-groups", 0, 0, 0, [
        LayerSave(l["name"], l["save_ids"], hashes) for l in case["layers"]])
    for l in layers:
        l.zero_gpu()
    hits, lease = engine.query_prefix("test-hybrid-groups", hashes)
    assert hits == 2
    engine.batch_load_kv_blocks_multi_layer(
        "test-hybrid-groups", 0, 0, [["full_attention"], [], ["gdn"]], lease,
        [[2, 3], [None, None], [None, 0]]).wait()
    for l in layers:
        want = np.zeros(4 * 1024, dtype=np.uint8)
        for blk, fill in case["expect"][l.name].items():
            want[int(blk) * 1024:(int(blk) + 1) * 1024] = fill
        l.assert_gpu_matches(want)


def test_save_validation_and_load_errors(engine):
    """save_validation.rs:12-42 and the load-side checks of lib.rs:715-883."""
    layer = Layer("layer_0", 4, 1024)
    register(engine, "test-validate", [layer])
    with pytest.raises(_lib.InvalidArgument, match="block_ids length 2 does not match block_hashes 1"):
        engine.batch_save_kv_blocks("test-validate", 0, 0, 0,
                                    [LayerSave("layer_0", [0, 1], make_block_hashes(1, 9))])
    with pytest.raises(_lib.InvalidArgument, match=r"block_id 4 out of range \(num_blocks=4\) for layer layer_0"):
        engine.batch_save_kv_blocks("test-validate", 0, 0, 0,
                                    [LayerSave("layer_0", [4], make_block_hashes(1, 9))])
    with pytest.raises(_lib.InvalidArgument, match="layer nope is not registered"):
        engine.batch_save_kv_blocks("test-validate", 0, 0, 0,
                                    [LayerSave("nope", [0], make_block_hashes(1, 9))])
    with pytest.raises(_lib.InstanceMissing):
        engine.batch_save_kv_blocks("ghost", 0, 0, 0, [])
    with pytest.raises(_lib.InvalidArgument, match="registered for tp_rank 0, pp_rank 0"):
        engine.batch_save_kv_blocks("test-validate", 0, 1, 0,
                                    [LayerSave("layer_0", [0], make_block_hashes(1, 9))])
    assert engine.pool_usage()[0] == 0
    hashes = make_block_hashes(2, 5)
    engine.batch_save_kv_blocks("test-validate", 0, 0, 0, [LayerSave("layer_0", [0, 1], hashes)])
    # prefix semantics: a miss in the middle ends the prefix
    hits, lease = engine.query_prefix("test-validate", [hashes[0], b"missing", hashes[1]])
    assert hits == 1
    ls = LoadState()
    with pytest.raises(_lib.InvalidArgument, match="does not match destination block count"):
        engine.batch_load_kv_blocks_multi_layer("test-validate", 0, 0, [["layer_0"]], lease,
                                                [[0, 1]], load_state=ls)
    assert ls.get() == LOAD_STATE_ERROR  # pre-submit failure marks the LoadState
    ls.close()
    with pytest.raises(_lib.StorageError, match="query lease"):
        engine.batch_load_kv_blocks_multi_layer("test-validate", 0, 0, [["layer_0"]], lease, [[0]])
    # zero resolved blocks: completes at once with success
    hits, lease = engine.query_prefix("test-validate", hashes)
    ls = LoadState()
    engine.batch_load_kv_blocks_multi_layer("test-validate", 0, 0, [["layer_0"]], lease,
                                            [[None, None]], load_state=ls).wait()
    assert ls.get() == LOAD_STATE_SUCCESS
    ls.close()
    # registration errors
    with pytest.raises(_lib.InvalidArgument, match="already exists"):
        register(engine, "test-validate", [layer])
    with pytest.raises(_lib.InvalidArgument, match="exists with tp=1, world=1, page_first=false"):
        engine.register_context_layer_batch("test-validate", "test-ns", 0, 0, 0, 2, 2, ["x"],
                                            [layer.gpu.ptr], [4096], [4], [1024], [0], [1])
    with pytest.raises(_lib.InvalidArgument, match="layer bad: .*too small"):
        engine.register_context_layer_batch("fresh", "test-ns", 0, 0, 0, 1, 1, ["bad"],
                                            [layer.gpu.ptr], [1024], [4], [1024], [0], [1])
    engine.unregister_instance("test-validate")
    with pytest.raises(_lib.InstanceMissing):
        engine.unregister_instance("test-validate")


def test_pool_pressure_evicts_oldest_unleased_blocks(gpu):
    """storage/mod.rs:294-330: allocate, evict, retry; exhausted when nothing
    can be evicted."""
    e = PegaEngine(pool_size=64 * 1024)
    layer = Layer("layer_0", 64, 4096)
    register(e, "pressure", [layer])
    first = make_block_hashes(8, 1)
    e.batch_save_kv_blocks("pressure", 0, 0, 0, [LayerSave("layer_0", list(range(8)), first)])
    second = make_block_hashes(8, 2)
    e.batch_save_kv_blocks("pressure", 0, 0, 0, [LayerSave("layer_0", list(range(8, 16)), second)])
    assert e.cached_blocks == 16 and e.pool_usage()[0] == 64 * 1024
    # a third batch only fits after evicting an older batch's allocation
    third = make_block_hashes(8, 3)
    e.batch_save_kv_blocks("pressure", 0, 0, 0, [LayerSave("layer_0", list(range(16, 24)), third)])
    assert e.query_prefix("pressure", first)[0] == 0
    assert e.query_prefix("pressure", third)[0] == 8
    # leased blocks are not evictable: with everything leased the pool is exhausted
    _h, l2 = e.query_prefix("pressure", second)
    _h, l3 = e.query_prefix("pressure", third)
    with pytest.raises(_lib.StorageError, match="pinned pool exhausted"):
        e.batch_save_kv_blocks("pressure", 0, 0, 0,
                               [LayerSave("layer_0", list(range(24, 32)), make_block_hashes(8, 4))])
    e.release_query_lease(l2)
    e.release_query_lease(l3)
    e.close()


def test_eviction_is_least_recently_used(gpu):
    """A prefix query makes its hits the most recently used blocks
    (storage/read_cache.rs): the batch that was not touched goes first."""
    e = PegaEngine(pool_size=64 * 1024)
    layer = Layer("layer_0", 64, 4096)
    register(e, "lru", [layer])
    first, second, third = (make_block_hashes(8, s) for s in (1, 2, 3))
    e.batch_save_kv_blocks("lru", 0, 0, 0, [LayerSave("layer_0", list(range(8)), first)])
    e.batch_save_kv_blocks("lru", 0, 0, 0, [LayerSave("layer_0", list(range(8, 16)), second)])
    hits, lease = e.query_prefix("lru", first)      # touch the older batch ...
    assert hits == 8
    e.release_query_lease(lease)                    # ... without keeping it pinned
    e.batch_save_kv_blocks("lru", 0, 0, 0, [LayerSave("layer_0", list(range(16, 24)), third)])
    assert e.query_prefix("lru", second)[0] == 0    # the untouched batch was evicted
    h1, l1 = e.query_prefix("lru", first)
    h3, l3 = e.query_prefix("lru", third)
    assert (h1, h3) == (8, 8)
    e.release_query_lease(l1)
    e.release_query_lease(l3)
    e.close()


def test_blockwise_alloc_and_odd_segment_size(gpu):
    """--blockwise-alloc gives every block its own K and V allocation (the
    worker then falls back to per-fragment descriptors); 1000-byte segments in
    512-byte pool units leave unit padding that must never be written."""
    for kw in (dict(blockwise_alloc=True), dict(unit_size_hint=512)):
        e = PegaEngine(pool_size=8 << 20, **kw)
        layer = Layer("kv", 16, 1000, split_kv_stride=16 * 1000)  # 1000-byte segments
        register(e, "bw", [layer], mode=TransferMode.KERNEL)
        hashes = make_block_hashes(5, 7)
        ids = [2, 4, 6, 8, 10]
        e.batch_save_kv_blocks("bw", 0, 0, 0, [LayerSave("kv", ids, hashes)])
        layer.zero_gpu()
        _h, lease = e.query_prefix("bw", hashes)
        e.batch_load_kv_blocks_multi_layer("bw", 0, 0, [["kv"]], lease, [ids]).wait()
        want = np.zeros_like(layer.expected)
        for b in ids:
            for region in (0, 16 * 1000):
                want[region + b * 1000: region + (b + 1) * 1000] = \
                    layer.expected[region + b * 1000: region + (b + 1) * 1000]
        layer.assert_gpu_matches(want)
        e.close()


@pytest.mark.parametrize("use_desc", [False, True], ids=["block_ids", "descriptors"])
@pytest.mark.parametrize("mode", [TransferMode.DIRECT, TransferMode.KERNEL, TransferMode.ZEROCOPY],
                         ids=["direct", "kernel", "zerocopy"])
def test_worker_pool_matches_oracle(gpu, mode, use_desc):
    """Raw worker ABI: a save task then a load task with a LoadState, checked
    against the oracle's descriptor executor on the same inputs."""
    rng = np.random.default_rng(40)
    nb, seg, n = 64, 8192, 24
    cache0 = random_bytes(rng, 2 * nb * seg)
    dev = DeviceBuffer(cache0.nbytes)
    dev.copy_from_host(cache0)
    host = PinnedMemory(2 * n * seg)
    host.as_numpy()[:] = 0xC3
    layout = KVCacheLayout(dev.ptr, cache0.nbytes, nb, seg, nb * seg, 2)
    ids = rng.choice(nb, n, replace=False)
    blocks = [HostBlock((host.host_ptr + i * seg, host.host_ptr + (n + i) * seg),
                        (host.device_ptr + i * seg, host.device_ptr + (n + i) * seg), (1, 2),
                        (seg, seg)) for i in range(n)]
    pool = GpuWorkerPool(0, -1, mode, use_descriptor_backends=use_desc)
    res = pool.batch_save([LayerTransferData("kv", layout, ids, blocks)]).wait()
    assert res.done and res.bytes == 2 * n * seg
    ocache = cache0.copy()
    ok = np.full(n * seg, 0xC3, dtype=np.uint8)
    ov = np.full(n * seg, 0xC3, dtype=np.uint8)
    O.transfer_layer(O.layout_over(ocache, nb, seg, nb * seg, 2), ids.astype(np.uint32), ok, ov,
                     host_is_src=False)
    img = host.as_numpy()
    assert np.array_equal(img[: n * seg], ok) and np.array_equal(img[n * seg:], ov)
    dest = rng.choice(nb, n, replace=False)
    dev.fill(0x11)
    ls = LoadState()
    pool.submit_load([LayerTransferData("kv", layout, dest, blocks)], ls).wait()
    assert ls.get() == LOAD_STATE_SUCCESS
    ocache2 = np.full_like(cache0, 0x11)
    O.transfer_layer(O.layout_over(ocache2, nb, seg, nb * seg, 2), dest.astype(np.uint32), ok, ov,
                     host_is_src=True)
    assert np.array_equal(dev.copy_to_host(), ocache2)
    # failure: a bad block id fails the task and flips the LoadState to error
    bad_ls = LoadState()
    bad = pool.submit_load([LayerTransferData("model.layers.3", layout, [nb], blocks[:1])], bad_ls)
    with pytest.raises(_lib.StorageError, match=r"layer model.layers.3: block 64 out of range \(64 blocks\)"):
        bad.wait()
    assert bad_ls.get() == LOAD_STATE_ERROR
    assert np.array_equal(dev.copy_to_host(), ocache2)
    for x in (ls, bad_ls):
        x.close()
    pool.close()
    host.close()
    dev.close()


@pytest.mark.parametrize("use_desc", [False, True], ids=["block_ids", "descriptors"])
def test_worker_pool_split_cache_with_single_segment_host_blocks(gpu, use_desc):
    """gpu_worker.rs:373-379: a split K/V cache moved to or from host blocks of
    one segment puts V right behind K (`k_ptr + k.bytes`)."""
    rng = np.random.default_rng(41)
    nb, seg, n = 48, 4112, 17
    cache0 = random_bytes(rng, 2 * nb * seg)
    dev = DeviceBuffer(cache0.nbytes)
    dev.copy_from_host(cache0)
    host = PinnedMemory(2 * n * seg)
    host.as_numpy()[:] = 0x5A
    layout = KVCacheLayout(dev.ptr, cache0.nbytes, nb, seg, nb * seg, 2)
    ids = rng.choice(nb, n, replace=False)
    blocks = [HostBlock((host.host_ptr + i * 2 * seg,), (host.device_ptr + i * 2 * seg,), (7,),
                        (2 * seg,)) for i in range(n)]
    pool = GpuWorkerPool(0, -1, TransferMode.DIRECT, use_descriptor_backends=use_desc)
    res = pool.batch_save([LayerTransferData("kv", layout, ids, blocks)]).wait()
    assert res.done and res.bytes == 2 * n * seg
    img = host.as_numpy().reshape(n, 2, seg)
    kv = cache0.reshape(2, nb, seg)
    assert np.array_equal(img[:, 0], kv[0, ids]) and np.array_equal(img[:, 1], kv[1, ids])
    dest = rng.choice(nb, n, replace=False)
    dev.fill(0x22)
    pool.submit_load([LayerTransferData("kv", layout, dest, blocks)], None).wait()
    want = np.full_like(kv, 0x22)
    want[0, dest] = kv[0, ids]
    want[1, dest] = kv[1, ids]
    assert np.array_equal(dev.copy_to_host().reshape(2, nb, seg), want)
    pool.close()
    host.close()
    dev.close()


def test_worker_pool_init_failure_is_synchronous(gpu):
    with pytest.raises(_lib.PegaHipError, match="Failed to initialise GPU worker on device 99"):
        GpuWorkerPool(99)


def test_layers_saved_in_separate_calls_complete_the_same_blocks(engine):
    """Slots of a block may arrive in several saves (block.rs:346-454): the block
    is queryable only once every layer's slot is in, and layers that carry
    different hash lists in one call are kept apart."""
    a = Layer("layer_a", 8, 2048)
    b = Layer("layer_b", 8, 1024, overwrite=7, split_kv_stride=8 * 1024)
    register(engine, "two-calls", [a, b])
    hashes = make_block_hashes(4, 9)
    ids_a, ids_b = [0, 2, 4, 6], [7, 5, 3, 1]
    engine.batch_save_kv_blocks("two-calls", 0, 0, 0, [LayerSave("layer_a", ids_a, hashes)])
    assert engine.query_prefix("two-calls", hashes) == (0, 0)
    assert engine.cached_blocks == 0
    other = make_block_hashes(2, 10)
    engine.batch_save_kv_blocks("two-calls", 0, 0, 0, [
        LayerSave("layer_b", ids_b, hashes),           # completes the four blocks
        LayerSave("layer_a", [1, 3], other),           # a different list in the same call
    ])
    hits, lease = engine.query_prefix("two-calls", hashes)
    assert hits == 4 and engine.cached_blocks == 4
    assert engine.query_prefix("two-calls", other) == (0, 0)    # layer_b's slots still missing
    a.zero_gpu()
    b.zero_gpu()
    dest = [1, 3, 5, 7]
    engine.batch_load_kv_blocks_multi_layer("two-calls", 0, 0, [["layer_a", "layer_b"]], lease,
                                            [dest]).wait()
    want_a = np.zeros_like(a.expected)
    want_b = np.zeros_like(b.expected)
    for pos, dst in enumerate(dest):
        want_a[dst * 2048:(dst + 1) * 2048] = a.expected[ids_a[pos] * 2048:(ids_a[pos] + 1) * 2048]
        for region in (0, 8 * 1024):
            src = ids_b[pos]
            want_b[region + dst * 1024: region + (dst + 1) * 1024] = \
                b.expected[region + src * 1024: region + (src + 1) * 1024]
    a.assert_gpu_matches(want_a)
    b.assert_gpu_matches(want_b)


def test_repeated_hash_in_one_list_keeps_the_first_image(engine):
    """Duplicate hashes are not rejected (offload.rs:348-368): every occurrence is
    copied, the first one enters the store."""
    layer = Layer("layer_0", 8, 1024)
    register(engine, "dup-hash", [layer])
    h = make_block_hashes(2, 4)
    engine.batch_save_kv_blocks("dup-hash", 0, 0, 0,
                                [LayerSave("layer_0", [5, 6, 2], [h[0], h[1], h[0]])])
    assert engine.cached_blocks == 2
    layer.zero_gpu()
    hits, lease = engine.query_prefix("dup-hash", h)
    assert hits == 2
    engine.batch_load_kv_blocks_multi_layer("dup-hash", 0, 0, [["layer_0"]], lease, [[0, 1]]).wait()
    want = np.zeros_like(layer.expected)
    want[0:1024] = layer.expected[5 * 1024:6 * 1024]
    want[1024:2048] = layer.expected[6 * 1024:7 * 1024]
    layer.assert_gpu_matches(want)
    prof = engine.last_save_profile()
    assert prof["bytes"] == 3 * 1024 and prof["total_ms"] >= prof["transfer_ms"] > 0


def test_packed_saves_are_reusable_and_share_hash_lists(engine):
    from pegaflow_amd.engine import PackedSaves
    layers = [Layer(f"l{i}", 6, 512, overwrite=i) for i in range(3)]
    register(engine, "packed", layers)
    hashes = make_block_hashes(3, 6)
    packed = PackedSaves([LayerSave(l.name, np.array([4, 0, 2], dtype=np.uint64), hashes)
                          for l in layers])
    engine.batch_save_kv_blocks("packed", 0, 0, 0, packed)
    assert engine.cached_blocks == 3
    engine.evict_all()
    assert engine.cached_blocks == 0
    engine.batch_save_kv_blocks("packed", 0, 0, 0, packed)
    hits, lease = engine.query_prefix("packed", hashes)
    assert hits == 3
    for l in layers:
        l.zero_gpu()
    engine.batch_load_kv_blocks_multi_layer("packed", 0, 0, [[l.name for l in layers]], lease,
                                            [[1, 3, 5]]).wait()
    for l in layers:
        want = np.zeros_like(l.expected)
        for src, dst in zip([4, 0, 2], [1, 3, 5]):
            want[dst * 512:(dst + 1) * 512] = l.expected[src * 512:(src + 1) * 512]
        l.assert_gpu_matches(want)


def test_unsealed_instance_rejects_topology_access(gpu):
    """instance/tests.rs:269-286: with one of two workers registered nothing can
    be saved, and the same device cannot register twice."""
    e = PegaEngine(pool_size=1 << 20)
    layer = Layer("layer_0", 4, 1024)
    e.register_context_layer_batch("partial", "partial-ns", 0, 0, 0, 2, 2, ["layer_0"],
                                   [layer.gpu.ptr], [layer.expected.nbytes], [4], [1024], [0], [1])
    with pytest.raises(_lib.PegaHipError, match="registration incomplete: 1/2"):
        e.batch_save_kv_blocks("partial", 0, 0, 0, [LayerSave("layer_0", [0], make_block_hashes(1, 1))])
    with pytest.raises(_lib.PegaHipError, match="already exists"):
        e.register_context_layer_batch("partial", "partial-ns", 0, 0, 0, 2, 2, ["layer_0"],
                                       [layer.gpu.ptr], [layer.expected.nbytes], [4], [1024], [0], [1])
    e.close()


# ---------------------------------------------------------------------------
# pegaflow-core/tests/prefix_semantics.rs and eviction.rs, one test each
# ---------------------------------------------------------------------------

def _one_layer_engine(instance, num_blocks, block_bytes, **engine_kw):
    e = PegaEngine(**engine_kw)
    layer = Layer("layer_0", num_blocks, block_bytes)
    register(e, instance, [layer])
    return e, layer


def _save(e, instance, hashes, ids=None):
    ids = list(range(len(hashes))) if ids is None else ids
    e.batch_save_kv_blocks(instance, 0, 0, 0, [LayerSave("layer_0", ids, hashes)])


def _hits_then_release(e, instance, hashes):
    hits, lease = e.query_prefix(instance, hashes)
    if lease:
        e.release_query_lease(lease)
    return hits


def test_partial_prefix_reports_contiguous_hit_count(gpu):
    """prefix_semantics.rs:13-30: 3 of 5 saved -> 3 hits, 2 missing."""
    e, _ = _one_layer_engine("test-partial-prefix", 3, 1024, pool_size=1 << 20)
    _save(e, "test-partial-prefix", make_block_hashes(3, 10))
    assert _hits_then_release(e, "test-partial-prefix", make_block_hashes(5, 10)) == 3
    e.close()


def test_gap_in_cached_blocks_breaks_prefix(gpu):
    """prefix_semantics.rs:33-57: h0, h2, h3 cached -> the prefix stops at h1."""
    e, _ = _one_layer_engine("test-gap-prefix", 3, 1024, pool_size=1 << 20)
    h = make_block_hashes(4, 20)
    _save(e, "test-gap-prefix", [h[0], h[2], h[3]])
    assert _hits_then_release(e, "test-gap-prefix", h) == 1
    e.close()


def test_first_block_missing_yields_zero_prefix_hit(gpu):
    """prefix_semantics.rs:60-82: no lease is created for zero hits."""
    e, _ = _one_layer_engine("test-no-prefix", 3, 1024, pool_size=1 << 20)
    h = make_block_hashes(4, 30)
    _save(e, "test-no-prefix", [h[1], h[2], h[3]])
    assert e.query_prefix("test-no-prefix", h) == (0, 0)
    e.close()


def test_miss_does_not_poison_later_hit_and_empty_query(gpu):
    """prefix_semantics.rs:86-127: a miss leaves no state behind; an empty
    query is zero hits."""
    e, _ = _one_layer_engine("test-ram-miss-then-hit", 4, 1024, pool_size=1 << 20)
    h = make_block_hashes(4, 40)
    assert e.query_prefix("test-ram-miss-then-hit", h) == (0, 0)
    _save(e, "test-ram-miss-then-hit", h)
    assert _hits_then_release(e, "test-ram-miss-then-hit", h) == 4
    assert e.query_prefix("test-ram-miss-then-hit", []) == (0, 0)
    e.close()


@pytest.mark.parametrize("shards", [1, 2], ids=["one_pool", "two_shards"])
def test_eviction_reclaims_old_blocks_for_new(gpu, shards):
    """eviction.rs:27-48,87-107: the pool fits two batches of 4 x 4096 B; the new
    batch round-trips with the overwritten data, also with a sharded pool."""
    e, layer = _one_layer_engine("inst-evict", 4, 4096, pool_size=4 * 4096 * 2, pool_shards=shards)
    _save(e, "inst-evict", make_block_hashes(4, 1))
    overwritten = (layer.expected.astype(np.uint16) + 42).astype(np.uint8)
    layer.gpu.copy_from_host(overwritten)
    new = make_block_hashes(4, 2)
    _save(e, "inst-evict", new)
    _save(e, "inst-evict", make_block_hashes(4, 3))          # a third batch must evict the first
    assert _hits_then_release(e, "inst-evict", make_block_hashes(4, 1)) == 0
    layer.zero_gpu()
    hits, lease = e.query_prefix("inst-evict", new)
    assert hits == 4
    e.batch_load_kv_blocks_multi_layer("inst-evict", 0, 0, [["layer_0"]], lease, [[0, 1, 2, 3]]).wait()
    layer.assert_gpu_matches(overwritten)
    e.close()


def test_leased_blocks_survive_eviction_pressure(gpu):
    """eviction.rs:52-84: a lease pins the blocks and their place in the cache."""
    e, layer = _one_layer_engine("inst-lease", 4, 4096, pool_size=4 * 4096 * 2)
    hashes = make_block_hashes(4, 10)
    _save(e, "inst-lease", hashes)
    hits, lease = e.query_prefix("inst-lease", hashes)
    assert hits == 4
    reclaimed = make_block_hashes(4, 20)
    _save(e, "inst-lease", reclaimed)
    _save(e, "inst-lease", make_block_hashes(4, 21))          # pressure: reclaims the unleased batch
    assert _hits_then_release(e, "inst-lease", reclaimed) == 0
    assert _hits_then_release(e, "inst-lease", hashes) == 4   # still the same prefix
    layer.zero_gpu()
    e.batch_load_kv_blocks_multi_layer("inst-lease", 0, 0, [["layer_0"]], lease, [[0, 1, 2, 3]]).wait()
    layer.assert_gpu_matches(layer.expected)
    e.close()


def test_unconsumed_lease_expires_and_frees_its_blocks(gpu):
    """lease.rs:11,47,91-118,174-181: a lease that no worker consumes (a crashed
    worker, a request aborted after the query) pins its blocks only until its
    time is up.  Afterwards a save under pool pressure may evict them instead of
    failing, and a load that still names the lease is told so."""
    import time
    e, layer = _one_layer_engine("inst-ttl", 4, 4096, pool_size=4 * 4096 * 2, lease_ttl_ms=800)
    first = make_block_hashes(4, 30)
    _save(e, "inst-ttl", first)
    hits, lease = e.query_prefix("inst-ttl", first)
    assert hits == 4 and e.live_leases() == 1
    _save(e, "inst-ttl", make_block_hashes(4, 31))           # fills the pool
    # while the lease lives, its blocks cannot go: the pool has no room for a third batch
    # once the unleased batch is gone, and the save fails rather than touch them
    _save(e, "inst-ttl", make_block_hashes(4, 32))           # evicts batch 31
    assert _hits_then_release(e, "inst-ttl", first) == 4
    hits2, lease2 = e.query_prefix("inst-ttl", make_block_hashes(4, 32))
    assert hits2 == 4                                         # now both resident batches are leased
    with pytest.raises(_lib.StorageError, match="exhausted|allocate"):
        _save(e, "inst-ttl", make_block_hashes(4, 33))
    time.sleep(1.0)                                           # both leases are past their time
    _save(e, "inst-ttl", make_block_hashes(4, 34))           # succeeds: expired leases no longer pin
    assert e.live_leases() == 0
    assert _hits_then_release(e, "inst-ttl", make_block_hashes(4, 34)) == 4
    with pytest.raises(_lib.StorageError, match="query lease is unknown or expired"):
        e.batch_load_kv_blocks_multi_layer("inst-ttl", 0, 0, [["layer_0"]], lease, [[0, 1, 2, 3]])
    with pytest.raises(_lib.StorageError, match="not found"):
        e.release_query_lease(lease2)                         # swept, like an unknown one
    e.close()


def test_lease_consumed_in_time_loads_and_sweep_counts(gpu):
    """A lease consumed before its time serves the load; the periodic sweep
    (lease.rs:66-80) drops only the ones that are past it."""
    import time
    e, layer = _one_layer_engine("inst-ttl2", 4, 1024, pool_size=1 << 20, lease_ttl_ms=1000)
    hashes = make_block_hashes(4, 40)
    _save(e, "inst-ttl2", hashes)
    _h, stale = e.query_prefix("inst-ttl2", hashes)
    time.sleep(0.6)
    _h, fresh = e.query_prefix("inst-ttl2", hashes)
    assert e.sweep_expired_leases() == 0 and e.live_leases() == 2
    time.sleep(0.6)                                           # `stale` is past its time, `fresh` is not
    assert e.sweep_expired_leases() == 1 and e.live_leases() == 1
    layer.zero_gpu()
    e.batch_load_kv_blocks_multi_layer("inst-ttl2", 0, 0, [["layer_0"]], fresh, [[0, 1, 2, 3]]).wait()
    layer.assert_gpu_matches(layer.expected)
    with pytest.raises(_lib.StorageError, match="query lease is unknown or expired"):
        e.batch_load_kv_blocks_multi_layer("inst-ttl2", 0, 0, [["layer_0"]], stale, [[0, 1, 2, 3]])
    e.close()


def test_recurrent_group_seals_final_block_save(engine):
    """hybrid_groups.rs:14-176: the recurrent group seals a tail-only checkpoint
    save, membership is per group, and one load with two leases restores the
    attention prefix and the recurrent state block (5 -> 7)."""
    attn_block, recur_block = 1024, 2048
    layers = [Layer("attn_0", 8, attn_block), Layer("attn_1", 8, attn_block, overwrite=3),
              Layer("recurrent_state", 8, recur_block, overwrite=9)]
    register(engine, "hybrid-hma", layers, ns="hybrid-hma-ns", groups=[0, 0, 1])
    hashes = make_block_hashes(8, 10)
    prefix = hashes[:3]
    engine.batch_save_kv_blocks("hybrid-hma", 0, 0, 0, [LayerSave("attn_0", [0, 1, 2], prefix),
                                                        LayerSave("attn_1", [0, 1, 2], prefix)])
    engine.batch_save_kv_blocks("hybrid-hma", 0, 0, 0, [LayerSave("recurrent_state", [5], [hashes[2]])])
    assert engine.query_group_membership("hybrid-hma", 0, prefix) == [True, True, True]
    assert engine.query_group_membership("hybrid-hma", 1, prefix) == [False, False, True]
    with pytest.raises(_lib.InvalidArgument):
        engine.query_group_membership("hybrid-hma", 2, prefix)       # unknown group: an error
    hits, attn_lease = engine.query_prefix("hybrid-hma", prefix)     # classic prefix query: group 0
    assert hits == 3
    recur_lease = engine.create_group_lease("hybrid-hma", 1, [hashes[2]])
    with pytest.raises(_lib.InvalidArgument, match="query lease requires at least one block"):
        engine.create_group_lease("hybrid-hma", 1, [])
    with pytest.raises(_lib.StorageError, match="not resident"):
        engine.create_group_lease("hybrid-hma", 1, [hashes[0]])
    # membership and lease in one step (what the QueryPrefetch handler uses)
    present, both = engine.query_group_lease("hybrid-hma", 1, prefix)
    assert present == [False, False, True] and both != 0
    engine.release_query_lease(both)
    present, none = engine.query_group_lease("hybrid-hma", 1, prefix, require_all=True)
    assert present == [False, False, True] and none == 0
    present, none = engine.query_group_lease("hybrid-hma", 1, prefix[:2])
    assert present == [False, False] and none == 0
    for l in layers:
        l.zero_gpu()
    state = LoadState()
    engine.batch_load_multi("hybrid-hma", 0, 0, [["attn_0", "attn_1"], ["recurrent_state"]], [
        (attn_lease, [[0, 1, 2], [None, None, None]]),
        (recur_lease, [[None], [7]]),
    ], state).wait()
    assert state.get() == LOAD_STATE_SUCCESS
    for l in layers[:2]:
        want = np.zeros_like(l.expected)
        want[:3 * attn_block] = l.expected[:3 * attn_block]
        l.assert_gpu_matches(want)
    want = np.zeros_like(layers[2].expected)
    want[7 * recur_block:8 * recur_block] = layers[2].expected[5 * recur_block:6 * recur_block]
    layers[2].assert_gpu_matches(want)
    state.close()


def test_single_group_instances_are_unaffected(engine):
    """hybrid_groups.rs:181-211: membership on an instance without layer groups
    answers for group 0; a group the instance does not have is an error, not an
    all-miss answer."""
    layers = [Layer("layer_0", 4, 1024), Layer("layer_1", 4, 1024)]
    register(engine, "hybrid-compat", layers, ns="hybrid-compat-ns")
    hashes = make_block_hashes(4, 7)
    engine.batch_save_kv_blocks("hybrid-compat", 0, 0, 0,
                                [LayerSave(l.name, [0, 1], hashes[:2]) for l in layers])
    assert engine.query_group_membership("hybrid-compat", 0, hashes) == [True, True, False, False]
    with pytest.raises(_lib.InvalidArgument):
        engine.query_group_membership("hybrid-compat", 7, hashes[:1])


def test_recurrent_membership_is_an_exact_want_set(engine):
    """hybrid_groups.rs:221-322: a recurrent want-set resolves only when every
    member is stored in that group; a set with an absent member comes back
    short and cannot be leased; a hash stored under the attention group alone
    never satisfies the recurrent set."""
    layers = [Layer("attn_0", 8, 1024), Layer("recurrent_state", 8, 2048, overwrite=5)]
    register(engine, "hybrid-pd", layers, ns="hybrid-pd-ns", groups=[0, 1])
    hashes = make_block_hashes(8, 21)
    engine.batch_save_kv_blocks("hybrid-pd", 0, 0, 0, [LayerSave("attn_0", [0, 1, 2], hashes[:3])])
    engine.batch_save_kv_blocks("hybrid-pd", 0, 0, 0,
                                [LayerSave("recurrent_state", [4, 5], [hashes[1], hashes[2]])])
    want = [hashes[1], hashes[2]]
    assert engine.query_group_membership("hybrid-pd", 1, want) == [True, True]
    lease = engine.create_group_lease("hybrid-pd", 1, want)          # complete set: leasable
    short = [hashes[1], hashes[5], hashes[2]]
    assert engine.query_group_membership("hybrid-pd", 1, short) == [True, False, True]
    with pytest.raises(_lib.StorageError, match="block 1 of the lease is not resident in group 1"):
        engine.create_group_lease("hybrid-pd", 1, short)
    assert engine.query_group_membership("hybrid-pd", 1, [hashes[0]]) == [False]
    assert engine.query_group_membership("hybrid-pd", 0, [hashes[0]]) == [True]
    # the leased checkpoints load in the requested order
    layers[1].zero_gpu()
    engine.batch_load_multi("hybrid-pd", 0, 0, [["attn_0"], ["recurrent_state"]],
                            [(lease, [[None, None], [6, 7]])]).wait()
    want_bytes = np.zeros_like(layers[1].expected)
    want_bytes[6 * 2048:8 * 2048] = layers[1].expected[4 * 2048:6 * 2048]
    layers[1].assert_gpu_matches(want_bytes)


def test_save_query_load_roundtrip_with_numa(gpu):
    """engine_basic.rs:160-176: the same round trip with one pinned pool per NUMA node."""
    e = PegaEngine(pool_size=64 << 20, numa_aware=True)
    layer = Layer("layer_0", 4, 1024)
    register(e, "test-roundtrip-numa", [layer])
    hashes = make_block_hashes(4, 0)
    e.batch_save_kv_blocks("test-roundtrip-numa", 0, 0, 0, [LayerSave("layer_0", [0, 1, 2, 3], hashes)])
    layer.zero_gpu()
    hits, lease = e.query_prefix("test-roundtrip-numa", hashes)
    assert hits == 4
    e.batch_load_kv_blocks_multi_layer("test-roundtrip-numa", 0, 0, [["layer_0"]], lease,
                                       [[0, 1, 2, 3]]).wait()
    layer.assert_gpu_matches(layer.expected)
    e.close()


def test_incomplete_blocks_wait_are_collected_and_late_saves_are_dropped(engine):
    """The write path's rules for blocks that do not have all their slots yet
    (storage/write_path.rs:445-603): a repeated slot changes nothing, a save
    from an instance with another slot count skips the key, a late save for a
    block that is already complete leaves nothing behind, and incomplete blocks
    that grow old are collected with their pinned memory."""
    two = [Layer("layer_0", 4, 1024), Layer("layer_1", 4, 1024)]
    four = [Layer(f"layer_{i}", 4, 1024, overwrite=7) for i in range(4)]
    register(engine, "two-slots", two, ns="shared")
    register(engine, "four-slots", four, ns="shared")
    h = make_block_hashes(2, 77)
    engine.batch_save_kv_blocks("two-slots", 0, 0, 0, [LayerSave("layer_0", [0, 1], h)])
    assert engine.inflight_blocks == 2 and engine.cached_blocks == 0
    used_one_slot = engine.pool_usage()[0]
    # the same slot again: idempotent
    engine.batch_save_kv_blocks("two-slots", 0, 0, 0, [LayerSave("layer_0", [2, 3], h)])
    assert engine.inflight_blocks == 2 and engine.query_prefix("two-slots", h) == (0, 0)
    # another layout tries to fill the same keys: skipped, nothing completes, nothing leaks
    engine.batch_save_kv_blocks("four-slots", 0, 0, 0, [LayerSave("layer_1", [0, 1], h)])
    assert engine.inflight_blocks == 2 and engine.cached_blocks == 0
    assert engine.pool_usage()[0] == used_one_slot
    # the rightful second slot completes both blocks, with the first slot's original bytes
    engine.batch_save_kv_blocks("two-slots", 0, 0, 0, [LayerSave("layer_1", [0, 1], h)])
    assert engine.inflight_blocks == 0 and engine.cached_blocks == 2
    used_sealed = engine.pool_usage()[0]
    # a late save for complete blocks is dropped without a trace
    engine.batch_save_kv_blocks("two-slots", 0, 0, 0, [LayerSave("layer_0", [0, 1], h)])
    assert engine.inflight_blocks == 0 and engine.pool_usage()[0] == used_sealed
    for l in two:
        l.zero_gpu()
    hits, lease = engine.query_prefix("two-slots", h)
    assert hits == 2
    engine.batch_load_kv_blocks_multi_layer("two-slots", 0, 0, [["layer_0", "layer_1"]], lease,
                                            [[0, 1]]).wait()
    for l in two:
        want = np.zeros_like(l.expected)
        want[:2048] = l.expected[:2048]
        l.assert_gpu_matches(want)
    # stale incomplete blocks: kept while young, collected when older than the limit
    g = make_block_hashes(3, 78)
    engine.batch_save_kv_blocks("two-slots", 0, 0, 0, [LayerSave("layer_0", [0, 1, 2], g)])
    assert engine.inflight_blocks == 3
    assert engine.gc_stale_inflight(60.0) == 0 and engine.inflight_blocks == 3
    assert engine.gc_stale_inflight(0.0) == 3 and engine.inflight_blocks == 0
    assert engine.pool_usage()[0] == used_sealed


def test_namespace_isolation(engine):
    """engine_basic.rs:254-271: blocks of one namespace are invisible to another."""
    a, b = Layer("layer_0", 4, 1024), Layer("layer_0", 4, 1024)
    register(engine, "inst-a", [a], ns="ns-a")
    register(engine, "inst-b", [b], ns="ns-b")
    hashes = make_block_hashes(4, 50)
    engine.batch_save_kv_blocks("inst-a", 0, 0, 0, [LayerSave("layer_0", [0, 1, 2, 3], hashes)])
    assert engine.query_prefix("inst-b", hashes) == (0, 0)
    hits, lease = engine.query_prefix("inst-a", hashes)
    assert hits == 4
    engine.release_query_lease(lease)


def test_load_requires_a_live_lease(engine):
    """prefetch_lease.rs:11-27: a released (or unknown) lease cannot be loaded."""
    layer = Layer("layer_0", 4, 1024)
    register(engine, "inst-lease-gone", [layer])
    hashes = make_block_hashes(4, 60)
    engine.batch_save_kv_blocks("inst-lease-gone", 0, 0, 0, [LayerSave("layer_0", [0, 1, 2, 3], hashes)])
    _hits, lease = engine.query_prefix("inst-lease-gone", hashes)
    engine.release_query_lease(lease)
    state = LoadState()
    with pytest.raises(_lib.StorageError, match="query lease is unknown or expired"):
        engine.batch_load_kv_blocks_multi_layer("inst-lease-gone", 0, 0, [["layer_0"]], lease,
                                                [[0, 1, 2, 3]], state)
    assert state.get() == LOAD_STATE_ERROR
    state.close()


def test_lease_of_another_instance_is_refused_without_being_consumed(engine):
    """lease.rs:192-219 through the load path (lib.rs:779-782)."""
    a, b = Layer("layer_0", 4, 1024), Layer("layer_0", 4, 1024)
    register(engine, "inst-a", [a], ns="shared-ns")
    register(engine, "inst-b", [b], ns="shared-ns")
    hashes = make_block_hashes(4, 70)
    engine.batch_save_kv_blocks("inst-a", 0, 0, 0, [LayerSave("layer_0", [0, 1, 2, 3], hashes)])
    _hits, lease = engine.query_prefix("inst-a", hashes)
    with pytest.raises(_lib.StorageError, match="query lease belongs to instance inst-a, got inst-b"):
        engine.batch_load_kv_blocks_multi_layer("inst-b", 0, 0, [["layer_0"]], lease, [[0, 1, 2, 3]])
    a.zero_gpu()
    engine.batch_load_kv_blocks_multi_layer("inst-a", 0, 0, [["layer_0"]], lease, [[0, 1, 2, 3]]).wait()
    a.assert_gpu_matches(a.expected)
    # consumed by its one worker (world size 1): a second load finds it gone
    with pytest.raises(_lib.StorageError, match="query lease is unknown or expired"):
        engine.batch_load_kv_blocks_multi_layer("inst-a", 0, 0, [["layer_0"]], lease, [[0, 1, 2, 3]])


def test_partially_cached_save_stores_only_the_new_blocks(engine):
    """engine_basic.rs:178-190 (dedupe) with a mixed list: hashes already in the
    cache are skipped position by position, the rest keep their own block ids."""
    layer = Layer("layer_0", 16, 1024)
    register(engine, "partial-dedupe", [layer])
    h = make_block_hashes(6, 80)
    engine.batch_save_kv_blocks("partial-dedupe", 0, 0, 0, [LayerSave("layer_0", [0, 1, 2, 3], h[:4])])
    used = engine.pool_usage()[0]
    # h2, h3 again (from other device blocks: must NOT be re-read), h4, h5 new
    engine.batch_save_kv_blocks("partial-dedupe", 0, 0, 0,
                                [LayerSave("layer_0", [9, 8, 7, 6], [h[2], h[3], h[4], h[5]])])
    assert engine.cached_blocks == 6
    assert engine.pool_usage()[0] == used + 2 * 1024
    layer.zero_gpu()
    hits, lease = engine.query_prefix("partial-dedupe", h)
    assert hits == 6
    engine.batch_load_kv_blocks_multi_layer("partial-dedupe", 0, 0, [["layer_0"]], lease,
                                            [[10, 11, 12, 13, 14, 15]]).wait()
    want = np.zeros_like(layer.expected)
    for dst, src in zip(range(10, 16), [0, 1, 2, 3, 7, 6]):
        want[dst * 1024:(dst + 1) * 1024] = layer.expected[src * 1024:(src + 1) * 1024]
    layer.assert_gpu_matches(want)


def test_lower_staging_threshold_moves_the_same_bytes(gpu):
    """pf_engine_config.auto_staged_min_bytes: with the workers' threshold at
    1 MiB a 6 MiB save and load go through device staging instead of the
    resident zero-copy kernel; the bytes are the same."""
    e = PegaEngine(pool_size=64 << 20, auto_staged_min_bytes=1 << 20)
    layers = [Layer(f"layer_{i}", 64, 16384, split_kv_stride=64 * 16384) for i in range(3)]
    register(e, "staged-small", layers)
    hashes = make_block_hashes(48, 3)
    ids = list(range(8, 56))
    e.batch_save_kv_blocks("staged-small", 0, 0, 0, [LayerSave(l.name, ids, hashes) for l in layers])
    for l in layers:
        l.zero_gpu()
    hits, lease = e.query_prefix("staged-small", hashes)
    assert hits == 48
    dest = list(range(0, 48))
    e.batch_load_kv_blocks_multi_layer("staged-small", 0, 0, [[l.name for l in layers]], lease,
                                       [dest]).wait()
    for l in layers:
        want = np.zeros_like(l.expected)
        view = want.reshape(2, 64, 16384)
        src = l.expected.reshape(2, 64, 16384)
        view[:, dest] = src[:, ids]
        l.assert_gpu_matches(want)
    e.close()


@pytest.mark.parametrize("mode,use_desc,small_paths,large_paths", [
    (TransferMode.DIRECT, False, ("zerocopy",), ("staged",)),
    (TransferMode.KERNEL, False, ("zerocopy",), ("staged",)),
    (TransferMode.ZEROCOPY, False, ("zerocopy",), ("zerocopy",)),
    (TransferMode.DIRECT, True, ("descriptors",), ("descriptors",)),
    (TransferMode.KERNEL, True, ("descriptors",), ("descriptors",)),
], ids=["direct", "kernel", "zerocopy", "direct-descriptors", "kernel-descriptors"])
def test_task_result_reports_the_path_taken(gpu, mode, use_desc, small_paths, large_paths):
    """pf_task_result.paths: a 4 MiB task and a 300 MiB task through the workers
    of each mode.  `direct` and `kernel` pools choose per task (zero-copy kernel
    below 8 MiB of dense layers, staged above), a `zerocopy` pool never stages,
    descriptor pools go through the backends; the bytes are checked each time."""
    rng = np.random.default_rng(77)
    seg, nb = 32768, 5120                      # one K/V-split layer of 320 MiB
    cache0 = random_bytes(rng, 2 * nb * seg)
    dev = DeviceBuffer(cache0.nbytes)
    dev.copy_from_host(cache0)
    layout = KVCacheLayout(dev.ptr, cache0.nbytes, nb, seg, nb * seg, 2)
    kv = cache0.reshape(2, nb, seg)
    pool = GpuWorkerPool(0, -1, mode, use_descriptor_backends=use_desc)
    expected_staging = 0 if (use_desc or mode == TransferMode.ZEROCOPY) else 4 * (512 << 20)
    assert pool.staging_bytes == expected_staging
    for n, paths in ((64, small_paths), (4800, large_paths)):   # 4 MiB, 300 MiB
        host = PinnedMemory(2 * n * seg)
        host.as_numpy()[:] = 0
        ids = rng.choice(nb, n, replace=False)
        blocks = [HostBlock((host.host_ptr + i * seg, host.host_ptr + (n + i) * seg),
                            (host.device_ptr + i * seg, host.device_ptr + (n + i) * seg), (1, 2),
                            (seg, seg)) for i in range(n)]
        res = pool.batch_save([LayerTransferData("kv", layout, ids, blocks)]).wait()
        assert res.paths == paths, (n, res)
        assert res.bytes == 2 * n * seg
        if "staged" in paths:
            assert res.staged_groups >= 1 and res.link_copies >= 1 and res.zero_copy_launches == 0
        if paths == ("zerocopy",):
            assert res.zero_copy_launches >= 1 and res.staged_groups == 0
        # nothing is allocated inside a task: the slots exist since the pool was spawned
        assert res.phases_ms["staging_alloc"] == 0.0
        assert res.phases_ms["sync"] > 0.0 and res.elapsed_ms >= res.phases_ms["sync"]
        img = host.as_numpy().reshape(2, n, seg)
        assert np.array_equal(img[0], kv[0, ids]) and np.array_equal(img[1], kv[1, ids])
        dest = rng.choice(nb, n, replace=False)
        dev.fill(0)
        res = pool.submit_load([LayerTransferData("kv", layout, dest, blocks)], None).wait()
        assert res.paths == paths, (n, res)
        got = dev.copy_to_host().reshape(2, nb, seg)
        assert np.array_equal(got[:, dest], kv[:, ids])
        rest = np.ones(nb, dtype=bool)
        rest[dest] = False
        assert not got[:, rest].any()
        dev.copy_from_host(cache0)
        host.close()
    assert pool.staging_bytes == expected_staging
    pool.close()
    dev.close()


def test_lazy_staging_allocates_on_the_first_staged_task(gpu):
    """pf_worker_pool_config.lazy_staging / staging_slot_bytes: nothing is held
    until a worker stages, then two slots of the configured size per worker."""
    rng = np.random.default_rng(78)
    seg, nb, n = 32768, 1024, 512               # 32 MiB task
    cache0 = random_bytes(rng, 2 * nb * seg)
    dev = DeviceBuffer(cache0.nbytes)
    dev.copy_from_host(cache0)
    layout = KVCacheLayout(dev.ptr, cache0.nbytes, nb, seg, nb * seg, 2)
    pool = GpuWorkerPool(0, -1, TransferMode.DIRECT, staging_slot_bytes=48 << 20, lazy_staging=True)
    assert pool.staging_bytes == 0
    host = PinnedMemory(2 * n * seg)
    ids = rng.choice(nb, n, replace=False)
    blocks = [HostBlock((host.host_ptr + i * seg, host.host_ptr + (n + i) * seg),
                        (host.device_ptr + i * seg, host.device_ptr + (n + i) * seg), (1, 2),
                        (seg, seg)) for i in range(n)]
    res = pool.batch_save([LayerTransferData("kv", layout, ids, blocks)]).wait()
    assert res.paths == ("staged",) and res.phases_ms["staging_alloc"] > 0.0
    assert pool.staging_bytes == 2 * (48 << 20)          # the save worker's two slots
    img = host.as_numpy().reshape(2, n, seg)
    kv = cache0.reshape(2, nb, seg)
    assert np.array_equal(img[0], kv[0, ids]) and np.array_equal(img[1], kv[1, ids])
    res = pool.batch_save([LayerTransferData("kv", layout, ids, blocks)]).wait()
    assert res.phases_ms["staging_alloc"] == 0.0
    pool.close()
    host.close()
    dev.close()


def test_pool_without_room_for_staging_still_moves_tasks(gpu):
    """A pool whose staging slots cannot be allocated (1 TiB each) is spawned
    all the same, holds no staging memory, and moves a 32 MiB task - which it
    would stage - over the zero-copy path, bytes as ever."""
    rng = np.random.default_rng(80)
    seg, nb, n = 32768, 1024, 512
    cache0 = random_bytes(rng, 2 * nb * seg)
    dev = DeviceBuffer(cache0.nbytes)
    dev.copy_from_host(cache0)
    layout = KVCacheLayout(dev.ptr, cache0.nbytes, nb, seg, nb * seg, 2)
    pool = GpuWorkerPool(0, -1, TransferMode.DIRECT, staging_slot_bytes=1 << 40)
    assert pool.staging_bytes == 0
    host = PinnedMemory(2 * n * seg)
    ids = rng.choice(nb, n, replace=False)
    blocks = [HostBlock((host.host_ptr + i * seg, host.host_ptr + (n + i) * seg),
                        (host.device_ptr + i * seg, host.device_ptr + (n + i) * seg), (1, 2),
                        (seg, seg)) for i in range(n)]
    res = pool.batch_save([LayerTransferData("kv", layout, ids, blocks)]).wait()
    assert res.paths == ("zerocopy",)
    img = host.as_numpy().reshape(2, n, seg)
    kv = cache0.reshape(2, nb, seg)
    assert np.array_equal(img[0], kv[0, ids]) and np.array_equal(img[1], kv[1, ids])
    dest = rng.choice(nb, n, replace=False)
    dev.fill(0)
    res = pool.submit_load([LayerTransferData("kv", layout, dest, blocks)]).wait()
    assert res.paths == ("zerocopy",)
    got = dev.copy_to_host().reshape(2, nb, seg)
    assert np.array_equal(got[:, dest], kv[:, ids])
    pool.close()
    host.close()
    dev.close()


def test_side_copy_streams_move_the_same_bytes(gpu):
    """pf_worker_pool_config.side_copy_streams: the workers' link copies on a
    second stream each.  Four layers of 24 MiB in 32 MiB slots (several fills per
    task, so copies and kernels do overlap), saved and loaded back into other
    blocks; bytes as without the knob."""
    rng = np.random.default_rng(79)
    seg, nb, n, n_layers = 32768, 512, 384, 4
    caches0 = [random_bytes(rng, 2 * nb * seg) for _ in range(n_layers)]
    devs = [DeviceBuffer(c.nbytes) for c in caches0]
    for d, c in zip(devs, caches0):
        d.copy_from_host(c)
    layouts = [KVCacheLayout(d.ptr, c.nbytes, nb, seg, nb * seg, 2) for d, c in zip(devs, caches0)]
    pool = GpuWorkerPool(0, -1, TransferMode.DIRECT, staging_slot_bytes=32 << 20,
                         side_copy_streams=True)
    hosts = [PinnedMemory(2 * n * seg) for _ in range(n_layers)]
    ids = rng.choice(nb, n, replace=False)

    def blocks_of(host):
        return [HostBlock((host.host_ptr + i * seg, host.host_ptr + (n + i) * seg),
                          (host.device_ptr + i * seg, host.device_ptr + (n + i) * seg), (1, 2),
                          (seg, seg)) for i in range(n)]

    res = pool.batch_save([LayerTransferData(f"kv{li}", layouts[li], ids, blocks_of(hosts[li]))
                           for li in range(n_layers)]).wait()
    assert res.paths == ("staged",) and res.staged_groups >= 3
    for li in range(n_layers):
        img = hosts[li].as_numpy().reshape(2, n, seg)
        kv = caches0[li].reshape(2, nb, seg)
        assert np.array_equal(img[0], kv[0, ids]) and np.array_equal(img[1], kv[1, ids]), li
    dest = rng.choice(nb, n, replace=False)
    for d in devs:
        d.fill(0)
    res = pool.submit_load([LayerTransferData(f"kv{li}", layouts[li], dest, blocks_of(hosts[li]))
                           for li in range(n_layers)]).wait()
    assert res.paths == ("staged",) and res.staged_groups >= 3
    rest = np.ones(nb, dtype=bool)
    rest[dest] = False
    for li in range(n_layers):
        got = devs[li].copy_to_host().reshape(2, nb, seg)
        kv = caches0[li].reshape(2, nb, seg)
        assert np.array_equal(got[:, dest], kv[:, ids]), li
        assert not got[:, rest].any(), li
    pool.close()
    for h in hosts:
        h.close()
    for d in devs:
        d.close()


def test_engine_load_profile_and_staging_report(gpu):
    """pf_engine_last_load_profile mirrors the task's own result; a context's
    staging is sized by what its layers can fill, not by the 512 MiB default;
    kernel_mode_zerocopy gives KERNEL registrations the reference's kernel mode."""
    e = PegaEngine(pool_size=64 << 20)
    assert e.last_load_profile() is None
    layers = [Layer(f"layer_{i}", 64, 16384, split_kv_stride=64 * 16384) for i in range(3)]
    register(e, "profile", layers)
    # 2 MiB layers: slots at the 32 MiB floor, 2 workers x 2 slots
    assert e.staging_bytes == 4 * (32 << 20)
    hashes = make_block_hashes(48, 5)
    ids = list(range(8, 56))
    e.batch_save_kv_blocks("profile", 0, 0, 0, [LayerSave(l.name, ids, hashes) for l in layers])
    _hits, lease = e.query_prefix("profile", hashes)
    res = e.batch_load_kv_blocks_multi_layer("profile", 0, 0, [[l.name for l in layers]], lease,
                                             [ids]).wait()
    assert res.paths == ("zerocopy",)            # 4.5 MiB of dense layers: below the 8 MiB rule
    last = e.last_load_profile()
    assert last.bytes == res.bytes == 3 * 48 * 2 * 16384
    assert last.paths == res.paths and last.phases_ms == res.phases_ms
    assert res.phases_ms["resolve"] > 0.0
    e.close()
    z = PegaEngine(pool_size=64 << 20, kernel_mode_zerocopy=True)
    zlayers = [Layer(f"layer_{i}", 64, 16384, split_kv_stride=64 * 16384) for i in range(2)]
    register(z, "kernel-as-reference", zlayers, mode=TransferMode.KERNEL)
    assert z.staging_bytes == 0
    z.close()
