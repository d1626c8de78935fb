"""The benchmark configurations at their full sizes.

configs[0] (Qwen3-0.6B, the reference's CPU-runnable case) is small enough
for the oracle: the product's bytes are compared with the oracle's on every
layer.  The larger shapes (Llama-3.1-8B, Llama-3-70B fp8, DeepSeek-V3 MLA
page-first) are checked through properties that do not depend on the size:
save followed by load moves block save_ids[i] of the source cache to block
load_ids[i] of the destination cache and nothing else, and the host image
holds the blocks in list order (K buffer then V buffer per layer, or one page
per block with layers at their sorted-name offsets)."""

import numpy as np
import pytest

from bench import make_ids
from oracle import oracle as O
from pegaflow_amd.layout import KVCacheLayout
from pegaflow_amd.pool import LayerTopology, WorkerLayers
from pegaflow_amd.runtime import PinnedMemory, Stream
from pegaflow_amd.transfer import BlockTransfer, LayerBlocks, TransferPath
from tests.helpers import random_bytes

QWEN = dict(layers=28, num_blocks=2048, seg=32768, n=64)


def qwen_inputs(layers):
    """Layer caches [2, 2048, 16*8*128 bf16] as bytes and per-layer id draws."""
    rng = np.random.default_rng(0)
    nb, seg, n = QWEN["num_blocks"], QWEN["seg"], QWEN["n"]
    base = random_bytes(rng, 2 * nb * seg)
    caches = [base ^ np.uint8(li + 1) for li in range(layers)]
    ids = [rng.choice(nb, n, replace=False).astype(np.uint32) for _ in range(layers)]
    return caches, ids


def test_configs0_oracle_equals_numpy_gather():
    nb, seg, n = QWEN["num_blocks"], QWEN["seg"], QWEN["n"]
    caches, ids = qwen_inputs(QWEN["layers"])
    for cache, lid in zip(caches, ids):
        layout = O.layout_over(cache, nb, seg, nb * seg, 2)
        hk = np.zeros(n * seg, dtype=np.uint8)
        hv = np.zeros(n * seg, dtype=np.uint8)
        O.transfer_layer(layout, lid, hk, hv, host_is_src=False, backend="direct", threads=4)
        wk, wv = O.np_save_split(cache, nb, seg, lid)
        assert np.array_equal(hk, wk.reshape(-1)) and np.array_equal(hv, wv.reshape(-1))
        back = np.zeros_like(cache)
        O.transfer_layer(O.layout_over(back, nb, seg, nb * seg, 2), lid, hk, hv, host_is_src=True,
                         backend="kernel", threads=4)
        want = np.zeros_like(cache)
        O.np_load_split(want, nb, seg, lid, wk, wv)
        assert np.array_equal(back, want)


# ---------------------------------------------------------------------------
# GPU, full sizes
# ---------------------------------------------------------------------------

@pytest.fixture(scope="module")
def torch_dev(gpu):
    import torch
    torch.cuda.set_device(0)
    yield torch
    torch.cuda.empty_cache()


@pytest.mark.gpu
@pytest.mark.parametrize("path", [TransferPath.ZEROCOPY, TransferPath.STAGED],
                         ids=["zerocopy", "staged"])
def test_configs0_full_size_matches_oracle(path, torch_dev):
    torch = torch_dev
    nb, seg, n, layers = QWEN["num_blocks"], QWEN["seg"], QWEN["n"], QWEN["layers"]
    caches, ids = qwen_inputs(layers)
    dev = [torch.from_numpy(c).cuda() for c in caches]
    back = [torch.zeros_like(t) for t in dev]
    torch.cuda.synchronize()
    pool = PinnedMemory(layers * 2 * n * seg)
    img = pool.as_numpy()
    img[:] = 0xEE
    stream, xfer = Stream(), BlockTransfer()

    def layer_blocks(tensors):
        out = []
        for li, t in enumerate(tensors):
            off = li * 2 * n * seg
            out.append(LayerBlocks(
                layout=KVCacheLayout(t.data_ptr(), 2 * nb * seg, nb, seg, nb * seg, 2),
                block_ids=ids[li],
                host=(pool.host_ptr + off, pool.host_ptr + off + n * seg),
                host_device=(pool.device_ptr + off, pool.device_ptr + off + n * seg),
                host_len=(n * seg, n * seg), host_stride=seg))
        return out

    try:
        xfer.save(layer_blocks(dev), stream, path)
        stream.synchronize()
        for li, cache in enumerate(caches):
            hk = np.zeros(n * seg, dtype=np.uint8)
            hv = np.zeros(n * seg, dtype=np.uint8)
            O.transfer_layer(O.layout_over(cache, nb, seg, nb * seg, 2), ids[li], hk, hv,
                             host_is_src=False, backend="direct", threads=4)
            off = li * 2 * n * seg
            assert np.array_equal(img[off:off + n * seg], hk), f"layer {li} K image"
            assert np.array_equal(img[off + n * seg:off + 2 * n * seg], hv), f"layer {li} V image"
        xfer.load(layer_blocks(back), stream, path)
        stream.synchronize()
        for li in range(layers):
            want = np.zeros(2 * nb * seg, dtype=np.uint8)
            off = li * 2 * n * seg
            O.transfer_layer(O.layout_over(want, nb, seg, nb * seg, 2), ids[li],
                             img[off:off + n * seg], img[off + n * seg:off + 2 * n * seg],
                             host_is_src=True, backend="kernel", threads=4)
            assert np.array_equal(back[li].cpu().numpy(), want), f"layer {li} cache after load"
    finally:
        xfer.close()
        stream.close()
        pool.close()


FULL = {
    # name: layers, num_blocks, segment bytes, segments, n ids, id pattern, page-first
    "llama8b": (32, 8192, 32768, 2, 5000, "permutation", False),
    "llama70b_fp8": (80, 16384, 16384, 2, 8192, "runs_and_singles", False),
    "dsv3_mla": (61, 4096, 73728, 1, 2048, "permutation", True),
}


@pytest.mark.gpu
@pytest.mark.parametrize("path", [TransferPath.AUTO, TransferPath.ZEROCOPY], ids=["auto", "zerocopy"])
@pytest.mark.parametrize("name", sorted(FULL))
def test_full_size_round_trip_properties(name, path, torch_dev):
    torch = torch_dev
    layers, nb, seg, nseg, n, id_kind, page_first = FULL[name]
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    src = [torch.empty(nseg * nb * seg, device=dev, dtype=torch.uint8).random_(0, 256, generator=gen)
           for _ in range(layers)]
    dst = [torch.zeros(nseg * nb * seg, device=dev, dtype=torch.uint8) for _ in range(layers)]
    save_ids = make_ids(np, id_kind, nb, n, 0)
    load_ids = make_ids(np, "permutation", nb, n, 1)
    assert len(set(save_ids.tolist())) == n and len(set(load_ids.tolist())) == n
    names = [f"model.layers.{li}.self_attn.attn" for li in range(layers)]
    payload = layers * nseg * n * seg
    pool = PinnedMemory(payload)
    torch.cuda.synchronize()
    stream, xfer = Stream(), BlockTransfer()

    def layouts(tensors):
        return [KVCacheLayout(t.data_ptr(), nseg * nb * seg, nb, seg, nb * seg if nseg == 2 else 0, nseg)
                for t in tensors]

    if page_first:
        topo = LayerTopology([WorkerLayers(0, 0, dict(zip(names, layouts(src))))], tp_size=1,
                             page_first=True)
        page = topo.shard_page_size(0)
        assert page == layers * seg
        offsets = [topo.page_placement(topo.layer_id(nm))[0] for nm in names]
        # ids follow the byte-wise sorted names: "…layers.10…" sorts before "…layers.2…"
        assert offsets[2] > offsets[10]
        ph = (pool.host_ptr + np.arange(n, dtype=np.uint64) * page).astype(np.uint64)
        pd = (pool.device_ptr + np.arange(n, dtype=np.uint64) * page).astype(np.uint64)

        def blocks(tensors, ids):
            return [LayerBlocks(layout=L, block_ids=ids, page_host=ph, page_host_device=pd,
                                page_offset=offsets[li], page_len=page, layer_name=names[li])
                    for li, L in enumerate(layouts(tensors))]
    else:
        buf = n * seg

        def blocks(tensors, ids):
            out = []
            for li, L in enumerate(layouts(tensors)):
                off = li * nseg * buf
                out.append(LayerBlocks(
                    layout=L, block_ids=ids,
                    host=tuple(pool.host_ptr + off + s * buf for s in range(nseg)),
                    host_device=tuple(pool.device_ptr + off + s * buf for s in range(nseg)),
                    host_len=tuple(buf for _ in range(nseg)), host_stride=seg, layer_name=names[li]))
            return out

    try:
        xfer.save(blocks(src, save_ids), stream, path)
        xfer.load(blocks(dst, load_ids), stream, path)
        stream.synchronize()
        want_path = TransferPath.ZEROCOPY if path == TransferPath.ZEROCOPY else TransferPath.STAGED
        assert xfer.last_path == want_path
        sid = torch.from_numpy(save_ids.astype(np.int64)).to(dev)
        lid = torch.from_numpy(load_ids.astype(np.int64)).to(dev)
        untouched = torch.ones(nb, dtype=torch.bool, device=dev)
        untouched[lid] = False
        rest = torch.nonzero(untouched).reshape(-1)
        img = torch.from_numpy(pool.as_numpy())
        for li in range(layers):
            s = src[li].view(nseg, nb, seg)
            d = dst[li].view(nseg, nb, seg)
            assert torch.equal(d[:, lid], s[:, sid]), f"{name} layer {li}: moved blocks differ"
            assert not bool(d[:, rest].any()), f"{name} layer {li}: a block outside the list changed"
            if li in (0, 10, layers - 1):
                want = s[:, sid].cpu()
                if page_first:
                    got = img.view(n, page)[:, offsets[li]:offsets[li] + seg].reshape(1, n, seg)
                else:
                    off = li * nseg * n * seg
                    got = img[off:off + nseg * n * seg].view(nseg, n, seg)
                assert torch.equal(got, want), f"{name} layer {li}: host image"
    finally:
        xfer.close()
        stream.close()
        pool.close()
        del src, dst
        torch.cuda.empty_cache()


@pytest.mark.gpu
@pytest.mark.parametrize("shape", ["llama8b", "llama70b_fp8", "dsv3_mla"])
@pytest.mark.parametrize("backend_name", ["kernel", "direct"])
def test_full_fragment_sizes_through_the_descriptor_backends(backend_name, shape, torch_dev):
    """The reference-compatible backends at the fragment sizes and counts of
    the benchmark shapes (8 layers of each): one descriptor per fragment, K
    before V, device -> host, then host -> device into other slots; every
    block of every layer is compared on the device."""
    from pegaflow_amd.transfer import KernelBackend, MemcpyBackend, desc_array
    torch = torch_dev
    _, nb, seg, nseg, n, id_kind, _ = FULL[shape]
    layers = 8
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(4321)
    src = [torch.empty(nseg * nb * seg, device=dev, dtype=torch.uint8).random_(0, 256, generator=gen)
           for _ in range(layers)]
    dst = [torch.zeros(nseg * nb * seg, device=dev, dtype=torch.uint8) for _ in range(layers)]
    save_ids = make_ids(np, id_kind, nb, n, 0).astype(np.uint64)
    load_ids = make_ids(np, "permutation", nb, n, 1).astype(np.uint64)
    pool = PinnedMemory(layers * nseg * n * seg)
    torch.cuda.synchronize()
    stream = Stream()
    backend = KernelBackend() if backend_name == "kernel" else MemcpyBackend()
    pos = np.arange(n, dtype=np.uint64)

    def descriptors(tensors, ids):
        """[layer][block][segment] order, as build_copy_descs emits them."""
        per_layer = []
        for li, t in enumerate(tensors):
            rows = np.empty((n, nseg, 6), dtype=np.uint64)
            for s in range(nseg):
                host_off = (li * nseg + s) * n * seg + pos * seg
                rows[:, s, 0] = t.data_ptr() + s * nb * seg + ids * seg
                rows[:, s, 1] = pool.host_ptr + host_off
                rows[:, s, 2] = pool.device_ptr + host_off
                rows[:, s, 3] = seg
                rows[:, s, 4] = li
                rows[:, s, 5] = 1 + li * nseg + s       # one allocation per layer segment
            per_layer.append(rows.reshape(n * nseg, 6))
        rows = np.concatenate(per_layer)
        return desc_array(rows[:, 0], rows[:, 1], rows[:, 2], rows[:, 3], rows[:, 4], rows[:, 5])

    try:
        backend.d2h(descriptors(src, save_ids), stream)
        backend.h2d(descriptors(dst, load_ids), stream)
        stream.synchronize()
        sid = torch.from_numpy(save_ids.astype(np.int64)).to(dev)
        lid = torch.from_numpy(load_ids.astype(np.int64)).to(dev)
        untouched = torch.ones(nb, dtype=torch.bool, device=dev)
        untouched[lid] = False
        rest = torch.nonzero(untouched).reshape(-1)
        for li in range(layers):
            s = src[li].view(nseg, nb, seg)
            d = dst[li].view(nseg, nb, seg)
            assert torch.equal(d[:, lid], s[:, sid]), f"{shape} layer {li}: moved blocks differ"
            assert not bool(d[:, rest].any()), f"{shape} layer {li}: a block outside the list changed"
    finally:
        backend.close()
        stream.close()
        pool.close()
        del src, dst
        torch.cuda.empty_cache()


@pytest.mark.gpu
@pytest.mark.parametrize("config,path", [
    (dict(tile_unroll=1), TransferPath.ZEROCOPY),
    (dict(tile_unroll=2), TransferPath.ZEROCOPY),
    (dict(tile_unroll=8), TransferPath.ZEROCOPY),
    (dict(zerocopy_max_workgroups=8), TransferPath.ZEROCOPY),
    (dict(zerocopy_max_workgroups=4096), TransferPath.ZEROCOPY),
    (dict(staging_slot_bytes=48 << 20), TransferPath.STAGED),               # five units per layer
    (dict(staging_slot_bytes=48 << 20, staging_slots=3, copy_stream=1), TransferPath.STAGED),
    (dict(staging_slot_bytes=48 << 20, copy_stream=2), TransferPath.STAGED),
    (dict(copy_stream=1), TransferPath.STAGED),
    (dict(auto_staged_min_bytes=1 << 40), TransferPath.AUTO),               # never staged
    (dict(auto_staged_min_bytes=1 << 20), TransferPath.AUTO),               # staged from 1 MiB
], ids=lambda v: ",".join(f"{k}={x}" for k, x in v.items()) if isinstance(v, dict) else str(int(v)))
def test_engine_options_do_not_change_the_bytes(config, path, torch_dev):
    """Every option of the block-ID engine (tile size of the zero-copy kernel,
    its workgroup cap, staging slot size and count, where the link copies run,
    the AUTO threshold) on 4 layers x 3000 blocks of the Llama shape: the same
    blocks land in the same places."""
    torch = torch_dev
    layers, nb, seg, nseg, n = 4, 8192, 32768, 2, 3000
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(99)
    src = [torch.empty(nseg * nb * seg, device=dev, dtype=torch.uint8).random_(0, 256, generator=gen)
           for _ in range(layers)]
    dst = [torch.zeros(nseg * nb * seg, device=dev, dtype=torch.uint8) for _ in range(layers)]
    save_ids = make_ids(np, "permutation", nb, n, 5)
    load_ids = make_ids(np, "permutation", nb, n, 6)
    buf = n * seg
    pool = PinnedMemory(layers * nseg * buf)
    torch.cuda.synchronize()
    stream, xfer = Stream(), BlockTransfer(**config)

    def blocks(tensors, ids):
        return [LayerBlocks(
            layout=KVCacheLayout(t.data_ptr(), nseg * nb * seg, nb, seg, nb * seg, nseg),
            block_ids=ids,
            host=tuple(pool.host_ptr + (li * nseg + s) * buf for s in range(nseg)),
            host_device=tuple(pool.device_ptr + (li * nseg + s) * buf for s in range(nseg)),
            host_len=(buf, buf), host_stride=seg, layer_name=f"layer{li}")
            for li, t in enumerate(tensors)]

    try:
        xfer.save(blocks(src, save_ids), stream, path)
        xfer.load(blocks(dst, load_ids), stream, path)
        stream.synchronize()
        if "auto_staged_min_bytes" in config:
            staged = config["auto_staged_min_bytes"] <= nseg * buf
            assert xfer.last_path == (TransferPath.STAGED if staged else TransferPath.ZEROCOPY)
        sid = torch.from_numpy(save_ids.astype(np.int64)).to(dev)
        lid = torch.from_numpy(load_ids.astype(np.int64)).to(dev)
        untouched = torch.ones(nb, dtype=torch.bool, device=dev)
        untouched[lid] = False
        rest = torch.nonzero(untouched).reshape(-1)
        img = torch.from_numpy(pool.as_numpy())
        for li in range(layers):
            s = src[li].view(nseg, nb, seg)
            d = dst[li].view(nseg, nb, seg)
            assert torch.equal(d[:, lid], s[:, sid]), f"layer {li}: moved blocks differ"
            assert not bool(d[:, rest].any()), f"layer {li}: a block outside the list changed"
            got = img[li * nseg * buf:(li + 1) * nseg * buf].view(nseg, n, seg)
            assert torch.equal(got, s[:, sid].cpu()), f"layer {li}: host image"
    finally:
        xfer.close()
        stream.close()
        pool.close()
        del src, dst
        torch.cuda.empty_cache()
