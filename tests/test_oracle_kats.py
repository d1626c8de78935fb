"""Pins the CPU oracle (oracle/pf_oracle.c) against the reference's own
known-answer vectors (tests/golden/reference_kats.json) and against what the
mathematics fixes: the copy kernel's loop nest equals memcpy, and the layer
save/load equals numpy fancy indexing."""

import numpy as np
import pytest

from oracle import oracle as O
from tests.helpers import kernel_test_pattern, random_bytes


def _build(case):
    L = O.Layout(*case["new"])
    if "with_block_stride" in case:
        L.with_block_stride(case["with_block_stride"])
    if "with_ssd_padding" in case:
        L.with_ssd_padding(case["with_ssd_padding"])
    return L


def test_layout_kats(kats):
    for case in kats["layout"]:
        exp = case["expect"]
        if "error_contains" in exp:
            with pytest.raises(O.OracleError, match=exp["error_contains"]):
                O.Layout(*case["new"])
            continue
        if "stride_error_contains" in exp:
            L = O.Layout(*case["new"])
            with pytest.raises(O.OracleError, match=exp["stride_error_contains"]):
                L.with_block_stride(case["with_block_stride"])
            continue
        L = _build(case)
        if "is_split" in exp:
            assert L.is_split == exp["is_split"], case["name"]
        for key in ("padded_segment_bytes", "padded_block_bytes"):
            if key in exp:
                assert getattr(L, key) == exp[key], case["name"]
        for idx, copies in exp.get("copies", {}).items():
            assert [list(c) for c in L.block_copies(int(idx))] == copies, case["name"]
        for idx in exp.get("out_of_range", []):
            with pytest.raises(O.OracleError, match="out of range"):
                L.block_copies(idx)


def test_merge_kats(kats):
    base = 0x7000_0000
    for case in kats["merge"]:
        rows = [(d, base + h, 0, s, da, ha) for d, h, s, da, ha in case["descs"]]
        assert [r[2] for r in O.merge(rows)] == case["expect_sizes"], case["name"]


def test_merge_is_greedy_left_to_right():
    # device contiguity alone is not enough: host must be contiguous too
    rows = [(0, 1000, 0, 10, 0, 0), (10, 2000, 0, 10, 0, 0)]
    assert len(O.merge(rows)) == 2
    # three in a row collapse into one range
    rows = [(0, 1000, 0, 10, 1, 1), (10, 1010, 0, 10, 1, 1), (20, 1020, 0, 10, 1, 1)]
    assert O.merge(rows) == [(0, 1000, 30)]
    # only LIST-adjacent entries are joined: a, c, b never merges a with b
    rows = [(0, 1000, 0, 10, 1, 1), (100, 1100, 0, 10, 1, 1), (10, 1010, 0, 10, 1, 1)]
    assert len(O.merge(rows)) == 3
    assert O.merge([]) == []


def test_merge_run_boundaries_exact():
    rows = [(0, 1000, 0, 10, 0, 0), (10, 1010, 0, 10, 0, 0), (30, 1020, 0, 10, 0, 0),
            (40, 1030, 0, 5, 0, 0), (45, 1035, 0, 5, 0, 0), (50, 1040, 0, 5, 0, 0),
            (55, 1045, 0, 5, 0, 9)]
    # (30,1020,10)+(40,1030,5): device 30+10 == 40 and host 1020+10 == 1030 -> joined
    assert O.merge(rows) == [(0, 1000, 20), (30, 1020, 25), (55, 1045, 5)]


def test_page_layout_kats(kats):
    for case in kats["page_layout"]:
        exp = case["expect"]
        if "error_contains" in exp:
            with pytest.raises(O.OracleError, match=exp["error_contains"]):
                O.build_page_layout(case["sets"], case["n_layers"], case["padded"])
            continue
        got = O.build_page_layout(case["sets"], case["n_layers"], case["padded"])
        for key, val in exp.items():
            assert got[key] == val, (case["name"], key)


def test_page_layout_shard_order_is_by_min_layer_id():
    # registration order {2,3} then {0,1}: shard 0 must still be the one holding layer 0
    got = O.build_page_layout([[2, 3], [0, 1]], 4, [100, 200, 300, 400])
    assert got["layer_shard"] == [0, 0, 1, 1]
    assert got["layer_offsets"] == [0, 100, 0, 300]
    assert got["shard_page_sizes"] == [300, 700]


def test_kernel_loop_nest_equals_memcpy():
    """The reference kernel (16-byte words + byte tail, or a byte loop when
    unaligned) writes exactly src[0:size) to dst[0:size) for any grid/block."""
    rng = np.random.default_rng(7)
    src = random_bytes(rng, 1 << 16)
    for grid, block in [(1, 1), (3, 7), (65535, 256), (5, 64)]:
        dst = np.zeros(1 << 16, dtype=np.uint8)
        expect = np.zeros_like(dst)
        table = []
        cursor = 0
        for size, so, do in [(4112, 0, 0), (33, 16, 32), (100, 5, 0), (17, 0, 3), (0, 0, 0),
                             (4096, 16, 16), (15, 0, 0), (1, 7, 9)]:
            s_addr = src.ctypes.data + cursor + so
            d_addr = dst.ctypes.data + cursor + do
            table += [d_addr, s_addr, size]
            expect[cursor + do: cursor + do + size] = src[cursor + so: cursor + so + size]
            cursor += 8192
        O.emulate_batch_copy_kernel(np.array(table, dtype=np.uint64), grid, block)
        assert np.array_equal(dst, expect), (grid, block)


def test_reference_kernel_test_vector_through_both_executors():
    """kernel_matches_direct_both_directions (transfer/kernel.rs:203-267):
    257 fragments of 4112 bytes, pattern (i*31+7)&0xFF, both directions."""
    n, seg = 257, 4112
    total = n * seg
    pattern = kernel_test_pattern(total)
    for backend in ("kernel", "direct"):
        host = pattern.copy()
        dev = np.zeros(total, dtype=np.uint8)
        rows = [(dev.ctypes.data + k * seg, host.ctypes.data + k * seg,
                 host.ctypes.data + k * seg, seg, 0, 0) for k in range(n)]
        if backend == "direct":
            assert O.merge(rows) == [(dev.ctypes.data, host.ctypes.data, total)]
        O.exec_descs(rows, host_is_src=True, backend=backend)
        assert np.array_equal(dev, pattern)
        host[:] = 0
        O.exec_descs(rows, host_is_src=False, backend=backend)
        assert np.array_equal(host, pattern)


@pytest.mark.parametrize("threads", [1, 4])
def test_layer_transfer_equals_numpy_gather_split(threads):
    rng = np.random.default_rng(11)
    num_blocks, seg = 64, 4096
    cache = random_bytes(rng, 2 * num_blocks * seg)
    layout = O.layout_over(cache, num_blocks, seg, num_blocks * seg, 2)
    assert layout.is_split
    ids = rng.choice(num_blocks, 20, replace=False).astype(np.uint32)
    host_k = np.zeros(20 * seg, dtype=np.uint8)
    host_v = np.zeros(20 * seg, dtype=np.uint8)
    O.transfer_layer(layout, ids, host_k, host_v, host_is_src=False, threads=threads)
    ek, ev = O.np_save_split(cache, num_blocks, seg, ids)
    assert np.array_equal(host_k.reshape(20, seg), ek)
    assert np.array_equal(host_v.reshape(20, seg), ev)
    # load into a fresh cache at other slots
    dest_ids = rng.choice(num_blocks, 20, replace=False).astype(np.uint32)
    cache2 = np.full_like(cache, 0xEE)
    layout2 = O.layout_over(cache2, num_blocks, seg, num_blocks * seg, 2)
    O.transfer_layer(layout2, dest_ids, host_k, host_v, host_is_src=True, backend="direct",
                     threads=threads)
    expect = np.full_like(cache, 0xEE)
    O.np_load_split(expect, num_blocks, seg, dest_ids, host_k, host_v)
    assert np.array_equal(cache2, expect)


def test_layer_transfer_equals_numpy_gather_contiguous_and_paged():
    rng = np.random.default_rng(12)
    num_blocks, block = 32, 2304  # MLA-like, not a power of two
    cache = random_bytes(rng, num_blocks * block)
    layout = O.layout_over(cache, num_blocks, block, 0, 1)
    ids = rng.choice(num_blocks, 9, replace=False).astype(np.uint32)
    host = np.zeros(9 * block, dtype=np.uint8)
    O.transfer_layer(layout, ids, host, None, host_is_src=False)
    assert np.array_equal(host.reshape(9, block), O.np_save_contiguous(cache, num_blocks, block, ids))
    # paged: each block has its own page, layer at offset 512 inside it
    page_size = 512 + block + 256
    pages_mem = np.full(9 * page_size, 0xAB, dtype=np.uint8)
    pages = np.array([pages_mem.ctypes.data + i * page_size for i in range(9)], dtype=np.uint64)
    O.transfer_layer_paged(layout, ids, pages, 512, host_is_src=False)
    pm = pages_mem.reshape(9, page_size)
    assert np.array_equal(pm[:, 512:512 + block], O.np_save_contiguous(cache, num_blocks, block, ids))
    assert (pm[:, :512] == 0xAB).all() and (pm[:, 512 + block:] == 0xAB).all()


def test_build_copy_descs_order_and_single_segment_host_block():
    """K then V per block, layer-major; a split device layout over a
    single-segment host block puts V right after K (gpu_worker.rs:373-398)."""
    L = O.Layout(0x1000, 200 * 1024, 100, 1024, 100 * 1024, 2)
    layer = O.LayerBlocks(layout=L, block_idx=np.array([3, 7]),
                          seg0_host=np.array([0x9000, 0xA000]), seg0_dev=np.array([0x19000, 0x1A000]),
                          seg0_alloc=np.array([5, 5]))
    descs, total = O.build_copy_descs([layer])
    assert total == 4 * 1024
    assert descs == [
        (0x1000 + 3 * 1024, 0x9000, 0x19000, 1024, 0, 5),
        (0x1000 + 103 * 1024, 0x9000 + 1024, 0x19000 + 1024, 1024, 0, 5),
        (0x1000 + 7 * 1024, 0xA000, 0x1A000, 1024, 0, 5),
        (0x1000 + 107 * 1024, 0xA000 + 1024, 0x1A000 + 1024, 1024, 0, 5),
    ]
    # two-segment host block + page offset; second layer gets device_allocation 1
    layer2 = O.LayerBlocks(layout=L, block_idx=np.array([1]),
                           seg0_host=np.array([0x9000]), seg0_dev=np.array([0x19000]),
                           seg0_alloc=np.array([5]), seg1_host=np.array([0xB000]),
                           seg1_dev=np.array([0x1B000]), seg1_alloc=np.array([6]),
                           host_offset=np.array([256]))
    descs, total = O.build_copy_descs([layer, layer2])
    assert descs[4:] == [
        (0x1000 + 1024, 0x9000 + 256, 0x19000 + 256, 1024, 1, 5),
        (0x1000 + 101 * 1024, 0xB000 + 256, 0x1B000 + 256, 1024, 1, 6),
    ]
    bad = O.LayerBlocks(layout=L, block_idx=np.array([100]), seg0_host=np.array([1]),
                        seg0_dev=np.array([1]), seg0_alloc=np.array([1]))
    with pytest.raises(O.OracleError, match=r"block 100 out of range \(100 blocks\)"):
        O.build_copy_descs([bad])
