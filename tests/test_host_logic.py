"""Host-side logic of libpegahip through the C ABI (no GPU needed): layout
validation and addressing, the merge rule, descriptor construction.  Checked
against the reference's known-answer vectors and, on random cases, against
the CPU oracle."""

import ctypes as C

import numpy as np
import pytest

from oracle import oracle as O
from pegaflow_amd import _lib
from pegaflow_amd.layout import KVCacheLayout
from pegaflow_amd.transfer import (CopyDesc, HostBlock, LayerTransferData, TransferMode,
                                   build_copy_descs, merge)


def _build(case):
    L = KVCacheLayout(*case["new"])
    if "with_block_stride" in case:
        L.with_block_stride(case["with_block_stride"])
    if "with_ssd_padding" in case:
        L.with_ssd_padding(case["with_ssd_padding"])
    return L


def test_layout_kats(kats):
    for case in kats["layout"]:
        exp = case["expect"]
        if "error_contains" in exp:
            with pytest.raises(_lib.InvalidArgument, match=exp["error_contains"]):
                KVCacheLayout(*case["new"])
            continue
        if "stride_error_contains" in exp:
            L = KVCacheLayout(*case["new"])
            with pytest.raises(_lib.InvalidArgument, match=exp["stride_error_contains"]):
                L.with_block_stride(case["with_block_stride"])
            continue
        L = _build(case)
        if "is_split" in exp:
            assert L.is_split == exp["is_split"], case["name"]
        for key in ("padded_segment_bytes", "padded_block_bytes"):
            if key in exp:
                assert getattr(L, key) == exp[key], case["name"]
        for idx, copies in exp.get("copies", {}).items():
            got = [[c.addr, c.bytes] for c in L.block_copies(int(idx))]
            assert got == copies, case["name"]
        for idx in exp.get("out_of_range", []):
            with pytest.raises(_lib.InvalidArgument, match="out of range"):
                L.block_copies(idx)


def test_layout_error_messages_match_oracle_on_random_shapes():
    """Same accept/reject decision, same message, same addresses as the oracle
    for a few thousand random (mostly borderline) shapes."""
    rng = np.random.default_rng(2024)
    checked_ok = checked_err = 0
    for _ in range(4000):
        seg = int(rng.choice([1, 16, 100, 512, 1024, 4112]))
        nblk = int(rng.integers(1, 40))
        segments = int(rng.choice([1, 2, 2, 2, 3]))
        kv = int(rng.choice([0, seg // 2, seg, seg + 1, seg * nblk, seg * nblk + 7, seg * 3,
                             int(rng.integers(0, seg * nblk * 2 + 1))]))
        size = int(rng.choice([seg * nblk * segments, seg * nblk * segments - 1,
                               kv + seg * nblk, kv + seg * nblk - 1, 1 << 30, 1 << 30, 1 << 30, 0]))
        ptr = int(rng.choice([0, 0x1000, 0x1000, 0x1000, 0x7F00_0000_0000, 2**64 - 4096]))
        stride = int(rng.choice([0, seg, seg * 2, seg * segments, seg * segments - 1,
                                 int(rng.integers(1, seg * 4 + 1))]))
        args = (ptr, size, nblk, seg, kv, segments)
        try:
            ref = O.Layout(*args)
            if stride:
                ref.with_block_stride(stride)
            ref_err = None
        except O.OracleError as e:
            ref, ref_err = None, str(e)
        try:
            got = KVCacheLayout(*args)
            if stride:
                got.with_block_stride(stride)
            got_err = None
        except _lib.InvalidArgument as e:
            got, got_err = None, e.message
        assert got_err == ref_err, (args, stride)
        if ref is None:
            checked_err += 1
            continue
        checked_ok += 1
        assert got.is_split == ref.is_split
        assert got.block_stride_bytes == ref.c.block_stride_bytes
        for idx in {0, nblk - 1, int(rng.integers(0, nblk))}:
            assert [(c.addr, c.bytes) for c in got.block_copies(idx)] == ref.block_copies(idx)
        with pytest.raises(_lib.InvalidArgument):
            got.block_copies(nblk)
    assert checked_ok > 200 and checked_err > 200


def test_hand_filled_layout_struct_is_revalidated():
    L = KVCacheLayout(0x1000, 200 * 1024, 100, 1024, 100 * 1024, 2)
    c = _lib.PfKvLayout.from_buffer_copy(L.c)
    c.block_stride_bytes = 2048  # would make K/V regions collide 50 blocks apart
    out = (_lib.PfBlockCopy * 2)()
    n = C.c_uint32()
    rc = _lib.load().pf_layout_block_copies(C.byref(c), 0, out, C.byref(n))
    assert rc == _lib.PF_ERR_INVALID_ARGUMENT
    assert b"overlaps blocks 50 apart" in _lib.load().pf_last_error()


def test_merge_kats(kats):
    base = 0x7000_0000
    for case in kats["merge"]:
        copies = [CopyDesc(d, base + h, 0, s, da, ha) for d, h, s, da, ha in case["descs"]]
        assert [r[2] for r in merge(copies)] == case["expect_sizes"], case["name"]


def test_merge_matches_oracle_on_random_batches():
    rng = np.random.default_rng(5)
    for _ in range(200):
        n = int(rng.integers(0, 40))
        rows = []
        dev, host = 0x10000, 0x900000
        for _ in range(n):
            size = int(rng.choice([4, 16, 4096]))
            if rng.random() < 0.3:
                dev += int(rng.choice([0, 16, 4096]))
            if rng.random() < 0.3:
                host += int(rng.choice([0, 16, 4096]))
            rows.append((dev, host, host, size, int(rng.integers(0, 2)), int(rng.integers(0, 2))))
            dev += size
            host += size
        got = merge([CopyDesc(*r) for r in rows])
        assert got == O.merge(rows)


def _rand_layer(rng, layer_index, split):
    seg = int(rng.choice([512, 1024, 4112]))
    nblk = int(rng.integers(2, 50))
    if split:
        layout_args = (0x100000 * (layer_index + 1), 2 * nblk * seg, nblk, seg, nblk * seg, 2)
    else:
        layout_args = (0x100000 * (layer_index + 1), nblk * seg, nblk, seg, 0, 1)
    n = int(rng.integers(0, 12))
    ids = rng.integers(0, nblk, size=n)
    two_seg = split and rng.random() < 0.5
    page = rng.random() < 0.3
    host0 = 0x7F0000000000 + rng.integers(0, 1 << 20, size=n) * 16
    host1 = 0x7F1000000000 + rng.integers(0, 1 << 20, size=n) * 16
    offs = rng.integers(0, 8, size=n) * 512 if page else np.zeros(n, dtype=np.int64)
    alloc0 = rng.integers(1, 4, size=n)
    alloc1 = rng.integers(4, 8, size=n)
    return layout_args, ids, two_seg, host0, host1, offs, alloc0, alloc1


def test_build_copy_descs_matches_oracle():
    rng = np.random.default_rng(99)
    for trial in range(60):
        n_layers = int(rng.integers(1, 5))
        prod_layers, orc_layers = [], []
        for li in range(n_layers):
            args, ids, two_seg, h0, h1, offs, a0, a1 = _rand_layer(rng, li, split=bool(li % 2))
            blocks = []
            for j in range(len(ids)):
                if two_seg:
                    blocks.append(HostBlock((int(h0[j]), int(h1[j])),
                                            (int(h0[j]) + 0x1000, int(h1[j]) + 0x1000),
                                            (int(a0[j]), int(a1[j])), host_offset=int(offs[j])))
                else:
                    blocks.append(HostBlock((int(h0[j]),), (int(h0[j]) + 0x1000,), (int(a0[j]),),
                                            host_offset=int(offs[j])))
            prod_layers.append(LayerTransferData(f"layer_{li}", KVCacheLayout(*args), ids, blocks))
            orc_layers.append(O.LayerBlocks(
                layout=O.Layout(*args), block_idx=ids, seg0_host=h0, seg0_dev=h0 + 0x1000,
                seg0_alloc=a0, seg1_host=h1 if two_seg else None,
                seg1_dev=h1 + 0x1000 if two_seg else None, seg1_alloc=a1 if two_seg else None,
                host_offset=offs))
        got, got_total = build_copy_descs(prod_layers)
        ref, ref_total = O.build_copy_descs(orc_layers)
        assert got_total == ref_total
        assert [(d.device, d.host, d.host_device, d.size, d.device_allocation, d.host_allocation)
                for d in got] == ref


def test_build_copy_descs_errors():
    L = KVCacheLayout(0x1000, 1024 * 1024, 100, 1024, 0, 1)
    layer = LayerTransferData("model.layers.0", L, [100], [HostBlock((0x9000,), (0x9000,), (1,))])
    # gpu_worker.rs:363-366: EngineError::Storage("layer {name}: block ... out of range ...")
    with pytest.raises(_lib.StorageError, match=r"layer model.layers.0: block 100 out of range \(100 blocks\)"):
        build_copy_descs([layer])
    assert build_copy_descs([]) == ([], 0)


def test_transfer_mode_names():
    assert TransferMode.from_name("direct") == TransferMode.DIRECT
    assert TransferMode.from_name(" Kernel ") == TransferMode.KERNEL
    with pytest.raises(_lib.InvalidArgument, match="expected one of: direct, kernel"):
        TransferMode.from_name("nccl")
