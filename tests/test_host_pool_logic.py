"""Allocator, NUMA helpers, page layout and layer topology through the C ABI
(no GPU needed), against the reference's known-answer vectors."""

import numpy as np
import pytest

from oracle import oracle as O
from pegaflow_amd import _lib
from pegaflow_amd.layout import KVCacheLayout
from pegaflow_amd.pool import (LayerTopology, ScaledOffsetAllocator, WorkerLayers,
                               build_page_layout, compute_unit_size, format_cpu_list,
                               numa_node_display, parse_cpulist)


def test_allocator_kats(kats):
    for case in kats["allocator"]:
        exp = case.get("expect", {})
        if "create_error_contains" in exp:
            with pytest.raises(_lib.InvalidArgument, match=exp["create_error_contains"]):
                ScaledOffsetAllocator(case["total_bytes"], case["unit"], case["max_allocs"])
            continue
        a = ScaledOffsetAllocator(case["total_bytes"], case["unit"], case["max_allocs"])
        rep = a.report()
        if "total_units" in exp:
            assert rep["total_units"] == exp["total_units"], case["name"]
        if "total_bytes" in exp:
            assert rep["total_bytes"] == exp["total_bytes"], case["name"]
        named = {}
        for op in case.get("ops", []):
            if op[0] == "alloc":
                got = a.allocate(op[1])
                want = op[2]
                if want is None:
                    assert got is None, case["name"]
                    continue
                assert got is not None, case["name"]
                if "offset" in want:
                    assert (got.offset_bytes, got.size_bytes) == (want["offset"], want["size"]), case["name"]
                if "name" in want:
                    named[want["name"]] = got
            elif op[0] == "free":
                a.free(named[op[1]])
            elif op[0] == "report":
                rep = a.report()
                assert rep["total_free_bytes"] == op[1]["free"], case["name"]
                assert rep["largest_free_allocation_bytes"] == op[1]["largest"], case["name"]
            elif op[0] == "alloc_error":
                with pytest.raises(_lib.InvalidArgument, match=op[2]):
                    a.allocate(op[1])
        a.close()


def test_allocator_invariants_under_random_alloc_free():
    """What the mathematics fixes regardless of bin policy: regions lie inside
    the capacity, are unit-aligned, never overlap while live, sizes are the
    request rounded up to the unit, free space accounting is exact, and after
    freeing everything one allocation of the whole capacity succeeds at 0."""
    rng = np.random.default_rng(17)
    unit, units = 512, 4096
    a = ScaledOffsetAllocator(unit * units + 100, unit, 1 << 16)
    assert a.report()["total_bytes"] == unit * units
    live = {}
    used = 0
    for step in range(6000):
        if live and (rng.random() < 0.45 or used > unit * units * 0.8):
            key = list(live)[int(rng.integers(len(live)))]
            r = live.pop(key)
            a.free(r)
            used -= r.size_bytes
        else:
            want = int(rng.choice([1, 511, 512, 513, 4096, 32768, 100000]))
            r = a.allocate(want)
            if r is None:
                continue
            assert r.size_bytes == -(-want // unit) * unit
            assert r.offset_bytes % unit == 0 and r.offset_bytes + r.size_bytes <= unit * units
            for o in live.values():
                assert r.offset_bytes + r.size_bytes <= o.offset_bytes or \
                    o.offset_bytes + o.size_bytes <= r.offset_bytes
            live[step] = r
            used += r.size_bytes
        rep = a.report()
        assert rep["total_free_bytes"] == unit * units - used
        assert rep["largest_free_allocation_bytes"] <= rep["total_free_bytes"]
    for r in live.values():
        a.free(r)
    whole = a.allocate(unit * units)
    assert whole is not None and whole.offset_bytes == 0 and whole.size_bytes == unit * units
    assert a.allocate(1) is None
    a.close()


def test_allocator_same_size_allocations_are_consecutive():
    a = ScaledOffsetAllocator(1 << 30, 512, 4_000_000)
    offs = [a.allocate(65536).offset_bytes for _ in range(1000)]
    assert offs == [i * 65536 for i in range(1000)]
    a.close()


def test_compute_unit_size():
    # pinned_pool.rs:135-141: max(hint or 512, ceil(pool / u32::MAX)) rounded up to 512
    assert compute_unit_size(30 << 30, 0) == 512
    assert compute_unit_size(30 << 30, 1) == 512
    assert compute_unit_size(30 << 30, 4096) == 4096
    assert compute_unit_size(30 << 30, 4097) == 4608
    assert compute_unit_size(4 << 40, 0) == 1536  # ceil(4 TiB / (2^32-1)) = 1025 -> 1536
    assert compute_unit_size((2**32 - 1) * 512, 0) == 512
    assert compute_unit_size((2**32 - 1) * 512 + 1, 0) == 1024


def test_numa_kats(kats):
    n = kats["numa"]
    for cpus, text in n["format_cpu_list"]:
        assert format_cpu_list(cpus) == text
    for text, cpus in n["parse_cpulist"]:
        assert parse_cpulist(text) == cpus
    ht = n["parse_cpulist_hyperthreading"]
    cpus = parse_cpulist(ht["input"])
    assert (len(cpus), cpus[0], cpus[15], cpus[16], cpus[-1]) == \
        (ht["len"], ht["first"], ht["at15"], ht["at16"], ht["last"])
    for node, text in n["display"]:
        assert numa_node_display(node) == text
    with pytest.raises(_lib.InvalidArgument, match="Invalid CPU"):
        parse_cpulist("0-x")
    with pytest.raises(_lib.InvalidArgument, match="unknown"):
        _lib.check(_lib.load().pf_numa_pin_thread(-1))
    assert _lib.load().pf_numa_node_count() >= 1


def test_gpu_numa_lookup_reads_pci_sysfs(tmp_path):
    dev = tmp_path / "0000:c1:00.0"
    dev.mkdir()
    (dev / "numa_node").write_text("3\n")
    unknown = tmp_path / "0000:c2:00.0"
    unknown.mkdir()
    (unknown / "numa_node").write_text("-1\n")
    lib = _lib.load()
    assert lib.pf_numa_node_of_pci(b"0000:C1:00.0", str(tmp_path).encode()) == 3
    assert lib.pf_numa_node_of_pci(b"0000:c2:00.0", str(tmp_path).encode()) == -1
    assert lib.pf_numa_node_of_pci(b"0000:ff:00.0", str(tmp_path).encode()) == -1


def test_page_layout_kats(kats):
    for case in kats["page_layout"]:
        exp = case["expect"]
        if "error_contains" in exp:
            with pytest.raises(_lib.InvalidArgument, match=exp["error_contains"]):
                build_page_layout(case["sets"], case["n_layers"], case["padded"])
            continue
        got = build_page_layout(case["sets"], case["n_layers"], case["padded"])
        for key, val in exp.items():
            assert got[key] == val, (case["name"], key)


def test_page_layout_matches_oracle_on_random_partitions():
    rng = np.random.default_rng(23)
    for _ in range(300):
        n_layers = int(rng.integers(1, 12))
        n_shards = int(rng.integers(1, min(4, n_layers) + 1))
        owner = rng.integers(0, n_shards, size=n_layers)
        sets = [[int(l) for l in range(n_layers) if owner[l] == s] for s in range(n_shards)]
        sets = [s for s in sets if s]
        # replicas and shuffled registration order
        order = list(rng.permutation(len(sets)))
        workers = [sets[i] for i in order] + [sets[int(rng.integers(len(sets)))]]
        padded = [int(x) * 512 for x in rng.integers(1, 9, size=n_layers)]
        assert build_page_layout(workers, n_layers, padded) == \
            O.build_page_layout(workers, n_layers, padded)


def _layout(index, seg=1024):
    return KVCacheLayout(0x1000 + index * 0x10000, 1024 * 1024, 100, seg, 0, 1)


def test_topology_kats(kats):
    for case in kats["topology"]:
        workers = []
        for di, w in enumerate(case["workers"]):
            layers = {name: _layout(i, w["segment_bytes"]) for i, name in enumerate(w["layers"])}
            workers.append(WorkerLayers(device_id=di, tp_rank=w["tp_rank"], layers=layers))
        topo = LayerTopology(workers, tp_size=case["tp_size"], page_first=case["page_first"])
        exp = case["expect"]
        assert topo.num_layers == exp["num_layers"], case["name"]
        assert topo.total_slots == exp["total_slots"], case["name"]
        assert topo.is_page_first == case["page_first"]
        for name, lid in exp.get("layer_id", {}).items():
            assert topo.layer_id(name) == lid
        for name in exp.get("missing", []):
            with pytest.raises(_lib.InvalidArgument, match="is not registered"):
                topo.layer_id(name)
        for lid, tp, slot in exp.get("slot_index", []):
            assert topo.slot_index(lid, tp) == slot, case["name"]
        for shard, size in exp.get("shard_page_size", {}).items():
            assert topo.shard_page_size(int(shard)) == size
        for shard, cnt in exp.get("shard_layer_count", {}).items():
            assert topo.shard_layer_count(int(shard)) == cnt
        for lid, (off, nbytes) in exp.get("page_placement", {}).items():
            assert topo.page_placement(int(lid)) == (off, nbytes)
        topo.close()


def test_layer_ids_are_bytewise_sorted_names():
    """`model.layers.10...` sorts before `model.layers.2...` (instance.rs:544-550):
    the page offsets of an MLA model follow that order, not the numeric one."""
    names = [f"model.layers.{i}.self_attn.attn" for i in range(12)]
    layers = {n: _layout(i, 512 * (i + 1)) for i, n in enumerate(names)}
    topo = LayerTopology([WorkerLayers(0, 0, layers)], tp_size=1, page_first=True)
    ordered = sorted(names)
    assert ordered[:4] == ["model.layers.0.self_attn.attn", "model.layers.1.self_attn.attn",
                           "model.layers.10.self_attn.attn", "model.layers.11.self_attn.attn"]
    off = 0
    for rank, name in enumerate(ordered):
        assert topo.layer_id(name) == rank
        size = 512 * (names.index(name) + 1)
        assert topo.page_placement(rank) == (off, size)
        off += size
    assert topo.shard_page_size(0) == off
    topo.close()


def test_topology_rejections():
    a, b = _layout(0), _layout(1)
    # same name, different geometry across devices
    with pytest.raises(_lib.InvalidArgument, match="inconsistent geometry"):
        LayerTopology([WorkerLayers(0, 0, {"l": a}), WorkerLayers(1, 1, {"l": _layout(0, 2048)})],
                      tp_size=2)
    # missing (layer, tp_rank) owner
    with pytest.raises(_lib.InvalidArgument, match="has no owner for tp_rank 1"):
        LayerTopology([WorkerLayers(0, 0, {"l": a}), WorkerLayers(1, 0, {"l": a})], tp_size=2)
    # two pipeline stages claim one layer
    with pytest.raises(_lib.InvalidArgument, match="different pipeline stages"):
        LayerTopology([WorkerLayers(0, 0, {"l": a}, pp_rank=0),
                       WorkerLayers(1, 0, {"l": a}, pp_rank=1)], tp_size=1)
    # non-dense storage groups
    with pytest.raises(_lib.InvalidArgument, match="must be dense"):
        LayerTopology([WorkerLayers(0, 0, {"x": a, "y": b}, groups={"x": 0, "y": 2})])
    # page-first with two groups
    with pytest.raises(_lib.InvalidArgument, match="multiple storage groups"):
        LayerTopology([WorkerLayers(0, 0, {"x": a, "y": b}, groups={"x": 0, "y": 1})],
                      page_first=True)
    # hybrid groups: slots are dense within a group
    topo = LayerTopology([WorkerLayers(0, 0, {"att0": a, "gdn0": b, "att1": _layout(2)},
                                       groups={"att0": 0, "att1": 0, "gdn0": 1})])
    ids = {n: topo.layer_id(n) for n in ("att0", "att1", "gdn0")}
    assert [topo.slot_index(ids[n], 0) for n in ("att0", "att1", "gdn0")] == [0, 1, 0]
    topo.close()
