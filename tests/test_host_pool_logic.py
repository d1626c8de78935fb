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


# ---------------------------------------------------------------------------
# The remaining cases of pegaflow-core/src/instance/tests.rs, one test each,
# with the reference's inputs and assertions (the reference needs two CUDA
# devices for several of them; sealing itself touches no device).
# ---------------------------------------------------------------------------

def _workers(*specs):
    """specs: (device_id, tp_rank, pp_rank, [layer names] or [(name, group)], segment_bytes)."""
    out = []
    for device_id, tp_rank, pp_rank, layers, seg in specs:
        names = [l if isinstance(l, str) else l[0] for l in layers]
        groups = {l[0]: l[1] for l in layers if not isinstance(l, str)} or None
        out.append(WorkerLayers(device_id, tp_rank, {n: _layout(i, seg) for i, n in enumerate(names)},
                                pp_rank=pp_rank, groups=groups))
    return out


def test_seal_derives_layer_space_from_union_of_workers():
    """instance/tests.rs:311-343: pipeline stages register disjoint layers
    (stage 1 also a speculative MTP layer); ids span the union."""
    topo = LayerTopology(_workers(
        (0, 0, 0, ["model.layers.0.self_attn.attn"], 1024),
        (1, 0, 1, ["model.layers.1.self_attn.attn", "model.layers.2.self_attn.attn"], 1024)),
        tp_size=1)
    assert topo.num_layers == 3
    assert topo.layer_id("model.layers.2.self_attn.attn") == 2
    topo.close()


def test_mla_replica_registration_seals():
    """instance/tests.rs:360-378: MLA replicas collapse to tp_rank 0; several
    owners per slot are valid."""
    layers = ["model.layers.0.self_attn.attn", "model.layers.0.self_attn.indexer.k_cache",
              "model.layers.1.self_attn.attn", "model.layers.1.self_attn.indexer.k_cache"]
    topo = LayerTopology(_workers((0, 0, 0, layers, 1024), (1, 0, 0, layers, 1024)), tp_size=1)
    assert topo.num_layers == 4 and topo.total_slots == 4
    topo.close()


def test_seal_rejects_replicas_across_pipeline_stages():
    """instance/tests.rs:385-409."""
    layers = ["model.layers.0.self_attn.attn"]
    with pytest.raises(_lib.InvalidArgument, match="different pipeline stages"):
        LayerTopology(_workers((0, 0, 0, layers, 1024), (1, 0, 1, layers, 1024)), tp_size=1)


def test_seal_rejects_missing_slot_owner():
    """instance/tests.rs:415-437: every rank must register every layer; the
    complete worker set then seals."""
    with pytest.raises(_lib.InvalidArgument, match="incomplete KV registration") as exc:
        LayerTopology(_workers((0, 0, 0, ["layer_0", "layer_1"], 1024), (1, 1, 0, ["layer_0"], 1024)),
                      tp_size=2)
    assert "layer_1" in str(exc.value)
    topo = LayerTopology(_workers((0, 0, 0, ["layer_0", "layer_1"], 1024),
                                  (1, 1, 0, ["layer_0", "layer_1"], 1024)), tp_size=2)
    assert topo.total_slots == 4
    topo.close()


def test_seal_rejects_inconsistent_layer_geometry():
    """instance/tests.rs:443-468."""
    with pytest.raises(_lib.InvalidArgument, match="inconsistent geometry"):
        LayerTopology(_workers((0, 0, 0, ["layer_0"], 1024), (1, 0, 0, ["layer_0"], 2048)), tp_size=1)


def test_hybrid_topology_seals_per_group_slot_spaces():
    """instance/tests.rs:476-512."""
    topo = LayerTopology(_workers(
        (0, 0, 0, [("attn_a", 0), ("attn_b", 0), ("recurrent_c", 1), ("recurrent_d", 1)], 1024)))
    assert topo.num_layers == 4 and topo.num_groups == 2
    assert [topo.group_of_layer(i) for i in range(4)] == [0, 0, 1, 1]
    assert topo.group_total_slots(0) == 2 and topo.group_total_slots(1) == 2
    assert topo.total_slots == 4
    assert [topo.slot_index(i, 0) for i in range(4)] == [0, 1, 0, 1]
    topo.close()


def test_default_groups_keep_global_slot_layout():
    """instance/tests.rs:520-535."""
    topo = LayerTopology(_workers((0, 0, 0, ["layer_a", "layer_b", "layer_c"], 1024)))
    assert topo.num_groups == 1 and topo.group_total_slots(0) == 3
    for layer_id in range(3):
        assert topo.group_of_layer(layer_id) == 0
        assert topo.slot_index(layer_id, 0) == layer_id
    with pytest.raises(_lib.InvalidArgument):
        topo.group_total_slots(1)
    topo.close()


def test_seal_rejects_inconsistent_layer_group_across_devices():
    """instance/tests.rs:541-560."""
    with pytest.raises(_lib.InvalidArgument, match="storage group"):
        LayerTopology(_workers((0, 0, 0, [("layer_0", 0)], 1024), (1, 0, 0, [("layer_0", 1)], 1024)),
                      tp_size=1)


def test_seal_rejects_sparse_group_ids():
    """instance/tests.rs:565-576."""
    with pytest.raises(_lib.InvalidArgument, match="dense"):
        LayerTopology(_workers((0, 0, 0, [("layer_a", 0), ("layer_b", 2)], 1024)))


def test_page_first_rejects_multiple_groups():
    """instance/tests.rs:581-592."""
    with pytest.raises(_lib.InvalidArgument, match="page-first"):
        LayerTopology(_workers((0, 0, 0, [("layer_a", 0), ("layer_b", 1)], 1024)), page_first=True)


def test_registration_without_layers_is_rejected():
    """instance/tests.rs:291-300."""
    with pytest.raises(_lib.InvalidArgument, match="no KV cache layers"):
        LayerTopology([WorkerLayers(0, 0, {})])


def test_query_pages_numa():
    """numa.rs:606-636: no addresses -> nothing; touched heap pages sit on a
    valid node."""
    import ctypes as C
    lib = _lib.load()
    assert lib.pf_numa_query_pages(None, 0, None) == 0
    buf = np.zeros(8192 + 4096, dtype=np.uint8)
    base = (buf.ctypes.data + 4095) & ~4095
    buf[:] = 1
    addrs = (C.c_void_p * 2)(base, base + 4096)
    nodes = (C.c_int * 2)(-7, -7)
    _lib.check(lib.pf_numa_query_pages(addrs, 2, nodes))
    assert all(0 <= n < max(lib.pf_numa_node_count(), 1) for n in nodes), list(nodes)
