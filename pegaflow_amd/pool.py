"""Pinned pool, offset allocator, NUMA helpers and layer topology over the C
ABI.  Mirrors pegaflow-core/src/{allocator.rs,pinned_pool.rs,instance.rs} and
pegaflow-common/src/numa.rs of the reference for the transfer path."""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Sequence

import numpy as np

from . import _lib
from ._lib import check
from .layout import KVCacheLayout


@dataclass
class Region:
    offset_bytes: int
    size_bytes: int
    _raw: object = None


class ScaledOffsetAllocator:
    """Byte-unit wrapper over a u32 offset allocator (allocator.rs:63-142)."""

    def __init__(self, total_bytes: int, unit_size: int, max_allocs: int):
        self._lib = _lib.load()
        h = C.c_void_p()
        check(self._lib.pf_allocator_create(total_bytes, unit_size, max_allocs, C.byref(h)))
        self.handle = h

    def allocate(self, size_bytes: int) -> Region | None:
        r = _lib.PfAllocRegion()
        check(self._lib.pf_allocator_allocate(self.handle, size_bytes, C.byref(r)))
        if r.size_bytes == 0:
            return None
        return Region(r.offset_bytes, r.size_bytes, r)

    def free(self, region: Region) -> None:
        check(self._lib.pf_allocator_free(self.handle, C.byref(region._raw)))

    def report(self) -> dict:
        total, free, largest, units = C.c_uint64(), C.c_uint64(), C.c_uint64(), C.c_uint64()
        check(self._lib.pf_allocator_report(self.handle, C.byref(total), C.byref(free),
                                            C.byref(largest), C.byref(units)))
        return {"total_bytes": total.value, "total_free_bytes": free.value,
                "largest_free_allocation_bytes": largest.value, "total_units": units.value}

    def close(self) -> None:
        if self.handle is not None:
            self._lib.pf_allocator_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def compute_unit_size(pool_size: int, hint: int = 0) -> int:
    return _lib.load().pf_pool_compute_unit_size(pool_size, hint)


class PinnedAllocation:
    """RAII handle of one pool allocation: host pointer, device-visible
    pointer, reserved size (pinned_pool.rs:56-117)."""

    def __init__(self, raw):
        self._raw = raw

    @property
    def host_ptr(self) -> int:
        return self._raw.host or 0

    @property
    def device_ptr(self) -> int:
        return self._raw.device

    @property
    def size(self) -> int:
        return self._raw.size

    @property
    def allocation_id(self) -> int:
        return self._raw.handle

    def as_numpy(self) -> np.ndarray:
        buf = (C.c_uint8 * self.size).from_address(self.host_ptr)
        return np.frombuffer(buf, dtype=np.uint8)

    def free(self) -> None:
        if self._raw.handle:
            check(_lib.load().pf_pool_free(C.byref(self._raw)))

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class PinnedAllocator:
    """Global or NUMA-aware sharded pinned pool (pinned_pool.rs:599-715)."""

    def __init__(self, capacity: int, num_shards: int = 1, use_hugepages: bool = False,
                 ssd_enabled: bool = False, unit_size_hint: int = 0,
                 numa_nodes: Sequence[int] | None = None):
        self._lib = _lib.load()
        cfg = _lib.PfPoolConfig()
        cfg.capacity = capacity
        cfg.num_shards = num_shards
        cfg.use_hugepages = 1 if use_hugepages else 0
        cfg.ssd_enabled = 1 if ssd_enabled else 0
        cfg.unit_size_hint = unit_size_hint
        nodes = list(numa_nodes or [])
        self._nodes = (C.c_int32 * max(len(nodes), 1))(*nodes)
        cfg.n_numa_nodes = len(nodes)
        cfg.numa_nodes = self._nodes
        h = C.c_void_p()
        check(self._lib.pf_pool_create(C.byref(cfg), C.byref(h)))
        self.handle = h

    def allocate(self, size: int, numa_node: int = -1) -> PinnedAllocation | None:
        raw = _lib.PfAllocation()
        check(self._lib.pf_pool_allocate(self.handle, size, numa_node, C.byref(raw)))
        return PinnedAllocation(raw) if raw.handle else None

    def usage(self) -> tuple[int, int]:
        used, total = C.c_uint64(), C.c_uint64()
        check(self._lib.pf_pool_usage(self.handle, C.byref(used), C.byref(total)))
        return used.value, total.value

    def largest_free_allocation_for_node(self, numa_node: int = -1) -> int:
        out = C.c_uint64()
        check(self._lib.pf_pool_largest_free(self.handle, numa_node, C.byref(out)))
        return out.value

    @property
    def is_numa(self) -> bool:
        return bool(self._lib.pf_pool_is_numa(self.handle))

    def close(self) -> None:
        if self.handle is not None:
            self._lib.pf_pool_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def format_cpu_list(cpus: Sequence[int]) -> str:
    arr = (C.c_uint64 * max(len(cpus), 1))(*cpus)
    buf = C.create_string_buffer(4096)
    check(_lib.load().pf_numa_format_cpu_list(arr, len(cpus), buf, 4096))
    return buf.value.decode()


def parse_cpulist(text: str) -> list[int]:
    out = (C.c_uint64 * 4096)()
    n = C.c_uint64()
    check(_lib.load().pf_numa_parse_cpulist(text.encode(), out, 4096, C.byref(n)))
    return [out[i] for i in range(n.value)]


def numa_node_display(node: int) -> str:
    """Display form of a NUMA node id (numa.rs:36-45)."""
    return "UNKNOWN" if node < 0 else f"NUMA{node}"


def build_page_layout(worker_layer_sets, n_layers: int, padded_bytes) -> dict:
    """Shards and per-shard byte offsets of page-first storage (instance.rs:107-162)."""
    flat, off = [], [0]
    for s in worker_layer_sets:
        flat.extend(int(x) for x in s)
        off.append(len(flat))
    u64 = C.c_uint64
    flat_a = (u64 * max(len(flat), 1))(*flat)
    off_a = (u64 * len(off))(*off)
    pad_a = (u64 * max(n_layers, 1))(*[int(x) for x in padded_bytes])
    shard = (u64 * max(n_layers, 1))()
    offsets = (u64 * max(n_layers, 1))()
    nbytes = (u64 * max(n_layers, 1))()
    sizes = (u64 * max(len(worker_layer_sets), 1))()
    n_shards = u64()
    check(_lib.load().pf_build_page_layout(flat_a, off_a, len(worker_layer_sets), n_layers, pad_a,
                                           shard, offsets, nbytes, sizes, C.byref(n_shards)))
    return {"layer_shard": list(shard[:n_layers]), "layer_offsets": list(offsets[:n_layers]),
            "layer_bytes": list(nbytes[:n_layers]),
            "shard_page_sizes": list(sizes[: n_shards.value])}


@dataclass
class WorkerLayers:
    """What one worker registered: its layers and their layouts."""
    device_id: int
    tp_rank: int
    layers: dict  # name -> KVCacheLayout
    pp_rank: int = 0
    groups: dict | None = None  # name -> storage group


class LayerTopology:
    """Sealed layer-id space of an instance (instance.rs:46-269,488-672)."""

    def __init__(self, workers: Sequence[WorkerLayers], tp_size: int = 1, page_first: bool = False):
        self._lib = _lib.load()
        arr = (_lib.PfWorkerLayers * len(workers))()
        keep = []
        for i, w in enumerate(workers):
            names = list(w.layers)
            n = len(names)
            c_names = (C.c_char_p * max(n, 1))(*[s.encode() for s in names])
            c_layouts = (_lib.PfKvLayout * max(n, 1))(*[w.layers[s].c for s in names])
            keep += [c_names, c_layouts]
            arr[i].device_id = w.device_id
            arr[i].tp_rank = w.tp_rank
            arr[i].pp_rank = w.pp_rank
            arr[i].n_layers = n
            arr[i].layer_names = c_names
            arr[i].layouts = c_layouts
            if w.groups is not None:
                c_groups = (C.c_uint32 * max(n, 1))(*[w.groups.get(s, 0) for s in names])
                keep.append(c_groups)
                arr[i].group_ids = c_groups
        h = C.c_void_p()
        check(self._lib.pf_topology_seal(arr, len(workers), tp_size, 1 if page_first else 0,
                                         C.byref(h)))
        self.handle = h

    @property
    def num_layers(self) -> int:
        return self._lib.pf_topology_num_layers(self.handle)

    @property
    def total_slots(self) -> int:
        return self._lib.pf_topology_total_slots(self.handle)

    @property
    def is_page_first(self) -> bool:
        return bool(self._lib.pf_topology_is_page_first(self.handle))

    @property
    def num_groups(self) -> int:
        return self._lib.pf_topology_num_groups(self.handle)

    def group_of_layer(self, layer_id: int) -> int:
        out = C.c_uint32()
        check(self._lib.pf_topology_group_of_layer(self.handle, layer_id, C.byref(out)))
        return out.value

    def group_total_slots(self, group: int) -> int:
        out = C.c_uint64()
        check(self._lib.pf_topology_group_total_slots(self.handle, group, C.byref(out)))
        return out.value

    def layer_id(self, name: str) -> int:
        out = C.c_uint64()
        check(self._lib.pf_topology_layer_id(self.handle, name.encode(), C.byref(out)))
        return out.value

    def slot_index(self, layer_id: int, tp_rank: int) -> int:
        out = C.c_uint64()
        check(self._lib.pf_topology_slot_index(self.handle, layer_id, tp_rank, C.byref(out)))
        return out.value

    def page_placement(self, layer_id: int) -> tuple[int, int]:
        off, nbytes = C.c_uint64(), C.c_uint64()
        check(self._lib.pf_topology_page_placement(self.handle, layer_id, C.byref(off),
                                                   C.byref(nbytes)))
        return off.value, nbytes.value

    def shard_page_size(self, shard: int) -> int:
        out = C.c_uint64()
        check(self._lib.pf_topology_shard_page_size(self.handle, shard, C.byref(out)))
        return out.value

    def shard_layer_count(self, shard: int) -> int:
        out = C.c_uint64()
        check(self._lib.pf_topology_shard_layer_count(self.handle, shard, C.byref(out)))
        return out.value

    def close(self) -> None:
        if self.handle is not None:
            self._lib.pf_topology_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
