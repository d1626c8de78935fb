"""Worker pool, load-completion flag and the save/load-by-block-ID engine over
the C ABI.  Mirrors the reference's GpuWorkerPool
(pegaflow-core/src/gpu_worker.rs:116-243), LoadState (sync_state.rs:113-188)
and the path-relevant surface of PegaEngine (lib.rs:228-440,506-546,654-709,
offload.rs:293-659)."""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Sequence

import numpy as np

from . import _lib
from ._lib import check
from .transfer import LayerTransferData, TransferMode

LOAD_STATE_PENDING = 0
LOAD_STATE_SUCCESS = 1
LOAD_STATE_ERROR = -1


class LoadState:
    """Shared-memory completion flag a submitter polls."""

    def __init__(self, attach_to: str | None = None):
        self._lib = _lib.load()
        h = C.c_void_p()
        if attach_to is None:
            check(self._lib.pf_load_state_create(C.byref(h)))
        else:
            check(self._lib.pf_load_state_attach(attach_to.encode(), C.byref(h)))
        self.handle = h

    @property
    def shm_name(self) -> str:
        return self._lib.pf_load_state_name(self.handle).decode()

    def get(self) -> int:
        return self._lib.pf_load_state_get(self.handle)

    def set_completed(self) -> None:
        check(self._lib.pf_load_state_set(self.handle, LOAD_STATE_SUCCESS))

    def set_error(self) -> None:
        check(self._lib.pf_load_state_set(self.handle, LOAD_STATE_ERROR))

    def close(self) -> None:
        if self.handle is not None:
            self._lib.pf_load_state_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


TASK_PATH_NAMES = ((_lib.PF_TASK_PATH_STAGED, "staged"), (_lib.PF_TASK_PATH_ZEROCOPY, "zerocopy"),
                   (_lib.PF_TASK_PATH_DESCRIPTORS, "descriptors"))


@dataclass
class TaskResult:
    """What a settled task reports: bytes and duration (what the reference's
    workers log per task, gpu_worker.rs:458-474,505-520), which way the bytes
    crossed the link, and the task's phases in milliseconds."""
    done: bool
    bytes: int
    elapsed_ms: float
    paths: tuple = ()              # of "staged", "zerocopy", "descriptors"
    staged_groups: int = 0
    zero_copy_launches: int = 0
    link_copies: int = 0
    phases_ms: dict | None = None  # resolve, queue, convert, plan, staging_alloc, enqueue, sync,
                                   # device_first, device

    @classmethod
    def from_c(cls, r) -> "TaskResult":
        phases = {k[:-3]: getattr(r, k) for k in (
            "resolve_ms", "queue_ms", "convert_ms", "plan_ms", "staging_alloc_ms", "enqueue_ms",
            "sync_ms", "device_first_ms", "device_ms")}
        return cls(bool(r.done), r.bytes, r.elapsed_ms,
                   tuple(name for bit, name in TASK_PATH_NAMES if r.paths & bit),
                   r.staged_groups, r.zero_copy_launches, r.link_copies, phases)


class Task:
    """A submitted load or save; ``wait`` raises if the task failed."""

    def __init__(self, handle, keep=None):
        self._lib = _lib.load()
        self.handle = handle
        self._keep = keep

    def wait(self, timeout_ms: int = -1) -> TaskResult:
        r = _lib.PfTaskResult()
        check(self._lib.pf_task_wait(self.handle, timeout_ms, C.byref(r)))
        return TaskResult.from_c(r)

    def close(self) -> None:
        if self.handle is not None:
            self._lib.pf_task_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _pack_layer_transfers(layers: Sequence[LayerTransferData]):
    n_layers = len(layers)
    arr = (_lib.PfLayerTransfer * max(n_layers, 1))()
    keep = []
    for i, layer in enumerate(layers):
        nb = len(layer.blocks)
        idx = (C.c_uint64 * max(nb, 1))(*[int(b) for b in layer.block_idx])
        blocks = (_lib.PfHostBlock * max(nb, 1))()
        for j, hb in enumerate(layer.blocks):
            ns = len(hb.seg_host)
            blocks[j].num_segments = ns
            for s in range(ns):
                blocks[j].seg_host[s] = hb.seg_host[s]
                blocks[j].seg_device[s] = hb.seg_device[s]
                blocks[j].seg_alloc[s] = hb.seg_alloc[s]
                blocks[j].seg_size[s] = hb.seg_size[s] if s < len(hb.seg_size) else 0
            blocks[j].host_offset = hb.host_offset
        name = layer.layer_name.encode()
        keep.append((idx, blocks, name))
        arr[i].layer_name = name
        arr[i].layout = layer.layout.c
        arr[i].block_idx = idx
        arr[i].blocks = blocks
        arr[i].n_blocks = nb
    return arr, n_layers, keep


class GpuWorkerPool:
    """One load thread and one save thread for a GPU, each with its own
    stream; tasks run serially per thread with one synchronisation each."""

    def __init__(self, device_id: int, numa_node: int = -1, transfer_mode: int = TransferMode.DIRECT,
                 use_descriptor_backends: bool = False, staging_slot_bytes: int = 0,
                 auto_staged_min_bytes: int = 0, lazy_staging: bool = False,
                 side_copy_streams: bool = False):
        """A staging pool (block-ID engine, mode direct or kernel) holds
        2 workers x 2 slots of ``staging_slot_bytes`` (0 = 512 MiB) of device
        memory from here on, unless ``lazy_staging`` leaves the allocation to the
        first staged task of each worker.  ``side_copy_streams``: see PegaEngine."""
        self._lib = _lib.load()
        h = C.c_void_p()
        cfg = _lib.PfWorkerPoolConfig(device_id, numa_node, transfer_mode,
                                      1 if use_descriptor_backends else 0, staging_slot_bytes,
                                      auto_staged_min_bytes, 1 if lazy_staging else 0,
                                      1 if side_copy_streams else 0)
        check(self._lib.pf_worker_pool_spawn_ex(C.byref(cfg), C.byref(h)))
        self.handle = h

    @property
    def staging_bytes(self) -> int:
        """Device memory the two workers hold for staging right now."""
        return self._lib.pf_worker_pool_staging_bytes(self.handle)

    @property
    def queue_clashes(self) -> int:
        """Pairs of worker streams (this pool's two and the idle ones of the
        other pools probed at spawn) that were left sharing a hardware queue."""
        return self._lib.pf_worker_pool_queue_clashes(self.handle)

    def submit_load(self, layers: Sequence[LayerTransferData],
                    load_state: LoadState | None = None) -> Task:
        arr, n, keep = _pack_layer_transfers(layers)
        t = C.c_void_p()
        shm = load_state.shm_name.encode() if load_state is not None else None
        check(self._lib.pf_worker_submit_load(self.handle, arr, n, shm, C.byref(t)))
        return Task(t)

    def batch_save(self, layers: Sequence[LayerTransferData]) -> Task:
        arr, n, keep = _pack_layer_transfers(layers)
        t = C.c_void_p()
        check(self._lib.pf_worker_submit_save(self.handle, arr, n, C.byref(t)))
        return Task(t)

    def close(self) -> None:
        if self.handle is not None:
            self._lib.pf_worker_pool_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def worker_stream_report(device: int = 0) -> tuple[int, int, int]:
    """(worker streams of the live pools on ``device``, pairs among the idle
    ones that share a hardware queue right now, streams skipped because busy)."""
    a, b, c = C.c_uint64(), C.c_uint64(), C.c_uint64()
    check(_lib.load().pf_worker_stream_report(device, C.byref(a), C.byref(b), C.byref(c)))
    return a.value, b.value, c.value


@dataclass
class LayerSave:
    """Per-layer save input: layer name, device block ids, content hashes."""
    layer_name: str
    block_ids: Sequence[int]
    block_hashes: Sequence[bytes]


def _pack_hashes(hashes: Sequence[bytes]):
    """-> (pointer array, length array, backing buffer) for a list of byte strings."""
    n = len(hashes)
    lens_np = np.fromiter((len(h) for h in hashes), dtype=np.uint32, count=n)
    blob = np.frombuffer(b"".join(hashes) + b"\0", dtype=np.uint8)
    starts = np.zeros(max(n, 1), dtype=np.uint64)
    if n > 1:
        np.cumsum(lens_np[:-1], out=starts[1:n])
    addrs = (starts + np.uint64(blob.ctypes.data)).astype(np.uint64)
    ptrs = C.cast(addrs.ctypes.data, C.POINTER(C.POINTER(C.c_uint8)))
    lens_keep = np.ascontiguousarray(lens_np if n else np.zeros(1, dtype=np.uint32))
    lens = C.cast(lens_keep.ctypes.data, C.POINTER(C.c_uint32))
    return ptrs, lens, (blob, addrs, lens_keep)


class PackedSaves:
    """The C form of a list of LayerSave, reusable across calls.  Layers that
    pass the very same hash list object share one packed copy."""

    def __init__(self, saves: Sequence[LayerSave]):
        n = len(saves)
        self.n = n
        self.array = (_lib.PfLayerSave * max(n, 1))()
        self._keep = []
        packed_hashes = {}
        for i, s in enumerate(saves):
            if len(s.block_hashes) != len(s.block_ids):
                # offload.rs:328-335
                raise _lib.InvalidArgument(
                    _lib.PF_ERR_INVALID_ARGUMENT,
                    f"block_ids length {len(s.block_ids)} does not match block_hashes "
                    f"{len(s.block_hashes)} for layer {s.layer_name}")
            ids = np.ascontiguousarray(s.block_ids, dtype=np.uint64)
            if ids.size == 0:
                ids = np.zeros(1, dtype=np.uint64)
            name = s.layer_name.encode()
            key = id(s.block_hashes)
            if key not in packed_hashes:
                packed_hashes[key] = _pack_hashes(s.block_hashes)
            ptrs, lens, _ = packed_hashes[key]
            a = self.array[i]
            a.layer_name = name
            a.block_ids = C.cast(ids.ctypes.data, C.POINTER(C.c_uint64))
            a.n_blocks = len(s.block_ids)
            a.block_hashes = ptrs
            a.block_hash_lens = lens
            self._keep.append((ids, name, s.block_hashes))
        self._keep.append(packed_hashes)


class PegaEngine:
    """Save / query / load by block ID on one node."""

    def __init__(self, pool_size: int, use_hugepages: bool = False, numa_aware: bool = False,
                 pool_shards: int = 1, blockwise_alloc: bool = False, ssd_enabled: bool = False,
                 use_descriptor_backends: bool = False, unit_size_hint: int = 0,
                 lease_ttl_ms: int = 0, auto_staged_min_bytes: int = 0,
                 staging_slot_bytes: int = 0, lazy_staging: bool = False,
                 kernel_mode_zerocopy: bool = False, side_copy_streams: bool = False):
        """``lease_ttl_ms``: how long an unconsumed query lease pins its blocks
        (0 = the reference's 600 s, lease.rs:11).  ``auto_staged_min_bytes``: a
        task whose dense layers add up to this much is staged through device
        memory by the workers instead of moved with the resident zero-copy
        kernel (0 = 8 MiB; layers of 16 MiB and more are staged in any case);
        1 = stage whatever can be staged, for servers that would rather
        lengthen small loads than disturb the model's kernels.
        ``staging_slot_bytes``: upper bound of a worker's staging slot (0 =
        512 MiB); every registered context holds 2 workers x 2 slots of
        min(this, what its layers can fill) in device memory from registration
        on, unless ``lazy_staging``.  ``kernel_mode_zerocopy``: registrations
        with TransferMode.KERNEL get zero-copy workers, the reference's meaning
        of that mode, instead of the per-task choice.  ``side_copy_streams``:
        every worker moves its link copies on a second stream of its own (they
        then overlap its gather / scatter kernels: 1-2 % for a direction running
        alone) instead of in order on its one stream; four streams per context,
        for processes with one context per GPU (pf_engine_config)."""
        self._lib = _lib.load()
        cfg = _lib.PfEngineConfig(pool_size, int(use_hugepages), int(numa_aware), pool_shards,
                                  int(blockwise_alloc), int(ssd_enabled),
                                  int(use_descriptor_backends), unit_size_hint, lease_ttl_ms,
                                  auto_staged_min_bytes, staging_slot_bytes, int(lazy_staging),
                                  int(kernel_mode_zerocopy), int(side_copy_streams), 0)
        h = C.c_void_p()
        check(self._lib.pf_engine_create(C.byref(cfg), C.byref(h)))
        self.handle = h

    def register_context_layer_batch(self, instance_id: str, namespace: str, device_id: int,
                                     tp_rank: int, pp_rank: int, tp_size: int, world_size: int,
                                     layer_names: Sequence[str], data_ptrs: Sequence[int],
                                     size_bytes_list: Sequence[int], num_blocks_list: Sequence[int],
                                     bytes_per_block_list: Sequence[int],
                                     kv_stride_bytes_list: Sequence[int],
                                     segments_list: Sequence[int],
                                     transfer_mode: int = TransferMode.DIRECT,
                                     page_first: bool = False,
                                     block_stride_bytes_list: Sequence[int] | None = None,
                                     layer_group_ids: Sequence[int] | None = None) -> None:
        n = len(layer_names)
        lists = (data_ptrs, size_bytes_list, num_blocks_list, bytes_per_block_list,
                 kv_stride_bytes_list, segments_list)
        if any(len(x) != n for x in lists):
            raise _lib.InvalidArgument(
                _lib.PF_ERR_INVALID_ARGUMENT,
                f"registration metadata length mismatch: layer_names={n}, "
                + ", ".join(f"{k}={len(v)}" for k, v in zip(
                    ("data_ptrs", "size_bytes", "num_blocks", "bytes_per_block",
                     "kv_stride_bytes", "segments"), lists)))
        u64 = C.c_uint64
        names = (C.c_char_p * max(n, 1))(*[s.encode() for s in layer_names])
        arrs = [(u64 * max(n, 1))(*[int(v) for v in x]) for x in lists]
        strides = (u64 * max(n, 1))(*block_stride_bytes_list) if block_stride_bytes_list else None
        groups = (C.c_uint32 * max(n, 1))(*layer_group_ids) if layer_group_ids else None
        check(self._lib.pf_engine_register_context_layer_batch(
            self.handle, instance_id.encode(), namespace.encode(), device_id, tp_rank, pp_rank,
            tp_size, world_size, n, names, *arrs, strides, groups, transfer_mode,
            1 if page_first else 0))

    def unregister_instance(self, instance_id: str) -> None:
        check(self._lib.pf_engine_unregister_instance(self.handle, instance_id.encode()))

    def batch_save_kv_blocks(self, instance_id: str, tp_rank: int, pp_rank: int, device_id: int,
                             saves: Sequence[LayerSave] | PackedSaves) -> None:
        packed = saves if isinstance(saves, PackedSaves) else PackedSaves(saves)
        check(self._lib.pf_engine_batch_save(self.handle, instance_id.encode(), tp_rank, pp_rank,
                                             device_id, packed.array, packed.n))

    def query_prefix(self, instance_id: str, hashes: Sequence[bytes]) -> tuple[int, int]:
        """-> (hit blocks, lease id); lease 0 when nothing hit."""
        ptrs, lens, _bufs = _pack_hashes(hashes)
        hits, lease = C.c_uint64(), C.c_uint64()
        check(self._lib.pf_engine_query_prefix(self.handle, instance_id.encode(), ptrs, lens,
                                               len(hashes), C.byref(hits), C.byref(lease)))
        return hits.value, lease.value

    def release_query_lease(self, lease: int) -> None:
        check(self._lib.pf_engine_release_lease(self.handle, lease))

    def batch_load_kv_blocks_multi_layer(self, instance_id: str, tp_rank: int, device_id: int,
                                         layer_groups: Sequence[Sequence[str]], lease: int,
                                         dest_block_ids_by_group: Sequence[Sequence[int | None]],
                                         load_state: LoadState | None = None) -> Task:
        g = len(layer_groups)
        keep = []
        group_ptrs = (C.POINTER(C.c_char_p) * max(g, 1))()
        sizes = (C.c_uint64 * max(g, 1))()
        dests = (C.POINTER(C.c_int64) * max(g, 1))()
        n_blocks = len(dest_block_ids_by_group[0]) if g else 0
        for i, names in enumerate(layer_groups):
            arr = (C.c_char_p * max(len(names), 1))(*[s.encode() for s in names])
            keep.append(arr)
            group_ptrs[i] = arr
            sizes[i] = len(names)
            ids = dest_block_ids_by_group[i]
            if len(ids) != n_blocks:
                raise _lib.InvalidArgument(_lib.PF_ERR_INVALID_ARGUMENT,
                                           "every load group needs one destination per leased block")
            d = (C.c_int64 * max(n_blocks, 1))(*[-1 if v is None else int(v) for v in ids])
            keep.append(d)
            dests[i] = d
        t = C.c_void_p()
        shm = load_state.shm_name.encode() if load_state is not None else None
        check(self._lib.pf_engine_batch_load(self.handle, instance_id.encode(), tp_rank, device_id,
                                             g, group_ptrs, sizes, lease, dests, n_blocks, shm,
                                             C.byref(t)))
        return Task(t, keep)

    def query_group_membership(self, instance_id: str, group: int,
                               hashes: Sequence[bytes]) -> list[bool]:
        """Which of ``hashes`` are sealed in storage group ``group``, position by
        position (no prefix rule)."""
        ptrs, lens, _bufs = _pack_hashes(hashes)
        out = (C.c_uint8 * max(len(hashes), 1))()
        check(self._lib.pf_engine_query_group_membership(self.handle, instance_id.encode(), group,
                                                         ptrs, lens, len(hashes), out))
        return [bool(out[i]) for i in range(len(hashes))]

    def create_group_lease(self, instance_id: str, group: int, hashes: Sequence[bytes]) -> int:
        """A lease over exactly the blocks of ``hashes`` in ``group``."""
        ptrs, lens, _bufs = _pack_hashes(hashes)
        lease = C.c_uint64()
        check(self._lib.pf_engine_create_group_lease(self.handle, instance_id.encode(), group,
                                                     ptrs, lens, len(hashes), C.byref(lease)))
        return lease.value

    def query_group_lease(self, instance_id: str, group: int, hashes: Sequence[bytes],
                          require_all: bool = False) -> tuple[list[bool], int]:
        """Membership and lease in one step under the engine's lock: which of
        ``hashes`` are sealed in ``group`` and a lease over exactly those blocks
        (0 when none is, or when ``require_all`` and one is missing)."""
        ptrs, lens, _bufs = _pack_hashes(hashes)
        out = (C.c_uint8 * max(len(hashes), 1))()
        lease = C.c_uint64()
        check(self._lib.pf_engine_query_group_lease(self.handle, instance_id.encode(), group, ptrs,
                                                    lens, len(hashes), 1 if require_all else 0,
                                                    out, C.byref(lease)))
        return [bool(out[i]) for i in range(len(hashes))], lease.value

    def batch_load_multi(self, instance_id: str, tp_rank: int, device_id: int,
                         layer_groups: Sequence[Sequence[str]],
                         loads: Sequence[tuple[int, Sequence[Sequence[int | None]]]],
                         load_state: LoadState | None = None) -> Task:
        """Several leases in one load task: ``loads`` = [(lease, destinations
        per layer group)], each destination list as long as the lease."""
        g = len(layer_groups)
        keep = []
        group_ptrs = (C.POINTER(C.c_char_p) * max(g, 1))()
        sizes = (C.c_uint64 * max(g, 1))()
        for i, names in enumerate(layer_groups):
            arr = (C.c_char_p * max(len(names), 1))(*[s.encode() for s in names])
            keep.append(arr)
            group_ptrs[i] = arr
            sizes[i] = len(names)
        reqs = (_lib.PfLoadRequest * max(len(loads), 1))()
        for li, (lease, dests) in enumerate(loads):
            if len(dests) != g:
                raise _lib.InvalidArgument(
                    _lib.PF_ERR_INVALID_ARGUMENT,
                    f"load group count {len(dests)} does not match layer group count {g}")
            n_blocks = len(dests[0]) if g else 0
            ptrs = (C.POINTER(C.c_int64) * max(g, 1))()
            for gi, ids in enumerate(dests):
                if len(ids) != n_blocks:
                    raise _lib.InvalidArgument(
                        _lib.PF_ERR_INVALID_ARGUMENT,
                        "every load group needs one destination per leased block")
                d = (C.c_int64 * max(n_blocks, 1))(*[-1 if v is None else int(v) for v in ids])
                keep.append(d)
                ptrs[gi] = d
            keep.append(ptrs)
            reqs[li].lease = lease
            reqs[li].dest_block_ids = ptrs
            reqs[li].n_blocks = n_blocks
        t = C.c_void_p()
        shm = load_state.shm_name.encode() if load_state is not None else None
        check(self._lib.pf_engine_batch_load_multi(self.handle, instance_id.encode(), tp_rank,
                                                   device_id, g, group_ptrs, sizes, reqs, len(loads),
                                                   shm, C.byref(t)))
        return Task(t, keep)

    def last_save_profile(self) -> dict:
        """Milliseconds per phase of the last successful save (and its bytes)."""
        p = _lib.PfSaveProfile()
        check(self._lib.pf_engine_last_save_profile(self.handle, C.byref(p)))
        return {name: getattr(p, name) for name, _ in p._fields_}

    def last_load_profile(self) -> TaskResult | None:
        """The load task that settled last on this engine (None before any)."""
        r = _lib.PfTaskResult()
        if self._lib.pf_engine_last_load_profile(self.handle, C.byref(r)) != _lib.PF_OK:
            return None
        return TaskResult.from_c(r)

    @property
    def staging_bytes(self) -> int:
        """Device memory the worker pools of all registered contexts hold for staging."""
        return self._lib.pf_engine_staging_bytes(self.handle)

    def pool_usage(self) -> tuple[int, int]:
        used, total = C.c_uint64(), C.c_uint64()
        check(self._lib.pf_engine_pool_usage(self.handle, C.byref(used), C.byref(total)))
        return used.value, total.value

    @property
    def cached_blocks(self) -> int:
        return self._lib.pf_engine_cached_blocks(self.handle)

    @property
    def inflight_blocks(self) -> int:
        """Blocks that have some but not all of their slots."""
        return self._lib.pf_engine_inflight_blocks(self.handle)

    def gc_stale_inflight(self, max_age_seconds: float) -> int:
        """Drop incomplete blocks older than ``max_age_seconds``; returns how many."""
        return self._lib.pf_engine_gc_stale_inflight(self.handle, int(max_age_seconds * 1000))

    def evict_all(self) -> int:
        return self._lib.pf_engine_evict_all(self.handle)

    def sweep_expired_leases(self) -> int:
        """Drop the query leases whose time is up (the reference's periodic
        sweeper, lease.rs:66-80); returns how many."""
        return self._lib.pf_engine_sweep_expired_leases(self.handle)

    def live_leases(self) -> int:
        return self._lib.pf_engine_live_leases(self.handle)

    def close(self) -> None:
        if self.handle is not None:
            self._lib.pf_engine_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
