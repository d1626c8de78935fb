"""Transfer interfaces over the C ABI.

Mirrors the reference's ``CopyDesc`` / ``TransferBackend`` / ``TransferMode``
(pegaflow-core/src/transfer/mod.rs:36-76), ``merge``
(transfer/memcpy.rs:25-55), ``build_copy_descs``
(pegaflow-core/src/gpu_worker.rs:353-423) and adds the block-ID fast path
(``BlockTransfer``) that moves the same bytes without per-fragment
descriptors.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from typing import Sequence

import numpy as np

from . import _lib
from ._lib import check
from .layout import KVCacheLayout
from .runtime import Event, Stream


@dataclass(frozen=True)
class CopyDesc:
    """One contiguous copy between device memory and mapped pinned host
    memory; the direction is chosen by the backend method called."""
    device: int
    host: int
    host_device: int
    size: int
    device_allocation: int = 0
    host_allocation: int = 0


def desc_array(device, host, host_device, size, device_allocation=0, host_allocation=0) -> np.ndarray:
    """Descriptor batch as a uint64 array of shape (n, 6) in ``CopyDesc`` field
    order (the memory layout of ``pf_copy_desc``); arguments broadcast."""
    cols = np.broadcast_arrays(*[np.asarray(c, dtype=np.uint64) for c in
                                 (device, host, host_device, size, device_allocation,
                                  host_allocation)])
    return np.ascontiguousarray(np.stack(cols, axis=-1).reshape(-1, 6))


def _pack(copies):
    if isinstance(copies, np.ndarray):
        if copies.dtype != np.uint64 or copies.ndim != 2 or copies.shape[1] != 6 \
                or not copies.flags.c_contiguous:
            raise ValueError("descriptor array must be C-contiguous uint64 of shape (n, 6)")
        return C.cast(copies.ctypes.data, C.POINTER(_lib.PfCopyDesc)), copies.shape[0]
    n = len(copies)
    arr = (_lib.PfCopyDesc * max(n, 1))()
    for i, c in enumerate(copies):
        arr[i] = _lib.PfCopyDesc(c.device, c.host, c.host_device, c.size, c.device_allocation,
                                 c.host_allocation)
    return arr, n


def merge(copies: Sequence[CopyDesc]) -> list[tuple[int, int, int]]:
    """Coalesce list-adjacent copies contiguous on both sides within the same
    allocations -> [(device, host, size)]."""
    arr, n = _pack(copies)
    out = (_lib.PfMergedRange * max(n, 1))()
    m = C.c_uint64()
    check(_lib.load().pf_merge_copies(arr, n, out, C.byref(m)))
    return [(out[i].device, out[i].host or 0, out[i].size) for i in range(m.value)]


class TransferMode:
    DIRECT = _lib.PF_MODE_DIRECT
    KERNEL = _lib.PF_MODE_KERNEL
    ZEROCOPY = _lib.PF_MODE_ZEROCOPY   # worker pools / engine registrations only

    @staticmethod
    def from_name(name: str) -> int:
        mode = C.c_int()
        check(_lib.load().pf_transfer_mode_from_name(name.encode(), C.byref(mode)))
        return mode.value


class TransferBackend:
    """``h2d`` / ``d2h`` enqueue a descriptor batch on a stream and never
    synchronise.  One instance per worker thread."""

    def __init__(self, mode: int):
        self._lib = _lib.load()
        h = C.c_void_p()
        check(self._lib.pf_backend_create(mode, C.byref(h)))
        self.handle = h

    @property
    def name(self) -> str:
        return self._lib.pf_backend_name(self.handle).decode()

    def h2d(self, copies: Sequence[CopyDesc], stream: Stream) -> None:
        arr, n = _pack(copies)
        check(self._lib.pf_backend_h2d(self.handle, arr, n, stream.handle))

    def d2h(self, copies: Sequence[CopyDesc], stream: Stream) -> None:
        arr, n = _pack(copies)
        check(self._lib.pf_backend_d2h(self.handle, arr, n, stream.handle))

    def close(self) -> None:
        if self.handle is not None:
            self._lib.pf_backend_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def desc_copy_noalloc(copies, stream: Stream, host_is_src: bool):
    """The kernel backend's copy through ``pf_desc_copy_noalloc``: nothing is
    allocated, the batch is limited to ``desc_copy_noalloc_max()`` descriptors.
    Returns the packed descriptor array, which the caller keeps alive until
    the stream has been synchronised."""
    arr, n = _pack(copies)
    check(_lib.load().pf_desc_copy_noalloc(arr, n, 1 if host_is_src else 0, stream.handle))
    return arr


def desc_copy_noalloc_max() -> int:
    return int(_lib.load().pf_desc_copy_noalloc_max())


class MemcpyBackend(TransferBackend):
    """One DMA copy per merged range ("direct")."""

    def __init__(self):
        super().__init__(TransferMode.DIRECT)


class KernelBackend(TransferBackend):
    """One copy kernel over mapped pinned host memory ("kernel")."""

    def __init__(self):
        super().__init__(TransferMode.KERNEL)


def build_backend(mode: int) -> TransferBackend:
    return KernelBackend() if mode == TransferMode.KERNEL else MemcpyBackend()


@dataclass
class HostBlock:
    """Host image of one block as the transfer sees it: one or two segments
    (host address, device-visible address, allocation identity) plus the
    page-first byte offset of this layer."""
    seg_host: tuple[int, ...]
    seg_device: tuple[int, ...]
    seg_alloc: tuple[int, ...]
    seg_size: tuple[int, ...] = ()
    host_offset: int = 0


@dataclass
class LayerTransferData:
    """One layer of a transfer task: layout plus (device slot, host image)."""
    layer_name: str
    layout: KVCacheLayout
    block_idx: Sequence[int]
    blocks: Sequence[HostBlock]


def build_copy_descs(layers: Sequence[LayerTransferData]) -> tuple[list[CopyDesc], int]:
    """One ``CopyDesc`` per device segment of every block across all layers,
    in layer order then block order (K before V) -> (copies, total_bytes)."""
    lib = _lib.load()
    n_layers = len(layers)
    arr = (_lib.PfLayerTransfer * max(n_layers, 1))()
    keep = []
    cap = 0
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
        cap += 2 * nb
    out = (_lib.PfCopyDesc * max(cap, 1))()
    n_out = C.c_uint64()
    total = C.c_uint64()
    check(lib.pf_build_copy_descs(arr, n_layers, out, cap, C.byref(n_out), C.byref(total)))
    descs = [CopyDesc(d.device, d.host or 0, d.host_device, d.size, d.device_allocation,
                      d.host_allocation) for d in out[: n_out.value]]
    return descs, total.value


class TransferPath:
    AUTO = _lib.PF_PATH_AUTO
    ZEROCOPY = _lib.PF_PATH_ZEROCOPY
    STAGED = _lib.PF_PATH_STAGED


@dataclass
class LayerBlocks:
    """One layer of a block-ID transfer.

    Dense / strided host image: segment ``s`` of list position ``i`` lives at
    ``host[s] + i*host_stride``.  Page-first: at ``page_host[i] + page_offset``.
    ``block_ids[i]`` is the device slot of list position ``i``.
    """
    layout: KVCacheLayout
    block_ids: np.ndarray
    host: tuple[int, ...] = ()
    host_device: tuple[int, ...] = ()
    host_len: tuple[int, ...] = ()
    host_stride: int = 0
    page_host: np.ndarray | None = None
    page_host_device: np.ndarray | None = None
    page_offset: int = 0
    page_len: int = 0
    layer_name: str | None = None
    _keep: list = field(default_factory=list, repr=False)


@dataclass(frozen=True)
class FillUnit:
    """One unit of a staged call: list positions ``first .. first+count`` of
    layer ``layer``, at ``slot_offset`` of the staging slot of fill number
    ``fill`` (None: the layer is not staged)."""
    layer: int
    first: int
    count: int
    slot_offset: int
    fill: int | None


def plan_staged_fills(layer_blocks: Sequence[int], block_bytes: Sequence[int],
                      staging_slot_bytes: int = 0, staged_group_bytes: int = 0,
                      per_layer_events: bool = False) -> tuple[list[FillUnit], int]:
    """(units, number of fills) of a staged save or load of these layers: the
    planner ``BlockTransfer`` uses, as host arithmetic (pf_plan_staged_fills).
    One gather or scatter launch runs per fill."""
    lib = _lib.load()
    n = len(layer_blocks)
    if len(block_bytes) != n:
        raise ValueError("layer_blocks and block_bytes differ in length")
    blocks = (C.c_uint64 * max(n, 1))(*layer_blocks)
    sizes = (C.c_uint64 * max(n, 1))(*block_bytes)
    n_units, n_fills = C.c_uint64(), C.c_uint64()
    args = (blocks, sizes, n, staging_slot_bytes, staged_group_bytes, int(per_layer_events))
    check(lib.pf_plan_staged_fills(*args, None, 0, C.byref(n_units), C.byref(n_fills)))
    out = (_lib.PfFillUnit * max(n_units.value, 1))()
    check(lib.pf_plan_staged_fills(*args, out, n_units.value, C.byref(n_units), C.byref(n_fills)))
    none = (1 << 64) - 1
    units = [FillUnit(int(u.layer), int(u.first), int(u.count), int(u.slot_offset),
                      None if u.fill == none else int(u.fill)) for u in out[: n_units.value]]
    return units, int(n_fills.value)


class BlockTransfer:
    """Block-ID gather (save) / scatter (load) engine.  Enqueue-only; one
    instance per worker thread."""

    def __init__(self, staging_slot_bytes: int = 0, staging_slots: int = 0,
                 zerocopy_max_workgroups: int = 0, auto_staged_min_bytes: int = 0,
                 tile_unroll: int = 0, copy_stream: int = 0,
                 auto_staged_min_call_bytes: int = 0, staged_group_bytes: int = 0):
        self._lib = _lib.load()
        cfg = _lib.PfXferConfig(staging_slot_bytes, staging_slots, zerocopy_max_workgroups,
                                auto_staged_min_bytes, tile_unroll, copy_stream,
                                auto_staged_min_call_bytes, staged_group_bytes)
        h = C.c_void_p()
        check(self._lib.pf_xfer_create(C.byref(cfg), C.byref(h)))
        self.handle = h
        self._events_keep = None

    def _pack(self, layers: Sequence[LayerBlocks]):
        n = len(layers)
        arr = (_lib.PfLayerBlocks * max(n, 1))()
        keep = []
        for i, L in enumerate(layers):
            ids = np.ascontiguousarray(L.block_ids, dtype=np.uint32)
            keep.append(ids)
            a = arr[i]
            if L.layer_name is not None:
                name = L.layer_name.encode()
                keep.append(name)
                a.layer_name = name
            a.layout = L.layout.c
            a.block_ids = ids.ctypes.data_as(C.POINTER(C.c_uint32))
            a.n_blocks = ids.size
            for s in range(len(L.host)):
                a.host[s] = L.host[s]
                a.host_device[s] = L.host_device[s]
                a.host_len[s] = L.host_len[s]
            a.host_stride = L.host_stride
            if L.page_host is not None:
                ph = np.ascontiguousarray(L.page_host, dtype=np.uint64)
                pd = np.ascontiguousarray(L.page_host_device, dtype=np.uint64)
                keep += [ph, pd]
                a.page_host = ph.ctypes.data_as(C.POINTER(C.c_uint64))
                a.page_host_device = pd.ctypes.data_as(C.POINTER(C.c_uint64))
                a.page_offset = L.page_offset
                a.page_len = L.page_len
        return arr, n, keep

    def save(self, layers: Sequence[LayerBlocks], stream: Stream,
             path: int = TransferPath.AUTO) -> None:
        arr, n, _keep = self._pack(layers)
        check(self._lib.pf_xfer_save(self.handle, arr, n, path, stream.handle))

    def load(self, layers: Sequence[LayerBlocks], stream: Stream,
             path: int = TransferPath.AUTO) -> None:
        arr, n, _keep = self._pack(layers)
        check(self._lib.pf_xfer_load(self.handle, arr, n, path, stream.handle))

    def set_layer_events(self, events: Sequence[Event] | None) -> None:
        if not events:
            self._events_keep = None
            check(self._lib.pf_xfer_set_layer_events(self.handle, None, 0))
            return
        arr = (C.c_void_p * len(events))(*[e.handle for e in events])
        self._events_keep = (arr, list(events))
        check(self._lib.pf_xfer_set_layer_events(self.handle, arr, len(events)))

    @property
    def last_path(self) -> int:
        return self._lib.pf_xfer_last_path(self.handle)

    def set_kernel_timing(self, enable) -> None:
        """False/0 = off; True/1 = launches timed alone, figures per call; 2 =
        launches timed in place, figures add up until ``last_kernel_ms`` reads them."""
        check(self._lib.pf_xfer_set_kernel_timing(self.handle, int(enable)))

    def last_kernel_ms(self) -> tuple[float, int]:
        ms = C.c_float()
        n = C.c_uint32()
        check(self._lib.pf_xfer_last_kernel_ms(self.handle, C.byref(ms), C.byref(n)))
        return ms.value, n.value

    def close(self) -> None:
        if self.handle is not None:
            self._lib.pf_xfer_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
