"""ctypes front-end of the CPU oracle (``pf_oracle.c``) plus an independent
numpy restatement of block gather/scatter.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke``
and by the ``cpu_baseline`` leg of ``bench.py``.  The product package
``pegaflow_amd`` never imports it.

Reference lines each function follows are cited in ``pf_oracle.c``.
"""

from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libpf_oracle.so")


def build(force: bool = False) -> str:
    """Compile ``pf_oracle.c`` with gcc (a few hundred milliseconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-B", "-C", _HERE], check=True, capture_output=True)
    return _LIB_PATH


class OrcLayout(C.Structure):
    _fields_ = [
        ("data_ptr", C.c_uint64),
        ("size_bytes", C.c_uint64),
        ("num_blocks", C.c_uint64),
        ("block_stride_bytes", C.c_uint64),
        ("segment_bytes", C.c_uint64),
        ("segments", C.c_uint64),
        ("padded_segment_bytes", C.c_uint64),
        ("kv_stride_bytes", C.c_uint64),
        ("split", C.c_int32),
        ("pad_", C.c_int32),
    ]


class OrcDesc(C.Structure):
    _fields_ = [
        ("device", C.c_uint64),
        ("host", C.c_uint64),
        ("host_device", C.c_uint64),
        ("size", C.c_uint64),
        ("device_allocation", C.c_uint64),
        ("host_allocation", C.c_uint64),
    ]


class OrcRange(C.Structure):
    _fields_ = [("device", C.c_uint64), ("host", C.c_uint64), ("size", C.c_uint64)]


class OrcLayer(C.Structure):
    _fields_ = [
        ("layout", OrcLayout),
        ("block_idx", C.POINTER(C.c_uint64)),
        ("seg0_host", C.POINTER(C.c_uint64)),
        ("seg0_dev", C.POINTER(C.c_uint64)),
        ("seg0_alloc", C.POINTER(C.c_uint64)),
        ("seg1_host", C.POINTER(C.c_uint64)),
        ("seg1_dev", C.POINTER(C.c_uint64)),
        ("seg1_alloc", C.POINTER(C.c_uint64)),
        ("host_offset", C.POINTER(C.c_uint64)),
        ("n_blocks", C.c_uint64),
    ]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_merge.restype = C.c_uint64
        _lib.orc_sizeof_layout.restype = C.c_size_t
        _lib.orc_sizeof_desc.restype = C.c_size_t
        _lib.orc_sizeof_layer.restype = C.c_size_t
        assert _lib.orc_sizeof_layout() == C.sizeof(OrcLayout)
        assert _lib.orc_sizeof_desc() == C.sizeof(OrcDesc)
        assert _lib.orc_sizeof_layer() == C.sizeof(OrcLayer)
    return _lib


class OracleError(ValueError):
    pass


_ERRCAP = 512


def _u64(v):
    return C.c_uint64(int(v))


class Layout:
    """KVCacheLayout restated (layout.rs:13-286)."""

    def __init__(self, data_ptr, size_bytes, num_blocks, segment_bytes, kv_stride_bytes, segments):
        self.c = OrcLayout()
        err = C.create_string_buffer(_ERRCAP)
        rc = lib().orc_layout_new(
            _u64(data_ptr), _u64(size_bytes), _u64(num_blocks), _u64(segment_bytes),
            _u64(kv_stride_bytes), _u64(segments), C.byref(self.c), err, C.c_size_t(_ERRCAP))
        if rc:
            raise OracleError(err.value.decode())

    def with_block_stride(self, stride):
        err = C.create_string_buffer(_ERRCAP)
        if lib().orc_layout_with_block_stride(C.byref(self.c), _u64(stride), err, C.c_size_t(_ERRCAP)):
            raise OracleError(err.value.decode())
        return self

    def with_ssd_padding(self, alignment):
        lib().orc_layout_with_ssd_padding(C.byref(self.c), _u64(alignment))
        return self

    def block_copies(self, idx):
        addr = (C.c_uint64 * 2)()
        nbytes = (C.c_uint64 * 2)()
        n = C.c_int()
        err = C.create_string_buffer(_ERRCAP)
        if lib().orc_block_copies(C.byref(self.c), _u64(idx), addr, nbytes, C.byref(n), err,
                                  C.c_size_t(_ERRCAP)):
            raise OracleError(err.value.decode())
        return [(addr[i], nbytes[i]) for i in range(n.value)]

    @property
    def is_split(self):
        return bool(self.c.split)

    @property
    def segment_bytes(self):
        return self.c.segment_bytes

    @property
    def block_bytes(self):
        return self.c.segment_bytes * self.c.segments

    @property
    def padded_segment_bytes(self):
        return self.c.padded_segment_bytes

    @property
    def padded_block_bytes(self):
        return self.c.padded_segment_bytes * self.c.segments

    @property
    def num_blocks(self):
        return self.c.num_blocks

    @property
    def fragment_bytes(self):
        return self.c.segment_bytes if self.c.split else self.block_bytes

    @property
    def host_stride(self):
        """Host stride of one fragment in the layer-first batch image (offload.rs:472-499)."""
        return self.c.padded_segment_bytes if self.c.split else self.padded_block_bytes


def make_descs(rows):
    """rows: iterable of (device, host, host_device, size, dev_alloc, host_alloc)."""
    rows = list(rows)
    arr = (OrcDesc * max(len(rows), 1))()
    for i, r in enumerate(rows):
        arr[i] = OrcDesc(*[int(x) for x in r])
    return arr, len(rows)


def merge(rows):
    """merge() of memcpy.rs:25-55 -> list of (device, host, size)."""
    arr, n = make_descs(rows)
    out = (OrcRange * max(n, 1))()
    m = lib().orc_merge(arr, _u64(n), out)
    return [(out[i].device, out[i].host, out[i].size) for i in range(m)]


def exec_descs(rows, host_is_src: bool, backend: str = "kernel", threads: int = 1):
    arr, n = make_descs(rows)
    fn = lib().orc_exec_direct if backend == "direct" else lib().orc_exec_kernel
    fn(arr, _u64(n), C.c_int(1 if host_is_src else 0), C.c_int(threads))


def emulate_batch_copy_kernel(table: np.ndarray, grid: int, block: int):
    """Literal loop nest of the reference kernel (kernel.rs:25-46)."""
    table = np.ascontiguousarray(table, dtype=np.uint64)
    n = table.size // 3
    lib().orc_emulate_batch_copy_kernel(
        table.ctypes.data_as(C.POINTER(C.c_uint64)), C.c_int(n), C.c_uint(grid), C.c_uint(block))


def _p64(a):
    return a.ctypes.data_as(C.POINTER(C.c_uint64)) if a is not None else None


@dataclass
class LayerBlocks:
    """One layer of a transfer for build_copy_descs (gpu_worker.rs:54-101)."""
    layout: Layout
    block_idx: np.ndarray
    seg0_host: np.ndarray
    seg0_dev: np.ndarray
    seg0_alloc: np.ndarray
    seg1_host: np.ndarray | None = None
    seg1_dev: np.ndarray | None = None
    seg1_alloc: np.ndarray | None = None
    host_offset: np.ndarray | None = None


def build_copy_descs(layers):
    """build_copy_descs of gpu_worker.rs:353-423.

    Returns (list of desc tuples, total_bytes); raises OracleError with
    'layer #<index>: <cause>' on a bad block id.
    """
    n_layers = len(layers)
    arr = (OrcLayer * max(n_layers, 1))()
    keep = []
    cap = 0
    for i, L in enumerate(layers):
        cols = {}
        for name in ("block_idx", "seg0_host", "seg0_dev", "seg0_alloc", "seg1_host", "seg1_dev",
                     "seg1_alloc", "host_offset"):
            v = getattr(L, name)
            cols[name] = None if v is None else np.ascontiguousarray(v, dtype=np.uint64)
        keep.append(cols)
        arr[i].layout = L.layout.c
        for name, v in cols.items():
            setattr(arr[i], name, _p64(v))
        arr[i].n_blocks = len(cols["block_idx"])
        cap += 2 * len(cols["block_idx"])
    out = (OrcDesc * max(cap, 1))()
    n_out = C.c_uint64()
    total = C.c_uint64()
    bad = C.c_uint64()
    err = C.create_string_buffer(_ERRCAP)
    rc = lib().orc_build_copy_descs(arr, _u64(n_layers), out, _u64(cap), C.byref(n_out),
                                    C.byref(total), C.byref(bad), err, C.c_size_t(_ERRCAP))
    if rc:
        raise OracleError(f"layer #{bad.value}: {err.value.decode()}")
    descs = [(d.device, d.host, d.host_device, d.size, d.device_allocation, d.host_allocation)
             for d in out[: n_out.value]]
    return descs, total.value


def build_page_layout(worker_layer_sets, n_layers, padded_bytes):
    """build_page_layout of instance.rs:107-162.

    Returns dict(layer_shard, layer_offsets, layer_bytes, shard_page_sizes).
    """
    flat = []
    off = [0]
    for s in worker_layer_sets:
        flat.extend(int(x) for x in s)
        off.append(len(flat))
    flat_a = np.asarray(flat if flat else [0], dtype=np.uint64)
    off_a = np.asarray(off, dtype=np.uint64)
    padded = np.asarray(list(padded_bytes) if n_layers else [0], dtype=np.uint64)
    layer_shard = np.zeros(max(n_layers, 1), dtype=np.uint64)
    layer_offsets = np.zeros(max(n_layers, 1), dtype=np.uint64)
    layer_bytes = np.zeros(max(n_layers, 1), dtype=np.uint64)
    shard_sizes = np.zeros(max(len(worker_layer_sets), 1), dtype=np.uint64)
    n_shards = C.c_uint64()
    bad_layer, a, b = C.c_uint64(), C.c_uint64(), C.c_uint64()
    rc = lib().orc_build_page_layout(
        _p64(flat_a), _p64(off_a), _u64(len(worker_layer_sets)), _u64(n_layers), _p64(padded),
        _p64(layer_shard), _p64(layer_offsets), _p64(layer_bytes), _p64(shard_sizes),
        C.byref(n_shards), C.byref(bad_layer), C.byref(a), C.byref(b))
    if rc == 1:
        raise OracleError(
            f"page-first layer #{bad_layer.value} claimed by shards {a.value} and {b.value}")
    if rc == 2:
        raise OracleError(f"page-first layer #{bad_layer.value} has no shard owner after sealing")
    return {
        "layer_shard": [int(x) for x in layer_shard[:n_layers]],
        "layer_offsets": [int(x) for x in layer_offsets[:n_layers]],
        "layer_bytes": [int(x) for x in layer_bytes[:n_layers]],
        "shard_page_sizes": [int(x) for x in shard_sizes[: n_shards.value]],
    }


def layout_over(cache: np.ndarray, num_blocks, segment_bytes, kv_stride_bytes, segments):
    """A Layout whose 'device' memory is the numpy byte buffer ``cache``."""
    assert cache.dtype == np.uint8 and cache.flags.c_contiguous
    return Layout(cache.ctypes.data, cache.nbytes, num_blocks, segment_bytes, kv_stride_bytes,
                  segments)


def transfer_layer(layout: Layout, ids, host_k: np.ndarray, host_v: np.ndarray | None,
                   host_is_src: bool, backend: str = "kernel", threads: int = 1):
    """Save (host_is_src=False) or load one layer over the layer-first batch
    host image (offload.rs:454-509 + gpu_worker.rs:353-423 + a backend)."""
    ids = np.ascontiguousarray(ids, dtype=np.uint32)
    err = C.create_string_buffer(_ERRCAP)
    hv = host_v.ctypes.data_as(C.POINTER(C.c_uint8)) if host_v is not None else None
    rc = lib().orc_transfer_layer(
        C.byref(layout.c), ids.ctypes.data_as(C.POINTER(C.c_uint32)), _u64(len(ids)),
        host_k.ctypes.data_as(C.POINTER(C.c_uint8)), hv, C.c_int(1 if host_is_src else 0),
        C.c_int(1 if backend == "direct" else 0), C.c_int(threads), err, C.c_size_t(_ERRCAP))
    if rc:
        raise OracleError(err.value.decode())


def transfer_layer_paged(layout: Layout, ids, pages, offset: int, host_is_src: bool,
                         threads: int = 1):
    """Page-first save/load of one layer (offload.rs:182-282)."""
    ids = np.ascontiguousarray(ids, dtype=np.uint32)
    pages = np.ascontiguousarray(pages, dtype=np.uint64)
    err = C.create_string_buffer(_ERRCAP)
    rc = lib().orc_transfer_layer_paged(
        C.byref(layout.c), ids.ctypes.data_as(C.POINTER(C.c_uint32)), _u64(len(ids)), _p64(pages),
        _u64(offset), C.c_int(1 if host_is_src else 0), C.c_int(threads), err, C.c_size_t(_ERRCAP))
    if rc:
        raise OracleError(err.value.decode())


# ---------------------------------------------------------------------------
# Independent numpy restatement (no shared code with pf_oracle.c): the cache
# is viewed as arrays and blocks are moved by fancy indexing.  Only for the
# dense layouts the BASELINE configs use; it pins the C oracle on those.
# ---------------------------------------------------------------------------

def np_save_split(cache: np.ndarray, num_blocks: int, seg: int, ids) -> tuple[np.ndarray, np.ndarray]:
    """cache: uint8[2*num_blocks*seg] laid out [K blocks | V blocks]."""
    view = cache.reshape(2, num_blocks, seg)
    ids = np.asarray(ids, dtype=np.int64)
    return view[0, ids].copy(), view[1, ids].copy()


def np_load_split(cache: np.ndarray, num_blocks: int, seg: int, ids, host_k, host_v) -> None:
    view = cache.reshape(2, num_blocks, seg)
    ids = np.asarray(ids, dtype=np.int64)
    view[0, ids] = host_k.reshape(len(ids), seg)
    view[1, ids] = host_v.reshape(len(ids), seg)


def np_save_contiguous(cache: np.ndarray, num_blocks: int, block: int, ids) -> np.ndarray:
    view = cache.reshape(num_blocks, block)
    return view[np.asarray(ids, dtype=np.int64)].copy()


def np_load_contiguous(cache: np.ndarray, num_blocks: int, block: int, ids, host) -> None:
    view = cache.reshape(num_blocks, block)
    view[np.asarray(ids, dtype=np.int64)] = host.reshape(len(ids), block)
