"""Device memory shared between a worker process and the server process.

``HipIPCWrapper`` is the counterpart of the reference's ``CudaIPCWrapper``
(python/pegaflow/ipc_wrapper.py:15-190): it wraps a device tensor of THIS
process so that another process on the same GPU can map the same memory, and
it identifies the GPU by UUID because device ordinals differ between processes.
The record travels as plain bytes (``to_bytes`` / ``from_bytes``, a fixed
little-endian layout plus a JSON tail for dtype / shape / stride): unlike the
reference's pickled object, reading it executes nothing.

``TensorRegistry`` is the server side (pegaflow-server/src/registry.rs:45-203):
per context key it opens every layer's allocation once, returns the mapped
``data_ptr`` / ``size_bytes`` the engine registers, and keeps the mappings
until the context, the instance or everything is dropped.
"""

from __future__ import annotations

import ctypes as C
import json
import struct
from typing import Sequence

from . import _lib
from ._lib import check

_MAGIC = b"PFIPC1\0\0"
_FIXED = struct.Struct("<8s64sQQQ16sI")   # magic, handle, alloc_size, offset, size, uuid, json len


def device_uuid(device: int) -> bytes:
    buf = (C.c_uint8 * 16)()
    check(_lib.load().pf_device_uuid(device, buf))
    return bytes(buf)


def device_from_uuid(uuid: bytes) -> int:
    """Ordinal, in this process, of the device with this UUID
    (ipc_wrapper.py:75-98)."""
    buf = (C.c_uint8 * 16).from_buffer_copy(uuid)
    out = C.c_int()
    check(_lib.load().pf_device_from_uuid(buf, C.byref(out)))
    return out.value


class HipIPCWrapper:
    """IPC record of one device tensor: handle of the allocation behind it,
    where the tensor's storage sits inside that allocation, and the metadata
    needed to view it again (dtype name, shape, stride, storage offset)."""

    def __init__(self, tensor=None, *, data_ptr: int | None = None, size_bytes: int | None = None,
                 dtype: str = "uint8", shape: Sequence[int] | None = None,
                 stride: Sequence[int] | None = None):
        """From a torch tensor with zero storage offset (the reference's rule,
        ipc_wrapper.py:110), or from a raw ``data_ptr`` / ``size_bytes``."""
        if tensor is not None:
            assert tensor.storage_offset() == 0, "Tensor must have zero storage offset"
            storage = tensor.untyped_storage()
            data_ptr, size_bytes = storage.data_ptr(), storage.nbytes()
            dtype = str(tensor.dtype).replace("torch.", "")
            shape, stride = tuple(tensor.shape), tuple(tensor.stride())
        if data_ptr is None or size_bytes is None:
            raise ValueError("HipIPCWrapper needs a tensor or data_ptr and size_bytes")
        rec = _lib.PfIpcTensor()
        check(_lib.load().pf_ipc_export(data_ptr, size_bytes, C.byref(rec)))
        self.handle = bytes(rec.handle)
        self.alloc_size = rec.alloc_size
        self.offset = rec.offset
        self.size_bytes = rec.size_bytes
        self.device_uuid = bytes(rec.device_uuid)
        self.dtype = dtype
        self.shape = tuple(shape) if shape is not None else (size_bytes,)
        self.stride = tuple(stride) if stride is not None else (1,)
        self.storage_offset = 0

    # -- wire form ---------------------------------------------------------
    def to_bytes(self) -> bytes:
        tail = json.dumps({"dtype": self.dtype, "shape": list(self.shape),
                           "stride": list(self.stride),
                           "storage_offset": self.storage_offset}).encode()
        return _FIXED.pack(_MAGIC, self.handle, self.alloc_size, self.offset, self.size_bytes,
                           self.device_uuid, len(tail)) + tail

    @classmethod
    def from_bytes(cls, data: bytes) -> "HipIPCWrapper":
        if len(data) < _FIXED.size:
            raise ValueError(f"IPC record of {len(data)} bytes is too short")
        magic, handle, alloc_size, offset, size, uuid, n = _FIXED.unpack_from(data)
        if magic != _MAGIC:
            raise ValueError("not a HipIPCWrapper record")
        if len(data) != _FIXED.size + n:
            raise ValueError("IPC record has a truncated metadata tail")
        self = cls.__new__(cls)
        self.handle, self.alloc_size, self.offset, self.size_bytes = handle, alloc_size, offset, size
        self.device_uuid = uuid
        try:
            meta = json.loads(data[_FIXED.size:].decode())
            self.dtype = str(meta["dtype"])
            self.shape = tuple(int(x) for x in meta["shape"])
            self.stride = tuple(int(x) for x in meta["stride"])
            self.storage_offset = int(meta.get("storage_offset", 0))
        except (KeyError, TypeError, AttributeError, UnicodeDecodeError, ValueError) as exc:
            raise ValueError(f"IPC record has a malformed metadata tail: {exc}") from None
        return self

    def c_record(self) -> "_lib.PfIpcTensor":
        rec = _lib.PfIpcTensor()
        C.memmove(rec.handle, self.handle, 64)
        rec.alloc_size, rec.offset, rec.size_bytes = self.alloc_size, self.offset, self.size_bytes
        C.memmove(rec.device_uuid, self.device_uuid, 16)
        return rec

    def __eq__(self, other) -> bool:
        if not isinstance(other, HipIPCWrapper):
            return False
        return (self.handle, self.alloc_size, self.offset, self.size_bytes, self.device_uuid,
                self.dtype, self.shape, self.stride, self.storage_offset) == \
               (other.handle, other.alloc_size, other.offset, other.size_bytes, other.device_uuid,
                other.dtype, other.shape, other.stride, other.storage_offset)

    def __repr__(self) -> str:
        return (f"HipIPCWrapper(shape={self.shape}, dtype={self.dtype}, stride={self.stride}, "
                f"device_uuid={self.device_uuid.hex()})")


def context_key(instance_id: str, tp_rank: int, pp_rank: int, device_id: int) -> str:
    """pegaflow-server/src/service.rs:74-76."""
    return f"{instance_id}:tp{tp_rank}:pp{pp_rank}:dev{device_id}"


class TensorRegistry:
    """Server-side table of the device memory other processes handed over."""

    def __init__(self):
        self._lib = _lib.load()
        h = C.c_void_p()
        check(self._lib.pf_registry_create(C.byref(h)))
        self.handle = h

    def register_layers(self, key: str, device_id: int,
                        layers: Sequence[tuple[str, HipIPCWrapper | bytes]]
                        ) -> list[tuple[int, int]]:
        """-> [(data_ptr, size_bytes)] per layer, mapped in this process."""
        n = len(layers)
        names = (C.c_char_p * max(n, 1))(*[name.encode() for name, _ in layers])
        recs = (_lib.PfIpcTensor * max(n, 1))()
        for i, (_name, w) in enumerate(layers):
            if isinstance(w, (bytes, bytearray)):
                w = HipIPCWrapper.from_bytes(bytes(w))
            recs[i] = w.c_record()
        ptrs = (C.c_uint64 * max(n, 1))()
        sizes = (C.c_uint64 * max(n, 1))()
        check(self._lib.pf_registry_register_layers(self.handle, key.encode(), device_id, n, names,
                                                    recs, ptrs, sizes))
        return [(ptrs[i], sizes[i]) for i in range(n)]

    def drop_context(self, key: str) -> int:
        return self._lib.pf_registry_drop_context(self.handle, key.encode())

    def drop_instance(self, instance_id: str) -> int:
        return self._lib.pf_registry_drop_instance(self.handle, instance_id.encode())

    def clear(self) -> int:
        return self._lib.pf_registry_clear(self.handle)

    def __len__(self) -> int:
        return self._lib.pf_registry_context_count(self.handle)

    def close(self) -> None:
        if self.handle is not None:
            self._lib.pf_registry_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def register_context_batch(engine, registry: TensorRegistry, instance_id: str, namespace: str,
                           device_id: int, tp_rank: int, pp_rank: int, tp_size: int,
                           world_size: int, layer_names: Sequence[str],
                           wrappers: Sequence[HipIPCWrapper | bytes], num_blocks: Sequence[int],
                           bytes_per_block: Sequence[int], kv_stride_bytes: Sequence[int],
                           segments: Sequence[int], transfer_mode: int = 0,
                           page_first: bool = False,
                           layer_group_ids: Sequence[int] | None = None) -> None:
    """The server's RegisterContextBatch handler (service.rs:205-336): open the
    workers' tensors, register the mapped addresses with ``engine``, roll the
    mappings back when the engine refuses."""
    n = len(layer_names)
    arrays = (wrappers, num_blocks, bytes_per_block, kv_stride_bytes, segments)
    if n == 0 or any(len(a) != n for a in arrays):
        raise _lib.InvalidArgument(
            _lib.PF_ERR_INVALID_ARGUMENT,
            f"all layer arrays must have the same non-zero length (got layer_names={n})")
    names = (C.c_char_p * n)(*[nm.encode() for nm in layer_names])
    recs = (_lib.PfIpcTensor * n)()
    for i, w in enumerate(wrappers):
        if isinstance(w, (bytes, bytearray)):
            w = HipIPCWrapper.from_bytes(bytes(w))
        recs[i] = w.c_record()
    u64s = lambda xs: (C.c_uint64 * n)(*[int(x) for x in xs])
    groups = (C.c_uint32 * n)(*[int(g) for g in layer_group_ids]) if layer_group_ids else None
    check(_lib.load().pf_server_register_context_batch(
        engine.handle, registry.handle, instance_id.encode(), namespace.encode(), device_id,
        tp_rank, pp_rank, tp_size, world_size, n, names, recs, u64s(num_blocks),
        u64s(bytes_per_block), u64s(kv_stride_bytes), u64s(segments), groups, transfer_mode,
        int(page_first)))
