"""``KVCacheLayout`` over the C ABI (pegaflow-core/src/layout.rs:13-286)."""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

from . import _lib
from ._lib import check


@dataclass(frozen=True)
class BlockCopy:
    addr: int
    bytes: int


class KVCacheLayout:
    """One layer's KV cache: ``addr = data_ptr + block*block_stride + seg*kv_stride``.

    ``segment_bytes`` is ONE segment (K or V alone for split layouts).
    Raises ``InvalidArgument`` with the reference's messages on a bad shape.
    """

    def __init__(self, data_ptr: int, size_bytes: int, num_blocks: int, segment_bytes: int,
                 kv_stride_bytes: int, segments: int):
        self._lib = _lib.load()
        self.c = _lib.PfKvLayout()
        check(self._lib.pf_layout_new(data_ptr, size_bytes, num_blocks, segment_bytes,
                                      kv_stride_bytes, segments, C.byref(self.c)))

    def with_block_stride(self, stride: int) -> "KVCacheLayout":
        check(self._lib.pf_layout_with_block_stride(C.byref(self.c), stride))
        return self

    def with_ssd_padding(self, alignment: int) -> "KVCacheLayout":
        check(self._lib.pf_layout_with_ssd_padding(C.byref(self.c), alignment))
        return self

    def block_copies(self, block_idx: int) -> list[BlockCopy]:
        out = (_lib.PfBlockCopy * 2)()
        n = C.c_uint32()
        check(self._lib.pf_layout_block_copies(C.byref(self.c), block_idx, out, C.byref(n)))
        return [BlockCopy(out[i].addr, out[i].bytes) for i in range(n.value)]

    @property
    def num_blocks(self) -> int:
        return self.c.num_blocks

    @property
    def is_split(self) -> bool:
        return bool(self.c.split)

    @property
    def segment_bytes(self) -> int:
        return self.c.segment_bytes

    @property
    def block_bytes(self) -> int:
        return self._lib.pf_layout_block_bytes(C.byref(self.c))

    @property
    def padded_segment_bytes(self) -> int:
        return self.c.padded_segment_bytes

    @property
    def padded_block_bytes(self) -> int:
        return self._lib.pf_layout_padded_block_bytes(C.byref(self.c))

    @property
    def block_stride_bytes(self) -> int:
        return self.c.block_stride_bytes

    @property
    def fragment_bytes(self) -> int:
        """Bytes of one copied range: a segment when split, else the block."""
        return self.segment_bytes if self.is_split else self.block_bytes

    @property
    def host_stride(self) -> int:
        """Stride of one fragment in the layer-first batch host image
        (pegaflow-core/src/offload.rs:472-499)."""
        return self.padded_segment_bytes if self.is_split else self.padded_block_bytes
