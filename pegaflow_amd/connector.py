"""Connector-side pure functions that define what a vLLM KV tensor means to
the transfer path.  Mirrors ``_infer_kv_cache_registration``
(python/pegaflow/connector/worker.py:65-151) and ``resolve_transfer_backend``
(python/pegaflow/connector/common.py:577-594) of the reference: same names,
argument meaning and error messages.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Literal

KVCacheLayoutName = Literal["KV-first", "blocks-first"]


@dataclass(frozen=True)
class KVCacheRegistrationInfo:
    layout: KVCacheLayoutName
    num_blocks: int
    bytes_per_block: int
    kv_stride_bytes: int
    segments: int
    physical_blocks_per_logical_block: int


def infer_kv_cache_registration(
    kv_cache,
    logical_block_size: int,
    *,
    is_mla: bool = False,
    is_recurrent_state: bool = False,
) -> KVCacheRegistrationInfo:
    """Registration parameters of one KV cache tensor.

    ``kv_cache`` needs ``.shape``, ``.stride()`` (in elements) and
    ``.element_size()``.  Non-MLA tensors whose first dimension is 2 are
    K/V-first with two segments; everything else is blocks-first with one.
    MLA kernels may use a smaller block than the scheduler: then
    ``logical/physical`` physical rows form one registered block.
    """
    shape = tuple(kv_cache.shape)
    stride = tuple(kv_cache.stride())
    element_size = kv_cache.element_size()

    if logical_block_size <= 0:
        raise ValueError(f"logical block size must be > 0, got {logical_block_size}")

    if is_recurrent_state or not is_mla:
        kv_first = (not is_recurrent_state) and len(shape) >= 2 and shape[0] == 2
        block_dim = 1 if kv_first else 0
        num_blocks = shape[block_dim]
        bytes_per_block = stride[block_dim] * element_size
        if num_blocks <= 0:
            raise ValueError(f"physical block count must be > 0, got {num_blocks}")
        if bytes_per_block == 0:
            raise ValueError(f"Invalid bytes_per_block: shape={shape} stride={stride}")
        return KVCacheRegistrationInfo(
            layout="KV-first" if kv_first else "blocks-first",
            num_blocks=num_blocks,
            bytes_per_block=bytes_per_block,
            kv_stride_bytes=stride[0] * element_size if kv_first else 0,
            segments=2 if kv_first else 1,
            physical_blocks_per_logical_block=1,
        )

    physical_num_blocks = shape[0]
    physical_block_size = shape[1] if len(shape) >= 2 else logical_block_size
    if physical_num_blocks <= 0:
        raise ValueError(f"physical block count must be > 0, got {physical_num_blocks}")
    if physical_block_size <= 0:
        raise ValueError(f"physical block size must be > 0, got {physical_block_size}")
    if logical_block_size % physical_block_size != 0:
        raise ValueError(
            "logical block size must be a multiple of physical block size "
            f"(logical={logical_block_size}, physical={physical_block_size})"
        )
    ratio = logical_block_size // physical_block_size
    if physical_num_blocks % ratio != 0:
        raise ValueError(
            "physical block count must be divisible by physical/logical split ratio "
            f"(physical_blocks={physical_num_blocks}, ratio={ratio})"
        )
    bytes_per_block = stride[0] * element_size * ratio
    if bytes_per_block == 0:
        raise ValueError(f"Invalid bytes_per_block: shape={shape} stride={stride}")
    return KVCacheRegistrationInfo(
        layout="blocks-first",
        num_blocks=physical_num_blocks // ratio,
        bytes_per_block=bytes_per_block,
        kv_stride_bytes=0,
        segments=1,
        physical_blocks_per_logical_block=ratio,
    )


TRANSFER_BACKENDS = ("direct", "kernel")


def resolve_transfer_backend(is_mla: bool, override: str | None) -> str:
    """``kernel`` for MLA, ``direct`` otherwise; a given override wins and an
    unknown one is rejected."""
    if override is None:
        return "kernel" if is_mla else "direct"
    normalized = override.strip().lower()
    if normalized not in TRANSFER_BACKENDS:
        allowed = ", ".join(TRANSFER_BACKENDS)
        raise ValueError(
            f"Unsupported pegaflow.transfer_backend {override!r}; expected one of: {allowed}"
        )
    return normalized
