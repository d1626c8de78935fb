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


# ---------------------------------------------------------------------------
# Worker-side callers of the path (python/pegaflow/connector/worker.py): how a
# vLLM worker turns its KV tensors into a registration and its save intents
# into per-layer block lists.  In-process forms over PegaEngine; the
# reference sends the same values over gRPC with CUDA-IPC handles.
# ---------------------------------------------------------------------------

def registration_tensor(kv_cache):
    """The tensor that stands for a layer's cache (worker.py:154-176).  A plain
    tensor stands for itself.  A sequence of recurrent-state tensors is one
    page-strided allocation seen through several views: its first view is
    returned after checking that every view starts in the same storage, has the
    same number of blocks and steps from block to block by the same bytes."""
    if not isinstance(kv_cache, (tuple, list)):
        return kv_cache
    views = list(kv_cache)
    if not views or any(not hasattr(v, "untyped_storage") for v in views):
        raise TypeError("KV cache must be a tensor or a non-empty sequence of state tensors")
    head = views[0]
    if head.storage_offset() != 0:
        raise RuntimeError("the first recurrent-state tensor must start at storage offset zero")

    def facts(view):
        return (view.untyped_storage().data_ptr(), view.shape[0],
                view.stride(0) * view.element_size())

    complaints = ("recurrent-state tensors must share one CUDA allocation",
                  "recurrent-state tensors must have the same block count",
                  "recurrent-state tensors must have one common page stride")
    expected = facts(head)
    for view in views[1:]:
        for got, want, complaint in zip(facts(view), expected, complaints):
            if got != want:
                raise RuntimeError(complaint)
    return head


def register_kv_caches(engine, instance_id: str, namespace: str, device_id: int, kv_caches: dict,
                       block_size: int, *, is_mla: bool = False, tp_rank: int = 0,
                       pp_rank: int = 0, tp_size: int = 1, world_size: int = 1,
                       transfer_backend: str | None = None, page_first: bool = False,
                       recurrent_layer_names=(), layer_group_ids=None) -> list[str]:
    """Register exactly the KV caches of this device (worker.py:261-412) with
    an in-process engine.  Returns the registered layer names in order."""
    from .transfer import TransferMode
    if not kv_caches:
        raise RuntimeError("No KV cache layers were selected for registration")
    names, ptrs, sizes, num_blocks, bytes_per_block, kv_strides, segments = ([] for _ in range(7))
    for layer_name, kv_cache in kv_caches.items():
        recurrent = layer_name in recurrent_layer_names or isinstance(kv_cache, (tuple, list))
        tensor = registration_tensor(kv_cache)
        assert tensor.storage_offset() == 0, f"KV cache for {layer_name} must have zero storage offset"
        reg = infer_kv_cache_registration(tensor, block_size, is_mla=is_mla,
                                          is_recurrent_state=recurrent)
        names.append(layer_name)
        ptrs.append(tensor.data_ptr())
        sizes.append(tensor.untyped_storage().nbytes())
        num_blocks.append(reg.num_blocks)
        bytes_per_block.append(reg.bytes_per_block)
        kv_strides.append(reg.kv_stride_bytes)
        segments.append(reg.segments)
    mode = TransferMode.from_name(resolve_transfer_backend(is_mla, transfer_backend))
    engine.register_context_layer_batch(
        instance_id, namespace, device_id, tp_rank, pp_rank, tp_size, world_size, names, ptrs,
        sizes, num_blocks, bytes_per_block, kv_strides, segments, transfer_mode=mode,
        page_first=page_first, layer_group_ids=layer_group_ids)
    return names


def block_shard(block_ids, block_hashes, tp_rank: int, tp_size: int):
    """The (block ids, hashes) one rank saves under page-first: the stripe
    ``block_id % tp_size == tp_rank`` (worker.py:982-1005); everything when
    there is a single rank.  The stripes of all ranks are disjoint and cover
    every block, so each page is written exactly once."""
    pairs = list(zip(block_ids, block_hashes, strict=True))
    if tp_size > 1:
        pairs = [(block_id, block_hash) for block_id, block_hash in pairs
                 if block_id % tp_size == tp_rank]
    return [block_id for block_id, _ in pairs], [block_hash for _, block_hash in pairs]


def assemble_layer_saves(save_intents, registered_layers, *, layer_to_group=None,
                         page_first: bool = False, stripe: tuple[int, int] | None = None,
                         cross_layer_key: str | None = None):
    """Per-layer save lists of a batch of save intents (worker.py:826-885).

    Each intent carries ``block_ids_by_group`` and ``block_hashes``.  Every
    registered layer (or the one cross-layer pseudo-layer) receives the ids of
    its cache group; the vLLM null block (id 0) is dropped with its hash;
    under page-first with ``stripe = (tp_rank, tp_size)`` each rank keeps its
    block stripe.  Lists of several intents are concatenated per layer.
    Returns ``[(layer_name, block_ids, block_hashes)]`` in first-seen order."""
    layer_to_group = layer_to_group or {}
    saves: dict[str, tuple[list, list]] = {}
    for intent in save_intents:
        if not any(intent.block_ids_by_group):
            continue
        if cross_layer_key is not None:
            target_layers = (cross_layer_key,)
        else:
            assert registered_layers, "KV caches must be registered before submitting save intents"
            target_layers = tuple(registered_layers)
        for layer_name in target_layers:
            group_index = layer_to_group.get(layer_name, 0)
            try:
                block_ids = intent.block_ids_by_group[group_index]
            except IndexError as exc:
                raise RuntimeError(
                    f"save intent is missing cache group {group_index} for {layer_name}") from exc
            block_hashes = intent.block_hashes
            if len(block_ids) != len(block_hashes):
                raise RuntimeError(
                    f"save block/hash count mismatch for {layer_name}: "
                    f"blocks={len(block_ids)} hashes={len(block_hashes)}")
            non_null = [(b, h) for b, h in zip(block_ids, block_hashes, strict=True) if b != 0]
            ids = [b for b, _ in non_null]
            hashes = [h for _, h in non_null]
            if page_first and stripe is not None:
                ids, hashes = block_shard(ids, hashes, stripe[0], stripe[1])
            if not ids:
                continue
            entry = saves.setdefault(layer_name, ([], []))
            entry[0].extend(ids)
            entry[1].extend(hashes)
    return [(name, ids, hashes) for name, (ids, hashes) in saves.items()]


# ---------------------------------------------------------------------------
# Scheduler-side facts that decide what the worker is asked to move
# (python/pegaflow/connector/common.py): the storage namespace, the storage
# group of each cache group, and how a hybrid model's per-group query results
# combine into one resumable prefix.
# ---------------------------------------------------------------------------

def storage_group_ids(group_is_recurrent) -> tuple[int, ...]:
    """Engine storage group of every connector cache group (common.py:405-415):
    attention-like groups share storage group 0, recurrent groups are numbered
    1, 2, ... in cache-group order, wherever the attention group sits."""
    ids, next_recurrent = [], 1
    for recurrent in group_is_recurrent:
        if recurrent:
            ids.append(next_recurrent)
            next_recurrent += 1
        else:
            ids.append(0)
    return tuple(ids)


def reconcile_hybrid_hit(attention_hit_blocks: int, recurrent_hits):
    """One hit for a hybrid (attention + recurrent state) model
    (common.py:252-286).  ``recurrent_hits[g][s]`` = query positions whose
    checkpoint is stored in recurrent group ``g`` on TP shard ``s``.  A position
    is a legal resume point when it lies inside the attention prefix and every
    group holds it on every shard; the hit is the rightmost such position plus
    one block.  Returns ``(hit_blocks, checkpoint, usable_positions)``;
    ``(0, None, frozenset())`` when the prefix cannot be resumed."""
    nothing = (0, None, frozenset())
    if attention_hit_blocks <= 0 or not recurrent_hits:
        return nothing
    shard_sets = [frozenset(p for p in shard if p < attention_hit_blocks)
                  for group in recurrent_hits for shard in group]
    if not shard_sets:
        return nothing
    usable = frozenset.intersection(*shard_sets)
    if not usable:
        return nothing
    checkpoint = max(usable)
    return checkpoint + 1, checkpoint, usable


def derive_namespace(vllm_config, tp_size: int, dcp_world_size: int = 1, pcp_world_size: int = 1,
                     cross_layer_blocks: bool = False) -> str:
    """Storage namespace of a deployment (common.py:519-566): eight hex digits
    of SHA-256 over every setting that changes how a block is laid out in
    storage, so that two incompatible layouts can never answer each other's
    queries.  ``vllm_config`` is vLLM's config object (only attributes are read)."""
    import hashlib
    model, cache = vllm_config.model_config, vllm_config.cache_config
    extra = getattr(vllm_config, "additional_config", None) or {}
    factors = {
        "model": model.model,
        "dtype": str(model.dtype),
        "tp_size": tp_size,
        "pp_size": vllm_config.parallel_config.pipeline_parallel_size,
        "num_kv_heads": model.get_total_num_kv_heads(),
        "head_size": model.get_head_size(),
        "num_hidden_layers": model.get_total_num_hidden_layers(),
        "cache_dtype": str(cache.cache_dtype),
        "is_hma_enabled": not vllm_config.scheduler_config.disable_hybrid_kv_cache_manager,
        "dcp_world_size": dcp_world_size,
        "pcp_world_size": pcp_world_size,
        "cross_layer_blocks": cross_layer_blocks,
        "mla_layer_split_kv_cache": bool(extra.get("mla_layer_split_kv_cache", False)),
    }
    return hashlib.sha256(str(sorted(factors.items())).encode()).hexdigest()[:8]
