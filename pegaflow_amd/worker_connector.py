"""Worker side of the KV connector: what calls the transfer path inside a vLLM
worker process (python/pegaflow/connector/worker.py:179-1050).

Per scheduler step the worker receives a ``PegaConnectorMetadata``:
``load_intents`` (leases pinned by the scheduler plus destination block ids)
become ONE load task whose completion is polled through a ``LoadState``;
``save_intents`` become a save task that a background thread hands to the
engine, several queued tasks batched into one engine call.  vLLM learns about
completion through ``get_finished`` and about failed loads through
``get_block_ids_with_load_errors``; ``handle_preemptions`` blocks until every
save task of a request that is about to lose its blocks has finished.

The engine is reached through a client object with three calls --
``save(instance_id, tp_rank, pp_rank, device_id, [(layer, ids, hashes)])``,
``load(instance_id, tp_rank, device_id, load_state_shm, layer_groups, loads)``,
both returning ``(ok, message)``, and ``release(lease)`` -- which is the gRPC
client in the reference and ``InProcessEngineClient`` (over ``PegaEngine``) here.
"""

from __future__ import annotations

import logging
import queue
import threading
import time
from dataclasses import dataclass, field
from typing import Any, Iterable, Sequence

from .connector import assemble_layer_saves, register_kv_caches, storage_group_ids
from .engine import LayerSave, LoadState, PegaEngine

logger = logging.getLogger("pegaflow_amd.connector")

CROSS_LAYER_KEY = "ALL_LAYERS"   # worker.py:414-420: one pseudo-layer holding every layer


# ---------------------------------------------------------------------------
# What the scheduler side sends (connector/common.py:220-294,440-462)
# ---------------------------------------------------------------------------

@dataclass(frozen=True)
class SaveIntent:
    block_ids_by_group: tuple[tuple[int, ...], ...]
    block_hashes: tuple[bytes, ...]


@dataclass(frozen=True)
class RecurrentLoadHold:
    """Membership leases over the recurrent checkpoints of a hybrid load:
    ``leases[g][shard]``, ``hit_positions[g][shard]`` = query position of every
    leased block, ``checkpoint`` = the query position whose state is loaded."""
    leases: tuple[tuple[bytes, ...], ...]
    hit_positions: tuple[tuple[tuple[int, ...], ...], ...]
    checkpoint: int


@dataclass(frozen=True)
class LoadIntent:
    block_ids_by_group: tuple[tuple[int | None, ...], ...]
    leases: tuple[bytes, ...]
    num_tokens: int
    recurrent_hold: RecurrentLoadHold | None = None


class PegaConnectorMetadata:
    def __init__(self, load_intents=None, save_intents=None, ready_save_intents=None,
                 preempted_req_ids=None):
        self.load_intents: dict[str, LoadIntent] = load_intents or {}
        self.save_intents: dict[str, SaveIntent] = save_intents or {}
        self.ready_save_intents: dict[str, SaveIntent] = ready_save_intents or {}
        self.preempted_req_ids: set[str] = preempted_req_ids or set()


@dataclass(frozen=True)
class CacheGroups:
    """vLLM's cache groups as the worker needs them: which layers form which
    group and which groups hold recurrent state (common.py:296-436 derives the
    same facts from vLLM's KVCacheConfig)."""
    layer_names: tuple[tuple[str, ...], ...] = ((),)
    recurrent_group_indices: frozenset = frozenset()

    @property
    def group_count(self) -> int:
        return len(self.layer_names)

    @property
    def has_recurrent_state(self) -> bool:
        return bool(self.recurrent_group_indices)

    @property
    def storage_group_ids(self) -> tuple[int, ...]:
        return storage_group_ids(index in self.recurrent_group_indices
                                 for index in range(self.group_count))

    def storage_group_of(self, group_index: int) -> int:
        return self.storage_group_ids[group_index]

    @property
    def hash_group_index(self) -> int:
        """The attention group, whose block hashes key the whole request."""
        return next(index for index in range(self.group_count)
                    if index not in self.recurrent_group_indices)

    def layer_to_group(self) -> dict[str, int]:
        owner: dict[str, int] = {}
        for index, names in enumerate(self.layer_names):
            for name in names:
                if name in owner:
                    raise RuntimeError(f"KV cache layer belongs to multiple groups: {name}")
                owner[name] = index
        return owner


@dataclass(frozen=True)
class ConnectorContext:
    """The part of connector/common.py:120-218 the worker reads.  One GPU per
    engine here, so there is one TP shard and no rank remapping."""
    instance_id: str
    namespace: str
    block_size: int
    tp_size: int
    world_size: int
    tp_rank: int
    device_id: int
    engine_client: Any
    state_manager: Any = None
    is_mla: bool = False
    pp_rank: int = 0
    pp_size: int = 1
    dcp_world_size: int = 1
    transfer_backend: str | None = None
    tp_shard_count: int = 1
    tp_shard_index: int = 0

    @property
    def effective_tp_rank(self) -> int:
        # MLA caches are identical on every TP rank and stored once.
        return 0 if self.is_mla else self.tp_rank


class InProcessEngineClient:
    """The engine-client calls the worker makes, answered by a ``PegaEngine`` in
    this process.  Leases travel as 8-byte little-endian tokens."""

    def __init__(self, engine: PegaEngine):
        self.engine = engine
        self._tasks: list = []     # load tasks kept until they settle
        self._lock = threading.Lock()

    @staticmethod
    def lease_token(lease: int) -> bytes:
        return int(lease).to_bytes(8, "little")

    def query(self, instance_id: str, hashes: Sequence[bytes]) -> tuple[int, bytes]:
        hits, lease = self.engine.query_prefix(instance_id, hashes)
        return hits, (self.lease_token(lease) if lease else b"")

    def save(self, instance_id, tp_rank, pp_rank, device_id, saves) -> tuple[bool, str]:
        try:
            self.engine.batch_save_kv_blocks(
                instance_id, tp_rank, pp_rank, device_id,
                [LayerSave(name, list(ids), list(hashes)) for name, ids, hashes in saves])
        except Exception as exc:            # the RPC form reports (False, message)
            return False, str(exc)
        return True, ""

    def load(self, instance_id, tp_rank, device_id, load_state_shm, layer_groups,
             loads) -> tuple[bool, str]:
        state = LoadState(attach_to=load_state_shm)
        try:
            task = self.engine.batch_load_multi(
                instance_id, tp_rank, device_id, layer_groups,
                [(int.from_bytes(lease, "little"), groups) for lease, groups in loads], state)
        except Exception as exc:
            return False, str(exc)
        finally:
            state.close()
        with self._lock:
            self._tasks = [t for t in self._tasks if not self._settled(t)] + [task]
        return True, ""

    @staticmethod
    def _settled(task) -> bool:
        try:
            return task.wait(0).done
        except Exception:      # a failed load has settled too; its LoadState says so
            return True

    def release(self, lease: bytes) -> None:
        self.engine.release_query_lease(int.from_bytes(lease, "little"))

    def unregister_context(self, instance_id: str) -> tuple[bool, str]:
        try:
            self.engine.unregister_instance(instance_id)
        except Exception as exc:
            return False, str(exc)
        return True, ""


# ---------------------------------------------------------------------------
# Book-keeping
# ---------------------------------------------------------------------------

class _SaveLedger:
    """How many save tasks each request still has in flight.  A request counts
    as saved when its count returns to zero; a later task for the same request
    opens it again (worker.py:782-796,931-950)."""

    def __init__(self) -> None:
        self.lock = threading.Lock()
        self.outstanding: dict[str, int] = {}
        self.done_events: dict[str, threading.Event] = {}
        self.saved: set[str] = set()          # settled, not yet reported to vLLM
        self.released: set[str] = set()       # vLLM finished them while saves were pending

    def open(self, request_ids: Iterable[str]) -> None:
        with self.lock:
            for rid in request_ids:
                count = self.outstanding.get(rid, 0)
                if count == 0:
                    self.saved.discard(rid)
                    self.done_events[rid] = threading.Event()
                self.outstanding[rid] = count + 1

    def close(self, request_ids: Iterable[str]) -> list[str]:
        settled = []
        with self.lock:
            for rid in request_ids:
                count = self.outstanding.get(rid)
                if count is None:
                    continue
                if count > 1:
                    self.outstanding[rid] = count - 1
                    continue
                del self.outstanding[rid]
                self.saved.add(rid)
                settled.append(rid)
                event = self.done_events.pop(rid, None)
                if event is not None:
                    event.set()
        return settled

    def report(self, finished_req_ids: set[str]) -> set[str] | None:
        """Requests vLLM may now free: saved, and finished either now or in an
        earlier step (worker.py:426-437)."""
        with self.lock:
            self.released |= finished_req_ids & self.outstanding.keys()
            out = (self.saved & self.released) | (self.saved & finished_req_ids)
            self.saved -= out
            self.released -= out
        return out or None

    def events_of(self, request_ids: Iterable[str]) -> list[tuple[str, threading.Event]]:
        with self.lock:
            return [(rid, self.done_events[rid]) for rid in request_ids if rid in self.done_events]


@dataclass
class _LoadInFlight:
    state: Any                      # LoadState-like: get(), close()
    request_ids: set[str]
    started: float
    block_ids: list[int] = field(default_factory=list)


@dataclass
class _SaveTask:
    intents: dict[str, SaveIntent]
    request_ids: list[str]


# ---------------------------------------------------------------------------
# The worker connector
# ---------------------------------------------------------------------------

class WorkerConnector:
    # An in-flight load that has not settled after this long is reported to
    # vLLM as failed (worker.py:182-187).
    LOAD_TIMEOUT_SECONDS: int = 120

    def __init__(self, context: ConnectorContext, cache_groups: CacheGroups | None = None, *,
                 load_state_factory=LoadState, start_save_thread: bool = True,
                 device_synchronize=None):
        self._ctx = context
        self._cache_groups = cache_groups or CacheGroups()
        self._layer_to_group = self._cache_groups.layer_to_group()
        self._new_load_state = load_state_factory
        self._device_synchronize = device_synchronize
        self._registered_layers: list[str] = []
        self._page_first = False
        self._cross_layer_mode = False
        self._cross_layer_key = CROSS_LAYER_KEY
        self._current_metadata: PegaConnectorMetadata | None = None

        self._saves = _SaveLedger()
        self._save_queue: queue.Queue = queue.Queue()
        self._save_thread = threading.Thread(target=self._save_worker, daemon=True,
                                             name="PegaSaveWorker")
        self._save_thread_started = start_save_thread
        if start_save_thread:
            self._save_thread.start()

        self._load_lock = threading.Lock()
        self._loads: dict[str, _LoadInFlight] = {}       # shm name -> load
        self._failed_load_block_ids: set[int] = set()
        self._failed_load_reqs: set[str] = set()

    # ---- registration ---------------------------------------------------
    def register_kv_caches(self, kv_caches: dict[str, Any]) -> None:
        """worker.py:261-412, for an engine in this process."""
        client = self._ctx.engine_client
        if not isinstance(client, InProcessEngineClient):
            raise RuntimeError("register_kv_caches needs an in-process engine client")
        ctx = self._ctx
        self._page_first = self._use_page_first()
        group_ids = None
        if self._cache_groups.group_count > 1:
            strangers = [name for name in kv_caches if name not in self._layer_to_group]
            if strangers:
                raise RuntimeError(
                    f"HMA registration contains layers outside cache groups: {strangers[:8]}")
            # The engine is told the STORAGE group of each layer (attention 0,
            # recurrent groups 1, 2, ...), which is not the cache-group index
            # when a recurrent group comes first (worker.py:364-367).
            storage_ids = self._cache_groups.storage_group_ids
            group_ids = [storage_ids[self._layer_to_group[name]] for name in kv_caches]
        recurrent = {name for index in self._cache_groups.recurrent_group_indices
                     for name in self._cache_groups.layer_names[index]}
        self._registered_layers = register_kv_caches(
            client.engine, ctx.instance_id, ctx.namespace, ctx.device_id, kv_caches,
            ctx.block_size, is_mla=ctx.is_mla, tp_rank=ctx.effective_tp_rank, pp_rank=ctx.pp_rank,
            tp_size=1 if ctx.is_mla else ctx.tp_size, world_size=ctx.world_size,
            transfer_backend=ctx.transfer_backend, page_first=self._page_first,
            recurrent_layer_names=recurrent, layer_group_ids=group_ids)

    def register_cross_layers_kv_cache(self, kv_cache, attn_backend=None) -> None:
        """One tensor holds every layer of a block: it is registered as a single
        pseudo-layer, named per pipeline stage when there are several
        (worker.py:414-420)."""
        self._cross_layer_mode = True
        self._cross_layer_key = (f"{CROSS_LAYER_KEY}_pp{self._ctx.pp_rank}"
                                 if self._ctx.pp_size > 1 else CROSS_LAYER_KEY)
        self.register_kv_caches({self._cross_layer_key: kv_cache})

    def _use_page_first(self) -> bool:
        # worker.py:967-980: only when one worker writes every layer of a page.
        ctx = self._ctx
        return (ctx.is_mla and self._cache_groups.group_count == 1 and ctx.dcp_world_size == 1
                and ctx.pp_size == 1)

    def shutdown(self) -> None:
        if self._registered_layers and self._ctx.tp_rank == 0:
            unregister = getattr(self._ctx.engine_client, "unregister_context", None)
            if unregister is not None:
                ok, message = unregister(self._ctx.instance_id)
                if not ok:
                    logger.warning("unregister context failed: %s", message)
        self._registered_layers = []
        if self._save_thread_started:
            self._save_queue.put(None)
            self._save_thread.join()
            self._save_thread_started = False

    # ---- loads ----------------------------------------------------------
    def start_load_kv(self, metadata: PegaConnectorMetadata, forward_context=None) -> None:
        self._current_metadata = metadata
        if metadata.ready_save_intents:
            if not self._cache_groups.has_recurrent_state:
                raise RuntimeError("ready save intents are only valid for HMA")
            self._process_save_batch([self._make_save_task(metadata.ready_save_intents)])
        if not metadata.load_intents:
            return

        started = time.perf_counter()
        loads, wanted_blocks, request_ids = self._plan_loads(metadata.load_intents)
        if not wanted_blocks:
            return
        layer_groups = self._load_layer_groups()
        if not any(layer_groups):
            return

        state = self._new_load_state()
        shm_name = state.shm_name
        hybrid = self._cache_groups.group_count > 1
        failure = None
        try:
            ok, message = self._ctx.engine_client.load(
                self._ctx.instance_id, self._ctx.effective_tp_rank, self._ctx.device_id, shm_name,
                layer_groups, loads)
            if not ok:
                failure = f"load rpc failed: {message}"
        except Exception as exc:
            failure = f"load rpc exception: {exc}"
        if failure is not None:
            logger.error("%s (reqs=%s blocks=%d)", failure, request_ids, len(wanted_blocks))
            state.close()
            self._release_load_leases(loads)
            self._mark_unavailable(failure)
            if hybrid:
                # vLLM cannot recompute part of a hybrid load (worker.py:655-659).
                raise RuntimeError("PegaFlow HMA load failed; vLLM cannot recover failed loads "
                                   f"for multiple cache groups: {failure}")
            with self._load_lock:
                self._failed_load_reqs.update(request_ids)
                self._failed_load_block_ids.update(wanted_blocks)
            return
        with self._load_lock:
            self._loads[shm_name] = _LoadInFlight(state, set(request_ids), started, wanted_blocks)

    def _plan_loads(self, load_intents: dict[str, LoadIntent]):
        """[(lease, destination ids per cache group)], every destination id, request ids
        (worker.py:572-619)."""
        ctx = self._ctx
        recurrent_groups = sorted(self._cache_groups.recurrent_group_indices)
        loads: list[tuple[bytes, list[list[int | None]]]] = []
        wanted: list[int] = []
        request_ids: list[str] = []
        for req_id, intent in load_intents.items():
            if len(intent.leases) != ctx.tp_shard_count:
                raise RuntimeError(f"load intent has {len(intent.leases)} TP shard leases; "
                                   f"expected {ctx.tp_shard_count}")
            per_group = [list(ids) for ids in intent.block_ids_by_group]
            hold = intent.recurrent_hold
            if hold is not None:
                # The prefix lease covers the attention blocks only; recurrent
                # destinations ride on the membership leases below.
                for g in recurrent_groups:
                    per_group[g] = [None] * len(per_group[g])
            for ids in per_group:
                wanted.extend(b for b in ids if b is not None)
            loads.append((intent.leases[ctx.tp_shard_index], per_group))
            if hold is not None:
                for slot, g in enumerate(recurrent_groups):
                    positions = hold.hit_positions[slot][ctx.tp_shard_index]
                    if hold.checkpoint not in positions:
                        raise RuntimeError(
                            f"req {req_id}: recurrent group {g} shard {ctx.tp_shard_index} "
                            f"lease has no checkpoint at query position {hold.checkpoint}")
                    target = next((b for b in reversed(intent.block_ids_by_group[g])
                                   if b is not None), None)
                    if target is None:
                        raise RuntimeError(f"req {req_id}: no recurrent destination block in "
                                           f"group {g} for checkpoint {hold.checkpoint}")
                    vectors: list[list[int | None]] = [
                        [None] * len(positions) for _ in range(self._cache_groups.group_count)]
                    vectors[g][positions.index(hold.checkpoint)] = target
                    loads.append((hold.leases[slot][ctx.tp_shard_index], vectors))
                    wanted.append(target)
            request_ids.append(req_id)
        return loads, wanted, request_ids

    def _load_layer_groups(self) -> list[list[str]]:
        if self._cross_layer_mode:
            return [[self._cross_layer_key]]
        assert self._registered_layers, "KV caches must be registered before submitting load intents"
        groups: list[list[str]] = [[] for _ in range(self._cache_groups.group_count)]
        for name in self._registered_layers:
            groups[self._layer_to_group.get(name, 0)].append(name)
        return groups

    def _release_load_leases(self, loads) -> None:
        seen: set[bytes] = set()
        for lease, _ in loads:
            if not lease or lease in seen:
                continue
            seen.add(lease)
            try:
                self._ctx.engine_client.release(lease)
            except Exception:
                logger.exception("releasing a lease after a failed load")

    def _mark_unavailable(self, reason: str) -> None:
        if self._ctx.state_manager is not None:
            self._ctx.state_manager.mark_unavailable(reason)

    def wait_for_layer_load(self, layer_name: str) -> None:
        """Loads complete as a whole and are reported by get_finished (worker.py:712-713)."""

    def get_block_ids_with_load_errors(self) -> set[int]:
        with self._load_lock:
            failed, self._failed_load_block_ids = self._failed_load_block_ids, set()
        return failed

    # ---- saves ----------------------------------------------------------
    def save_kv_layer(self, metadata=None, layer_name=None, kv_layer=None, attn_metadata=None,
                      **kwargs) -> None:
        """Saves are driven by the step's metadata in wait_for_save, not per layer
        (worker.py:755-765)."""

    def wait_for_save(self) -> None:
        metadata, self._current_metadata = self._current_metadata, None
        if metadata is None or not metadata.save_intents:
            return
        task = self._make_save_task(metadata.save_intents)
        if self._cache_groups.has_recurrent_state:
            # The only live block of a recurrent state may be rewritten by the
            # next step: finish the copy before returning (worker.py:774-778).
            self._process_save_batch([task])
        else:
            self._save_queue.put(task)

    def _make_save_task(self, intents: dict[str, SaveIntent]) -> _SaveTask:
        request_ids = list(intents)
        self._saves.open(request_ids)
        return _SaveTask(dict(intents), request_ids)

    def _save_worker(self) -> None:
        while True:
            task = self._save_queue.get()
            if task is None:
                return
            batch, stop = [task], False
            while True:       # everything already queued joins this engine call
                try:
                    more = self._save_queue.get_nowait()
                except queue.Empty:
                    break
                if more is None:
                    stop = True
                    break
                batch.append(more)
            self._process_save_batch(batch)
            if stop:
                return

    def _process_save_batch(self, batch: list[_SaveTask]) -> None:
        request_ids = [rid for task in batch for rid in task.request_ids]
        try:
            ctx = self._ctx
            saves = assemble_layer_saves(
                [intent for task in batch for intent in task.intents.values()],
                self._registered_layers, layer_to_group=self._layer_to_group,
                page_first=self._page_first, stripe=(ctx.tp_rank, ctx.tp_size),
                cross_layer_key=self._cross_layer_key if self._cross_layer_mode else None)
            if saves:
                # The attention kernels that fill these blocks run asynchronously:
                # wait for the device before the engine reads the cache.
                if self._device_synchronize is not None:
                    self._device_synchronize()
                try:
                    ok, message = ctx.engine_client.save(ctx.instance_id, ctx.effective_tp_rank,
                                                         ctx.pp_rank, ctx.device_id, saves)
                    if not ok:
                        logger.error("save batch failed: %s (continuing without save)", message)
                except Exception as exc:
                    logger.error("save rpc exception: %s (continuing without save)", exc)
        finally:
            # The request's blocks become reusable whether or not the save worked.
            self._complete_save_requests(request_ids)

    def _complete_save_requests(self, request_ids: list[str]) -> None:
        for rid in self._saves.close(request_ids):
            logger.debug("request %s save completed", rid)

    def handle_preemptions(self, preempted_req_ids: set[str] | None) -> None:
        """Called before the blocks of preempted requests are handed out again:
        returns once none of their save tasks is still reading them."""
        if not preempted_req_ids:
            return
        for _rid, event in self._saves.events_of(preempted_req_ids):
            event.wait()

    # ---- completion -----------------------------------------------------
    def get_finished(self, finished_req_ids: set[str]) -> tuple[set[str] | None, set[str] | None]:
        finished_sending = self._saves.report(set(finished_req_ids))

        hybrid = self._cache_groups.group_count > 1
        hybrid_failure: str | None = None
        timed_out = False
        done_reqs: set[str] = set()
        now = time.perf_counter()
        with self._load_lock:
            for shm_name in list(self._loads):
                load = self._loads[shm_name]
                value = load.state.get()
                if value != 0:
                    if value < 0:
                        logger.error("async load failed: reqs=%s state=%d", load.request_ids, value)
                        if hybrid:
                            hybrid_failure = (f"async load failed for requests "
                                              f"{sorted(load.request_ids)}: state={value}")
                        else:
                            self._failed_load_block_ids.update(load.block_ids)
                elif now - load.started > self.LOAD_TIMEOUT_SECONDS:
                    elapsed = now - load.started
                    logger.error("load timeout: reqs=%s elapsed=%.1fs blocks=%d", load.request_ids,
                                 elapsed, len(load.block_ids))
                    if hybrid:
                        hybrid_failure = (f"load timed out for requests "
                                          f"{sorted(load.request_ids)} after {elapsed:.1f}s")
                    else:
                        self._failed_load_block_ids.update(load.block_ids)
                    timed_out = True
                else:
                    continue
                done_reqs |= load.request_ids
                load.state.close()
                del self._loads[shm_name]
            if self._failed_load_reqs:
                done_reqs |= self._failed_load_reqs
                self._failed_load_reqs = set()
        if timed_out:
            self._mark_unavailable("load timeout")
        if hybrid_failure is not None:
            self._mark_unavailable(hybrid_failure)
            raise RuntimeError("PegaFlow HMA load failed; vLLM cannot recover failed loads for "
                               f"multiple cache groups: {hybrid_failure}")
        return finished_sending, (done_reqs or None)


__all__ = ["CacheGroups", "ConnectorContext", "InProcessEngineClient", "LoadIntent",
           "PegaConnectorMetadata", "RecurrentLoadHold", "SaveIntent", "WorkerConnector"]
