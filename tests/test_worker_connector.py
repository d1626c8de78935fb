"""Worker-side connector logic (pegaflow_amd/worker_connector.py) against the
behaviour the reference's tests pin: python/tests/test_connector_save_lifecycle.py
(save tasks per request, reopening, preemption) and
python/tests/test_connector_fault_tolerance.py (load failures, time-outs,
hybrid-model failures, layer names).  The engine is a fake client here; the
GPU test in test_gpu_connector.py runs the same class over a real engine."""

import threading
from unittest.mock import MagicMock

import pytest

import pegaflow_amd.worker_connector as wc
from pegaflow_amd.worker_connector import (CacheGroups, ConnectorContext, LoadIntent,
                                           PegaConnectorMetadata, RecurrentLoadHold, SaveIntent,
                                           WorkerConnector)


class FakeLoadState:
    count = 0

    def __init__(self):
        FakeLoadState.count += 1
        self.shm_name = f"/fake_load_state_{FakeLoadState.count}"
        self.value = 0
        self.closed = False

    def get(self):
        return self.value

    def close(self):
        self.closed = True


class FakeEngineClient:
    def __init__(self):
        self.fail_load_with_ok_false = False
        self.fail_load_with_exception = None
        self.load_calls = []
        self.release_calls = []
        self.save_calls = []
        self.save_result = (True, "")

    def load(self, instance_id, tp_rank, device_id, load_state_shm, layer_groups, loads):
        block_ids = [b for _, groups in loads for ids in groups for b in ids]
        self.load_calls.append((instance_id, tp_rank, device_id, load_state_shm,
                                [list(g) for g in layer_groups], block_ids, list(loads)))
        if self.fail_load_with_exception is not None:
            raise self.fail_load_with_exception
        if self.fail_load_with_ok_false:
            return False, "simulated load failure"
        return True, "ok"

    def save(self, instance_id, tp_rank, pp_rank, device_id, saves):
        self.save_calls.append([(n, list(i), list(h)) for n, i, h in saves])
        return self.save_result

    def release(self, lease):
        self.release_calls.append(lease)


def make_worker(cache_groups=None, start_save_thread=False, **ctx):
    client = FakeEngineClient()
    state_manager = MagicMock()
    fields = dict(instance_id="test_instance", namespace="ns", block_size=16, tp_size=1,
                  world_size=1, tp_rank=0, device_id=0, engine_client=client,
                  state_manager=state_manager)
    fields.update(ctx)
    worker = WorkerConnector(ConnectorContext(**fields), cache_groups,
                             load_state_factory=FakeLoadState,
                             start_save_thread=start_save_thread)
    worker._cross_layer_mode = True       # one pseudo-layer unless a test registers layers
    return worker, client, state_manager


def enqueue_save(worker, block_id=1, block_hash=b"hash"):
    worker._current_metadata = PegaConnectorMetadata(save_intents={
        "request": SaveIntent(block_ids_by_group=((block_id,),), block_hashes=(block_hash,))})
    worker.wait_for_save()
    return worker._saves.done_events["request"]


def complete_next_save(worker):
    worker._complete_save_requests(worker._save_queue.get_nowait().request_ids)


def process_next_save(worker):
    worker._process_save_batch([worker._save_queue.get_nowait()])


# ---- save lifecycle (test_connector_save_lifecycle.py:66-197) ---------------

def test_blocks_are_not_reused_until_every_save_task_completes():
    worker, client, _ = make_worker()
    worker._cross_layer_mode = False
    worker._registered_layers = ["layer"]
    gpu_blocks = {1: b"first request block", 2: b"second request block"}
    stored = {}

    def save(_instance, _tp, _pp, _dev, saves):
        for _layer, ids, hashes in saves:
            for block_id, block_hash in zip(ids, hashes, strict=True):
                stored[block_hash] = gpu_blocks[block_id]
        return True, ""

    client.save = save
    enqueue_save(worker, 1, b"first hash")
    enqueue_save(worker, 2, b"second hash")
    process_next_save(worker)
    finished_sending, _ = worker.get_finished({"request"})
    if finished_sending:                      # vLLM would hand the blocks to someone else
        gpu_blocks[2] = b"reused by another request"
    process_next_save(worker)
    assert stored[b"second hash"] == b"second request block"


def test_later_save_reopens_completed_request():
    worker, _, _ = make_worker()
    first = enqueue_save(worker)
    complete_next_save(worker)
    assert first.is_set()
    second = enqueue_save(worker)
    assert not second.is_set()
    assert worker.get_finished({"request"})[0] is None
    complete_next_save(worker)
    assert second.is_set()
    assert worker.get_finished({"request"})[0] == {"request"}


def test_finished_request_is_reported_once_its_last_save_settles_in_a_later_step():
    worker, _, _ = make_worker()
    enqueue_save(worker)
    assert worker.get_finished({"request"})[0] is None       # finished while the save is pending
    complete_next_save(worker)
    assert worker.get_finished(set())[0] == {"request"}      # reported without being named again
    assert worker.get_finished(set())[0] is None


def test_committed_save_runs_on_a_no_forward_step():
    worker, client, _ = make_worker(CacheGroups((("layer",), ("state",)), frozenset({1})))
    worker._cross_layer_mode = False
    worker._registered_layers = ["layer"]
    metadata = PegaConnectorMetadata(ready_save_intents={
        "request": SaveIntent(block_ids_by_group=((1,), (1,)), block_hashes=(b"hash",))})
    worker.start_load_kv(metadata, None)
    assert len(client.save_calls) == 1
    assert worker.get_finished({"request"})[0] == {"request"}


def test_ready_save_intents_need_a_recurrent_group():
    worker, _, _ = make_worker()
    metadata = PegaConnectorMetadata(ready_save_intents={
        "request": SaveIntent(block_ids_by_group=((1,),), block_hashes=(b"hash",))})
    with pytest.raises(RuntimeError, match="only valid for HMA"):
        worker.start_load_kv(metadata, None)


def test_current_step_save_waits_for_forward_completion():
    worker, client, _ = make_worker(CacheGroups((("layer",), ("state",)), frozenset({1})))
    worker._cross_layer_mode = False
    worker._registered_layers = ["layer"]
    metadata = PegaConnectorMetadata(save_intents={
        "request": SaveIntent(block_ids_by_group=((1,), (1,)), block_hashes=(b"hash",))})
    worker.start_load_kv(metadata, None)
    assert client.save_calls == []
    worker.wait_for_save()                    # recurrent state: saved before returning
    assert len(client.save_calls) == 1


def test_preemption_waits_for_every_save_task():
    worker, _, _ = make_worker()
    enqueue_save(worker)
    enqueue_save(worker)
    returned = threading.Event()
    thread = threading.Thread(target=lambda: (worker.handle_preemptions({"request"}),
                                              returned.set()))
    thread.start()
    try:
        assert not returned.wait(timeout=0.1)
        complete_next_save(worker)
        assert not returned.wait(timeout=0.1)     # one task is still reading the blocks
        complete_next_save(worker)
        assert returned.wait(timeout=1)
    finally:
        while not worker._save_queue.empty():
            complete_next_save(worker)
        thread.join(timeout=1)
    assert not thread.is_alive()
    worker.handle_preemptions({"unknown"})         # nothing pending: returns at once
    worker.handle_preemptions(None)


def test_failed_save_still_completes_the_request_and_null_block_is_dropped():
    worker, client, _ = make_worker()
    worker._cross_layer_mode = False
    worker._registered_layers = ["l0", "l1"]
    client.save_result = (False, "disk full")
    worker._current_metadata = PegaConnectorMetadata(save_intents={
        "r": SaveIntent(block_ids_by_group=((0, 4, 5),), block_hashes=(b"a", b"b", b"c"))})
    worker.wait_for_save()
    process_next_save(worker)
    assert client.save_calls == [[("l0", [4, 5], [b"b", b"c"]), ("l1", [4, 5], [b"b", b"c"])]]
    assert worker.get_finished({"r"})[0] == {"r"}


def test_save_thread_batches_queued_tasks_into_one_engine_call():
    worker, client, _ = make_worker(start_save_thread=False)
    worker._cross_layer_mode = False
    worker._registered_layers = ["layer"]
    for req, block in (("a", 1), ("b", 2), ("c", 3)):
        worker._current_metadata = PegaConnectorMetadata(save_intents={
            req: SaveIntent(block_ids_by_group=((block,),), block_hashes=(req.encode(),))})
        worker.wait_for_save()
    worker._save_queue.put(None)
    worker._save_worker()                          # runs until the stop marker
    assert client.save_calls == [[("layer", [1, 2, 3], [b"a", b"b", b"c"])]]
    assert worker.get_finished({"a", "b", "c"})[0] == {"a", "b", "c"}


# ---- load fault tolerance (test_connector_fault_tolerance.py:185-351) --------

def load_metadata(req_id, block_ids):
    return PegaConnectorMetadata(load_intents={req_id: LoadIntent(
        block_ids_by_group=(tuple(block_ids),), leases=(f"lease-{req_id}".encode(),),
        num_tokens=len(block_ids) * 16)})


def hybrid_worker():
    worker, client, state = make_worker(CacheGroups((("attention",), ("recurrent",)),
                                                    frozenset({1})))
    worker._cross_layer_mode = False
    worker._registered_layers = ["attention", "recurrent"]
    return worker, client, state


def hybrid_metadata(req_id):
    return PegaConnectorMetadata(load_intents={req_id: LoadIntent(
        block_ids_by_group=((11,), (21,)), leases=(f"lease-{req_id}".encode(),), num_tokens=16)})


@pytest.mark.parametrize("mode,req_id,block_ids", [("ok_false", "req_fail_ok", (1, 2, 3)),
                                                   ("exception", "req_fail_exc", (10, 20))])
def test_load_rpc_failure_reports_failures_without_raise(mode, req_id, block_ids):
    worker, client, state = make_worker()
    if mode == "ok_false":
        client.fail_load_with_ok_false = True
    else:
        client.fail_load_with_exception = ConnectionError("server gone")
    worker.start_load_kv(load_metadata(req_id, block_ids))            # must not raise
    assert len(client.load_calls) == 1
    assert worker.get_block_ids_with_load_errors() == set(block_ids)
    assert worker.get_block_ids_with_load_errors() == set()
    assert worker.get_finished(set())[1] == {req_id}
    assert state.mark_unavailable.called
    assert client.release_calls == [f"lease-{req_id}".encode()]
    assert worker._loads == {}


@pytest.mark.parametrize("mode", ["ok_false", "exception"])
def test_hybrid_load_rpc_failure_raises(mode):
    worker, client, state = hybrid_worker()
    if mode == "ok_false":
        client.fail_load_with_ok_false = True
    else:
        client.fail_load_with_exception = ConnectionError("server gone")
    with pytest.raises(RuntimeError, match="cannot recover failed loads"):
        worker.start_load_kv(hybrid_metadata("hma-failure"))
    assert state.mark_unavailable.called
    assert client.release_calls == [b"lease-hma-failure"]
    assert worker._loads == {}


def test_hybrid_load_distinguishes_block_zero_from_absent_recurrent_target():
    worker, client, _ = hybrid_worker()
    worker.start_load_kv(PegaConnectorMetadata(load_intents={"hma-sparse": LoadIntent(
        block_ids_by_group=((0, 12), (None, 21)), leases=(b"lease-hma-sparse",), num_tokens=32)}))
    assert client.load_calls[0][5] == [0, 12, None, 21]
    assert client.load_calls[0][4] == [["attention"], ["recurrent"]]


def test_hybrid_load_timeout_raises(monkeypatch):
    worker, _, state = hybrid_worker()
    clock = {"now": 10_000.0}
    monkeypatch.setattr(wc.time, "perf_counter", lambda: clock["now"])
    worker.start_load_kv(hybrid_metadata("hma-timeout"))
    clock["now"] += worker.LOAD_TIMEOUT_SECONDS + 1
    with pytest.raises(RuntimeError, match="cannot recover failed loads"):
        worker.get_finished(set())
    assert state.mark_unavailable.called
    assert worker._loads == {}


def test_in_flight_load_timeout_respects_configured_boundary(monkeypatch):
    worker, _, state = make_worker()
    timeout = worker.LOAD_TIMEOUT_SECONDS
    clock = {"now": 10_000.0}
    monkeypatch.setattr(wc.time, "perf_counter", lambda: clock["now"])
    worker.start_load_kv(load_metadata("req_boundary", (5, 6, 7, 8)))
    assert len(worker._loads) == 1
    clock["now"] = 10_000.0 + (timeout - 1)
    assert worker.get_finished(set())[1] is None
    assert len(worker._loads) == 1
    assert worker.get_block_ids_with_load_errors() == set()
    assert not state.mark_unavailable.called
    clock["now"] = 10_000.0 + (timeout + 1)
    assert worker.get_finished(set())[1] == {"req_boundary"}
    assert worker.get_block_ids_with_load_errors() == {5, 6, 7, 8}
    assert state.mark_unavailable.called
    assert worker._loads == {}


def test_load_completion_and_async_failure_are_reported():
    worker, _, _ = make_worker()
    worker.start_load_kv(load_metadata("good", (1, 2)))
    worker.start_load_kv(load_metadata("bad", (3,)))
    assert worker.get_finished(set())[1] is None                 # both still pending
    good, bad = (load.state for load in worker._loads.values())
    good.value = 1
    assert worker.get_finished(set())[1] == {"good"}
    assert worker.get_block_ids_with_load_errors() == set()
    bad.value = -1
    assert worker.get_finished(set())[1] == {"bad"}
    assert worker.get_block_ids_with_load_errors() == {3}
    assert good.closed and bad.closed


def test_get_block_ids_with_load_errors_drains_between_calls():
    worker, client, _ = make_worker()
    client.fail_load_with_ok_false = True
    worker.start_load_kv(load_metadata("r1", (1,)))
    worker.start_load_kv(load_metadata("r2", (2, 3)))
    assert worker.get_block_ids_with_load_errors() == {1, 2, 3}
    assert worker.get_block_ids_with_load_errors() == set()


def test_load_uses_registered_layer_names():
    worker, client, _ = make_worker()
    worker._cross_layer_mode = False
    worker._registered_layers = ["registered.layer.0", "registered.layer.1"]
    forward_context = MagicMock()
    forward_context.no_compile_layers = {"model.layers.0.attn": MagicMock()}
    worker.start_load_kv(load_metadata("req", (1, 2)), forward_context)
    assert client.load_calls[0][4] == [["registered.layer.0", "registered.layer.1"]]


def test_cross_layer_mode_loads_the_pseudo_layer_and_empty_loads_do_nothing():
    worker, client, _ = make_worker()
    worker.start_load_kv(load_metadata("req", (7,)))
    assert client.load_calls[0][4] == [["ALL_LAYERS"]]
    worker.start_load_kv(PegaConnectorMetadata(load_intents={"none": LoadIntent(
        block_ids_by_group=((None, None),), leases=(b"l",), num_tokens=32)}))
    assert len(client.load_calls) == 1                           # nothing to load: no call
    with pytest.raises(RuntimeError, match="2 TP shard leases; expected 1"):
        worker.start_load_kv(PegaConnectorMetadata(load_intents={"x": LoadIntent(
            block_ids_by_group=((1,),), leases=(b"a", b"b"), num_tokens=16)}))


def test_recurrent_hold_adds_one_membership_load_per_recurrent_group():
    # worker.py:572-619: the prefix lease carries the attention destinations
    # only; the checkpoint's state block travels with the membership lease.
    worker, client, _ = hybrid_worker()
    hold = RecurrentLoadHold(leases=((b"member",),), hit_positions=(((0, 2),),), checkpoint=2)
    worker.start_load_kv(PegaConnectorMetadata(load_intents={"h": LoadIntent(
        block_ids_by_group=((11, 12, 13), (None, None, 31)), leases=(b"prefix",), num_tokens=48,
        recurrent_hold=hold)}))
    loads = client.load_calls[0][6]
    assert loads == [(b"prefix", [[11, 12, 13], [None, None, None]]),
                     (b"member", [[None, None], [None, 31]])]
    bad = RecurrentLoadHold(leases=((b"member",),), hit_positions=(((0, 1),),), checkpoint=2)
    with pytest.raises(RuntimeError, match="no checkpoint at query position 2"):
        worker.start_load_kv(PegaConnectorMetadata(load_intents={"h": LoadIntent(
            block_ids_by_group=((11,), (31,)), leases=(b"prefix",), num_tokens=16,
            recurrent_hold=bad)}))


# ---- registration (worker.py:261-420; test_connector_fault_tolerance.py:500-511) ----

def registering_worker(monkeypatch, cache_groups=None, **ctx):
    """A worker whose engine registration is captured instead of executed."""
    calls = []

    def fake_register(engine, instance_id, namespace, device_id, kv_caches, block_size, **kw):
        calls.append(dict(instance_id=instance_id, namespace=namespace, device_id=device_id,
                          layers=list(kv_caches), block_size=block_size, **kw))
        return list(kv_caches)

    monkeypatch.setattr(wc, "register_kv_caches", fake_register)
    client = wc.InProcessEngineClient(engine=None)
    fields = dict(instance_id="inst", namespace="ns", block_size=16, tp_size=1, world_size=1,
                  tp_rank=0, device_id=0, engine_client=client)
    fields.update(ctx)
    worker = WorkerConnector(ConnectorContext(**fields), cache_groups, start_save_thread=False)
    return worker, calls


def test_registration_passes_storage_group_ids(monkeypatch):
    groups = CacheGroups((("mamba.0", "mamba.1"), ("attn.0",)), frozenset({0}))
    worker, calls = registering_worker(monkeypatch, groups)
    worker.register_kv_caches({"attn.0": object(), "mamba.0": object(), "mamba.1": object()})
    assert calls[0]["layer_group_ids"] == [0, 1, 1]          # attention is storage group 0
    assert calls[0]["recurrent_layer_names"] == {"mamba.0", "mamba.1"}
    assert calls[0]["page_first"] is False
    assert worker._registered_layers == ["attn.0", "mamba.0", "mamba.1"]
    with pytest.raises(RuntimeError, match="layers outside cache groups: \\['stray'\\]"):
        worker.register_kv_caches({"attn.0": object(), "stray": object()})


def test_single_group_registration_and_page_first_choice(monkeypatch):
    worker, calls = registering_worker(monkeypatch, is_mla=True, tp_rank=3, tp_size=4)
    worker.register_kv_caches({"l0": object()})
    # MLA: stored once for all TP ranks, page-first when one worker writes whole pages
    assert calls[0]["layer_group_ids"] is None and calls[0]["page_first"] is True
    assert calls[0]["tp_rank"] == 0 and calls[0]["tp_size"] == 1
    worker, calls = registering_worker(monkeypatch, is_mla=True, pp_size=2)
    worker.register_kv_caches({"l0": object()})
    assert calls[0]["page_first"] is False                    # a pipeline stage holds part of a page


def test_cross_layer_registration_uses_pp_suffixed_name(monkeypatch):
    worker, calls = registering_worker(monkeypatch, pp_rank=2, pp_size=4)
    worker.register_cross_layers_kv_cache(object())
    assert calls[0]["layers"] == ["ALL_LAYERS_pp2"]
    assert worker._cross_layer_mode and worker._registered_layers == ["ALL_LAYERS_pp2"]
    worker, calls = registering_worker(monkeypatch)
    worker.register_cross_layers_kv_cache(object())
    assert calls[0]["layers"] == ["ALL_LAYERS"]
    assert worker._load_layer_groups() == [["ALL_LAYERS"]]    # loads then name the pseudo-layer
