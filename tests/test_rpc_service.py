"""The gRPC handlers and the client over a fake engine, on the CPU: argument
validation and status codes of pegaflow-server/src/service.rs (:205-358
register, :360-437 save, :439-541 load, :543-736 query, :738-766 release,
:768-809 unregister), the 16-byte lease on the wire (lease.rs:14-35), and the
liveness session (session.rs: the newest session of an instance owns it; a
superseded one cleans nothing up when it ends).  The same service runs over
the real engine in tests/test_gpu_rpc.py."""

import threading
import time

import pytest

grpc = pytest.importorskip("grpc")

from pegaflow_amd import _lib, rpc  # noqa: E402


class FakeTask:
    def __init__(self):
        self.closed = False

    def wait(self, _timeout):
        from pegaflow_amd.engine import TaskResult
        return TaskResult(True, 0, 0.0)

    def close(self):
        self.closed = True


class FakeEngine:
    def __init__(self):
        self.saved = []
        self.loads = []
        self.leases = {}
        self.next_lease = 41
        self.sealed = set()
        self.unregistered = []
        self.tasks = []

    def batch_save_kv_blocks(self, instance, tp_rank, pp_rank, device_id, saves):
        if instance == "missing":
            raise _lib.PegaHipError(_lib.PF_ERR_INSTANCE_MISSING, "instance missing not found")
        self.saved.append((instance, tp_rank, pp_rank, device_id,
                           [(s.layer_name, list(s.block_ids), list(s.block_hashes)) for s in saves]))
        for s in saves:
            self.sealed.update(s.block_hashes)

    def query_prefix(self, instance, hashes):
        hits = 0
        for h in hashes:
            if h not in self.sealed:
                break
            hits += 1
        if hits == 0:
            return 0, 0
        self.next_lease += 1
        self.leases[self.next_lease] = hashes[:hits]
        return hits, self.next_lease

    def query_group_membership(self, instance, group, hashes):
        return [h in self.sealed for h in hashes]

    def create_group_lease(self, instance, group, hashes):
        self.next_lease += 1
        self.leases[self.next_lease] = list(hashes)
        return self.next_lease

    def query_group_lease(self, instance, group, hashes, require_all=False):
        present = [h in self.sealed for h in hashes]
        hit = [h for h in hashes if h in self.sealed]
        if not hit or (require_all and len(hit) != len(hashes)):
            return present, 0
        return present, self.create_group_lease(instance, group, hit)

    def release_query_lease(self, lease):
        if lease not in self.leases:
            raise _lib.StorageError(_lib.PF_ERR_STORAGE, "query lease is unknown or expired")
        del self.leases[lease]

    def batch_load_multi(self, instance, tp_rank, device_id, groups, loads, state):
        self.loads.append((instance, tp_rank, device_id, groups, loads))
        task = FakeTask()
        self.tasks.append(task)
        return task

    def unregister_instance(self, instance):
        self.unregistered.append(instance)


class FakeRegistry:
    def __init__(self):
        self.dropped = []

    def drop_instance(self, instance):
        self.dropped.append(instance)
        return 1


@pytest.fixture()
def served():
    engine, registry = FakeEngine(), FakeRegistry()
    server, service, port = rpc.serve(engine, "127.0.0.1:0", registry=registry)
    client = rpc.EngineRpcClient(f"http://127.0.0.1:{port}")
    yield engine, registry, service, client, port
    client.close()
    service.close()
    server.stop(0)


def _rejected(fn):
    with pytest.raises(rpc.RpcRejected) as err:
        fn()
    return err.value.code, str(err.value)


def test_health_and_shutdown_flag(served):
    engine, registry, service, client, _ = served
    assert client.health() == (True, "")
    assert not service.shutdown_requested.is_set()
    assert client.shutdown()[0]
    assert service.shutdown_requested.is_set()


def test_register_validation_codes(served):
    _engine, _registry, service, client, _ = served
    args = dict(instance_id="i", namespace="n", tp_rank=0, pp_rank=0, tp_size=1, world_size=1,
                device_id=0, layer_names=["l0"], wrapper_bytes_list=[b"x"], num_blocks_list=[4],
                bytes_per_block_list=[1024], kv_stride_bytes_list=[0], segments_list=[1],
                transfer_backend="direct", page_first=False)
    assert _rejected(lambda: client.register_context_batch(**{**args, "tp_size": 0})) == \
        ("INVALID_ARGUMENT", "tp_size must be > 0")
    assert _rejected(lambda: client.register_context_batch(**{**args, "world_size": 0})) == \
        ("INVALID_ARGUMENT", "world_size must be > 0")
    assert _rejected(lambda: client.register_context_batch(**{**args, "tp_rank": 1})) == \
        ("INVALID_ARGUMENT", "tp_rank 1 out of range (tp_size 1)")
    code, text = _rejected(lambda: client.register_context_batch(**{**args, "num_blocks_list": []}))
    assert code == "INVALID_ARGUMENT" and "same non-zero length" in text
    # a wrapper the server cannot read is its own failure class, as a failed unpickle is
    with pytest.raises(rpc.PegaFlowError) as err:
        client.register_context_batch(**args)
    assert err.value.code == "INTERNAL" and "register tensor failed" in str(err.value)
    # a client of another release is refused before anything is touched (service.rs:212-222)
    service.version = "9.9.9"
    code, text = _rejected(lambda: client.register_context_batch(**args))
    assert code == "FAILED_PRECONDITION"
    assert text == f"PegaFlow version mismatch: client={rpc.PROTOCOL_VERSION} server=9.9.9"


def test_save_query_release_over_the_wire(served):
    engine, _registry, _service, client, _ = served
    hashes = [bytes([i]) * 32 for i in range(5)]
    assert client.save("inst", 0, 0, 0, [("l0", [3, 1, 4, 1, 5], hashes)]) == (True, "")
    assert engine.saved == [("inst", 0, 0, 0, [("l0", [3, 1, 4, 1, 5], hashes)])]
    assert _rejected(lambda: client.save("inst", 0, 0, 0, [("l0", [1, 2], hashes[:1])])) == \
        ("INVALID_ARGUMENT", "block_ids length 2 does not match block_hashes 1 for layer l0")
    # an engine error that is not the caller's fault travels as INTERNAL
    with pytest.raises(rpc.PegaFlowError) as err:
        client.save("missing", 0, 0, 0, [("l0", [1], hashes[:1])])
    assert "not found" in str(err.value)

    assert _rejected(lambda: client.query_prefetch("inst", hashes, "")) == \
        ("INVALID_ARGUMENT", "req_id must not be empty")
    cold = client.query_prefetch("inst", [b"\xff" * 32], "r0")
    assert isinstance(cold, rpc.QueryReady) and (cold.num_hit_blocks, cold.lease) == (0, b"")
    hit = client.query_prefetch("inst", hashes + [b"\xfe" * 32], "r1")
    assert hit.num_hit_blocks == 5 and len(hit.lease) == 16
    lease = rpc.lease_from_bytes(hit.lease)
    assert engine.leases[lease] == hashes
    client.release(hit.lease)
    assert lease not in engine.leases
    assert _rejected(lambda: client.release(hit.lease)) == \
        ("FAILED_PRECONDITION", "query lease is unknown or expired")
    code, _text = _rejected(lambda: client.release(b"short"))
    assert code == "INVALID_ARGUMENT"


def test_group_membership_query_and_want_sets(served):
    engine, _registry, _service, client, _ = served
    have = [bytes([i]) * 32 for i in range(3)]
    client.save("inst", 0, 0, 0, [("l0", [0, 1, 2], have)])
    want = [have[0], b"\xaa" * 32, have[2]]
    some = client.query_prefetch("inst", want, "g1", group_id=1)
    assert (some.num_hit_blocks, some.hit_positions) == (2, [0, 2]) and len(some.lease) == 16
    assert engine.leases[rpc.lease_from_bytes(some.lease)] == [have[0], have[2]]
    # all-or-nothing: a short answer carries no lease (service.rs:630-668)
    short = client.query_prefetch("inst", want, "g2", wait_for_full_prefix=True, group_id=1)
    assert short.num_hit_blocks == 2 and short.lease == b""
    full = client.query_prefetch("inst", have, "g3", wait_for_full_prefix=True, group_id=1)
    assert full.num_hit_blocks == 3 and len(full.lease) == 16


def test_load_carries_leases_groups_and_skipped_positions(served):
    engine, _registry, service, client, _ = served
    lease = rpc.lease_to_bytes(77)
    ok = client.load("inst", 0, 0, "", [["l0", "l1"], ["m0"]],
                     [(lease, [[5, None, 7], [None, 2, 3]])])
    assert ok == (True, "")
    assert engine.loads == [("inst", 0, 0, [["l0", "l1"], ["m0"]],
                             [(77, [[5, None, 7], [None, 2, 3]])])]
    service.close()
    assert all(t.closed for t in engine.tasks)   # settled loads give their handles back
    code, _ = _rejected(lambda: client.load("inst", 0, 0, "", [["l0"]], [(b"bad", [[1]])]))
    assert code == "INVALID_ARGUMENT"


def test_unregister_drops_engine_and_registry_state(served):
    engine, registry, _service, client, _ = served
    assert client.unregister_context("inst-a")[0]
    assert engine.unregistered == ["inst-a"] and registry.dropped == ["inst-a"]


def _wait_for(cond, seconds=5.0):
    deadline = time.monotonic() + seconds
    while time.monotonic() < deadline:
        if cond():
            return True
        time.sleep(0.02)
    return cond()


def test_session_end_cleans_up_unless_superseded(served):
    engine, registry, service, client, port = served
    client.start_session_watcher("inst-s", "ns", 1, 1)
    assert _wait_for(lambda: "inst-s" in service._sessions)
    # a second process takes the instance over (a restarted worker): the old
    # stream's end must not tear down what the new one registered
    second = rpc.EngineRpcClient(f"http://127.0.0.1:{port}")
    first_token = service._sessions["inst-s"]
    second.start_session_watcher("inst-s", "ns", 1, 1)
    assert _wait_for(lambda: service._sessions.get("inst-s", first_token) != first_token)
    client.stop_session_watcher()
    time.sleep(0.3)
    assert engine.unregistered == [] and registry.dropped == []
    # the owner's stream ends: the instance goes
    second.stop_session_watcher()
    assert _wait_for(lambda: engine.unregistered == ["inst-s"])
    assert registry.dropped == ["inst-s"] and "inst-s" not in service._sessions
    second.close()


def test_session_needs_an_instance_id(served):
    _engine, _registry, service, client, _ = served
    client.start_session_watcher("", "ns", 1, 1)
    time.sleep(0.3)
    assert service._sessions == {}


def test_lease_bytes_round_trip():
    for lease in (1, 77, 2**63 + 5):
        raw = rpc.lease_to_bytes(lease)
        assert len(raw) == 16 and rpc.lease_from_bytes(raw) == lease
    with pytest.raises(ValueError):
        rpc.lease_from_bytes(b"\x00" * 15)
