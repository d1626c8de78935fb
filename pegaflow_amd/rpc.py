"""The engine's gRPC boundary: the messages of the reference's `Engine` service
that sit on the save / load path, a server over ``PegaEngine`` +
``TensorRegistry``, and a client with the reference's method names.

Wire format: package ``pegaflow``, service ``Engine``, message and field
numbers of pegaflow-proto/proto/engine.proto:5-197,251-270
(RegisterContextBatch, Save, Load, QueryPrefetch, Release, UnregisterContext,
Health, Shutdown, and the liveness stream Session).  The descriptors are built at import time with protobuf's
descriptor API because the image has no protoc; the bytes on the wire are
those a stub generated from engine.proto produces.  Handlers follow
pegaflow-server/src/service.rs:85-96 (status codes), :110-160 (validation),
:205-540 (register / save / load), :543-760 (query, release),
:768-809 (unregister), :1017-1072 with session.rs (a worker's liveness stream:
when it closes, the instance's mappings and registrations are dropped).

Differences from the reference, on purpose:
  * ``wrapper_bytes`` carries ``HipIPCWrapper.to_bytes()`` records, not pickles;
  * a lease travels as 16 bytes (the reference's size) whose first 8 are this
    engine's 64-bit lease id;
  * RDMA / MetaServer RPCs are not served (UNIMPLEMENTED);
  * ``transfer_mode`` KERNEL (what the connector sends for MLA models,
    python/pegaflow/connector/common.py:577-594) registers workers that choose
    the way across the link per task, like DIRECT; an engine created with
    ``kernel_mode_zerocopy=True`` gives such registrations the reference's
    kernel mode (one copy kernel over mapped host memory).  The worker pool
    logs its choice when it is spawned and every settled load is logged here at
    debug level with the path it took.
"""

from __future__ import annotations

import logging
import threading
from concurrent import futures
from typing import Sequence

import grpc
from google.protobuf import descriptor_pb2, descriptor_pool, message_factory

from . import _lib
from .engine import LayerSave, LoadState, PegaEngine
from .ipc import TensorRegistry, register_context_batch
from .transfer import TransferMode

# The reference release whose client this server accepts
# (service.rs:118-130: client and server versions must match).
log = logging.getLogger(__name__)

PROTOCOL_VERSION = "0.23.12"
DEFAULT_ENDPOINT = "127.0.0.1:50055"

_F = descriptor_pb2.FieldDescriptorProto
_T = {"string": _F.TYPE_STRING, "bytes": _F.TYPE_BYTES, "bool": _F.TYPE_BOOL,
      "uint32": _F.TYPE_UINT32, "uint64": _F.TYPE_UINT64, "int32": _F.TYPE_INT32}


def _build_file() -> descriptor_pb2.FileDescriptorProto:
    f = descriptor_pb2.FileDescriptorProto(name="pegaflow_amd/engine_path.proto", package="pegaflow",
                                           syntax="proto3")
    enum = f.enum_type.add(name="TransferMode")
    enum.value.add(name="TRANSFER_MODE_DIRECT", number=0)
    enum.value.add(name="TRANSFER_MODE_KERNEL", number=1)

    def message(name, fields, oneofs=()):
        m = f.message_type.add(name=name)
        for o in oneofs:
            m.oneof_decl.add(name=o)
        for spec in fields:
            fname, number, ftype = spec[:3]
            repeated = len(spec) > 3 and spec[3] == "repeated"
            oneof = spec[3] if len(spec) > 3 and spec[3] != "repeated" else None
            fd = m.field.add(name=fname, number=number,
                             label=_F.LABEL_REPEATED if repeated else _F.LABEL_OPTIONAL)
            if ftype in _T:
                fd.type = _T[ftype]
            elif ftype == "TransferMode":
                fd.type, fd.type_name = _F.TYPE_ENUM, ".pegaflow.TransferMode"
            else:
                fd.type, fd.type_name = _F.TYPE_MESSAGE, ".pegaflow." + ftype
            if oneof is not None:
                fd.oneof_index = list(oneofs).index(oneof)
        return m

    message("ResponseStatus", [("ok", 1, "bool"), ("message", 2, "string")])
    message("RegisterContextRequest", [
        ("instance_id", 1, "string"), ("namespace", 2, "string"), ("tp_rank", 3, "uint32"),
        ("tp_size", 4, "uint32"), ("world_size", 5, "uint32"), ("device_id", 6, "int32"),
        ("layer_names", 8, "string", "repeated"), ("wrapper_bytes", 9, "bytes", "repeated"),
        ("num_blocks", 10, "uint64", "repeated"), ("bytes_per_block", 11, "uint64", "repeated"),
        ("kv_stride_bytes", 12, "uint64", "repeated"), ("segments", 13, "uint32", "repeated"),
        ("pp_rank", 14, "uint32"), ("client_version", 15, "string"),
        ("transfer_mode", 17, "TransferMode"), ("page_first", 18, "bool"),
        ("layer_group_ids", 19, "uint32", "repeated")])
    message("RegisterContextResponse", [("status", 1, "ResponseStatus")])
    message("SaveLayer", [("layer_name", 1, "string"), ("block_ids", 2, "uint32", "repeated"),
                          ("block_hashes", 3, "bytes", "repeated")])
    message("SaveRequest", [("instance_id", 1, "string"), ("tp_rank", 2, "uint32"),
                            ("device_id", 3, "int32"), ("saves", 4, "SaveLayer", "repeated"),
                            ("pp_rank", 5, "uint32")])
    message("SaveResponse", [("status", 1, "ResponseStatus")])
    message("LoadGroup", [("layer_names", 1, "string", "repeated")])
    message("LoadBlockTarget", [("block_id", 1, "uint32", "target")], oneofs=("target",))
    message("LoadBlockIds", [("targets", 1, "LoadBlockTarget", "repeated")])
    message("LeaseLoad", [("lease", 1, "bytes"),
                          ("block_ids_by_group", 2, "LoadBlockIds", "repeated")])
    message("LoadRequest", [("instance_id", 1, "string"), ("tp_rank", 2, "uint32"),
                            ("device_id", 3, "int32"), ("load_state_shm", 4, "string"),
                            ("groups", 5, "LoadGroup", "repeated"),
                            ("loads", 6, "LeaseLoad", "repeated")])
    message("LoadResponse", [("status", 1, "ResponseStatus")])
    message("QueryRequest", [("instance_id", 1, "string"), ("block_hashes", 2, "bytes", "repeated"),
                             ("req_id", 3, "string"), ("wait_for_full_prefix", 4, "bool"),
                             ("group_id", 5, "uint32")])
    message("QueryLoading", [])
    message("QueryReady", [("num_hit_blocks", 1, "uint64"), ("lease", 2, "bytes"),
                           ("hit_positions", 3, "uint32", "repeated")])
    message("QueryResponse", [("loading", 1, "QueryLoading", "outcome"),
                              ("ready", 2, "QueryReady", "outcome")], oneofs=("outcome",))
    message("ReleaseRequest", [("lease", 1, "bytes")])
    message("ReleaseResponse", [])
    message("UnregisterRequest", [("instance_id", 1, "string")])
    message("UnregisterResponse", [("status", 1, "ResponseStatus")])
    message("ShutdownRequest", [])
    message("ShutdownResponse", [("status", 1, "ResponseStatus")])
    message("HealthRequest", [])
    message("HealthResponse", [("status", 1, "ResponseStatus")])
    message("SessionRequest", [("instance_id", 1, "string"), ("namespace", 2, "string"),
                               ("tp_size", 3, "uint32"), ("world_size", 4, "uint32")])
    message("SessionEvent", [])
    return f


_POOL = descriptor_pool.DescriptorPool()
_POOL.Add(_build_file())


def _cls(name):
    return message_factory.GetMessageClass(_POOL.FindMessageTypeByName("pegaflow." + name))


ResponseStatus = _cls("ResponseStatus")
RegisterContextRequest, RegisterContextResponse = _cls("RegisterContextRequest"), _cls("RegisterContextResponse")
SaveLayer, SaveRequest, SaveResponse = _cls("SaveLayer"), _cls("SaveRequest"), _cls("SaveResponse")
LoadGroup, LoadBlockTarget, LoadBlockIds = _cls("LoadGroup"), _cls("LoadBlockTarget"), _cls("LoadBlockIds")
LeaseLoad, LoadRequest, LoadResponse = _cls("LeaseLoad"), _cls("LoadRequest"), _cls("LoadResponse")
QueryRequest, QueryResponse = _cls("QueryRequest"), _cls("QueryResponse")
QueryLoadingMsg, QueryReadyMsg = _cls("QueryLoading"), _cls("QueryReady")
ReleaseRequest, ReleaseResponse = _cls("ReleaseRequest"), _cls("ReleaseResponse")
UnregisterRequest, UnregisterResponse = _cls("UnregisterRequest"), _cls("UnregisterResponse")
ShutdownRequest, ShutdownResponse = _cls("ShutdownRequest"), _cls("ShutdownResponse")
HealthRequest, HealthResponse = _cls("HealthRequest"), _cls("HealthResponse")
SessionRequest, SessionEvent = _cls("SessionRequest"), _cls("SessionEvent")

# method -> (request class, response class)
METHODS = {
    "RegisterContextBatch": (RegisterContextRequest, RegisterContextResponse),
    "Save": (SaveRequest, SaveResponse),
    "Load": (LoadRequest, LoadResponse),
    "QueryPrefetch": (QueryRequest, QueryResponse),
    "Release": (ReleaseRequest, ReleaseResponse),
    "UnregisterContext": (UnregisterRequest, UnregisterResponse),
    "Shutdown": (ShutdownRequest, ShutdownResponse),
    "Health": (HealthRequest, HealthResponse),
}
SERVICE = "pegaflow.Engine"


def lease_to_bytes(lease: int) -> bytes:
    """16 bytes, as the reference's QueryLeaseId (lease.rs:14-35)."""
    return int(lease).to_bytes(8, "little") + bytes(8)


def lease_from_bytes(data: bytes) -> int:
    if len(data) == 0:
        raise ValueError("query lease id must be non-empty")
    if len(data) != 16:
        raise ValueError(f"query lease id must be 16 bytes, got {len(data)}")
    return int.from_bytes(data[:8], "little")


def _ok():
    return ResponseStatus(ok=True, message="")


class _Abort(Exception):
    def __init__(self, code, message):
        super().__init__(message)
        self.code, self.message = code, message


def _map_engine_error(exc: Exception) -> _Abort:
    """service.rs:85-96."""
    if isinstance(exc, _lib.InvalidArgument):
        return _Abort(grpc.StatusCode.INVALID_ARGUMENT, exc.message)
    if isinstance(exc, (_lib.InstanceMissing, _lib.WorkerMissing)):
        return _Abort(grpc.StatusCode.FAILED_PRECONDITION, exc.message)
    if isinstance(exc, _lib.PegaHipError):
        return _Abort(grpc.StatusCode.INTERNAL, exc.message)
    if isinstance(exc, ValueError):
        return _Abort(grpc.StatusCode.INVALID_ARGUMENT, str(exc))
    return _Abort(grpc.StatusCode.INTERNAL, f"{type(exc).__name__}: {exc}")


def _validate_device_id(device_id: int) -> None:
    if device_id < 0:
        raise _Abort(grpc.StatusCode.INVALID_ARGUMENT, f"device_id {device_id} must be >= 0")


class EngineService:
    """The handlers; one instance serves every connection and shares one
    engine and one registry, as the reference's server does."""

    def __init__(self, engine: PegaEngine, registry: TensorRegistry | None = None,
                 version: str = PROTOCOL_VERSION):
        self.engine = engine
        self.registry = registry if registry is not None else TensorRegistry()
        self.version = version
        self.shutdown_requested = threading.Event()
        self._pending = []            # submitted loads whose handles are not yet released
        self._pending_lock = threading.Lock()
        # session.rs: the current liveness session of each instance; a newer one
        # supersedes the older, whose end then cleans nothing up
        self._sessions = {}
        self._sessions_lock = threading.Lock()
        self._next_session = 0

    def _reap(self, wait: bool = False) -> None:
        """Release the handles of loads that have settled (their outcome went to
        the LoadState); with ``wait``, of all of them."""
        with self._pending_lock:
            tasks, self._pending = self._pending, []
        keep = []
        for task in tasks:
            try:
                result = task.wait(-1 if wait else 0)
                if result.done:
                    # which way the bytes went and how long it took (the reference's
                    # worker logs the same per load, gpu_worker.rs:465-474)
                    if log.isEnabledFor(logging.DEBUG):
                        log.debug("load settled: %d bytes in %.3f ms, paths=%s staged_groups=%d "
                                  "zero_copy_launches=%d phases_ms=%s", result.bytes,
                                  result.elapsed_ms, ",".join(result.paths) or "-",
                                  result.staged_groups, result.zero_copy_launches,
                                  result.phases_ms)
                    task.close()
                else:
                    keep.append(task)
            except _lib.PegaHipError:
                task.close()          # failed: the LoadState already says so
        with self._pending_lock:
            self._pending.extend(keep)

    def close(self) -> None:
        self._reap(wait=True)

    # -- RegisterContextBatch (service.rs:205-358) -------------------------
    def RegisterContextBatch(self, req):
        if req.client_version != self.version:
            raise _Abort(grpc.StatusCode.FAILED_PRECONDITION,
                         f"PegaFlow version mismatch: client={req.client_version or '<missing>'} "
                         f"server={self.version}")
        _validate_device_id(req.device_id)
        if req.tp_size == 0:
            raise _Abort(grpc.StatusCode.INVALID_ARGUMENT, "tp_size must be > 0")
        if req.world_size == 0:
            raise _Abort(grpc.StatusCode.INVALID_ARGUMENT, "world_size must be > 0")
        if req.tp_rank >= req.tp_size:
            raise _Abort(grpc.StatusCode.INVALID_ARGUMENT,
                         f"tp_rank {req.tp_rank} out of range (tp_size {req.tp_size})")
        n = len(req.layer_names)
        if n == 0 or any(len(a) != n for a in (req.wrapper_bytes, req.num_blocks,
                                               req.bytes_per_block, req.kv_stride_bytes,
                                               req.segments)):
            raise _Abort(grpc.StatusCode.INVALID_ARGUMENT,
                         f"all layer arrays must have the same non-zero length (got layer_names={n})")
        mode = TransferMode.KERNEL if req.transfer_mode == 1 else TransferMode.DIRECT
        try:
            register_context_batch(
                self.engine, self.registry, req.instance_id, req.namespace, req.device_id,
                req.tp_rank, req.pp_rank, req.tp_size, req.world_size, list(req.layer_names),
                list(req.wrapper_bytes), list(req.num_blocks), list(req.bytes_per_block),
                list(req.kv_stride_bytes), list(req.segments), transfer_mode=mode,
                page_first=req.page_first, layer_group_ids=list(req.layer_group_ids) or None)
        except _lib.PegaHipError as exc:
            if "register tensor failed" in exc.message or "already registered" in exc.message \
                    or "appears more than once" in exc.message or "pinned to device" in exc.message:
                # service.rs:294: registry failures are INTERNAL
                raise _Abort(grpc.StatusCode.INTERNAL,
                             exc.message if exc.message.startswith("register tensor failed")
                             else f"register tensor failed: {exc.message}")
            raise _map_engine_error(exc)
        except ValueError as exc:
            # a wrapper that cannot be read (engine errors, some of which are
            # ValueErrors too, are handled above): the reference fails to
            # unpickle it and answers INTERNAL (service.rs:286-296)
            raise _Abort(grpc.StatusCode.INTERNAL, f"register tensor failed: {exc}")
        return RegisterContextResponse(status=_ok())

    # -- Save (service.rs:360-437) ------------------------------------------
    def Save(self, req):
        _validate_device_id(req.device_id)
        for layer in req.saves:
            if len(layer.block_ids) != len(layer.block_hashes):
                raise _Abort(grpc.StatusCode.INVALID_ARGUMENT,
                             f"block_ids length {len(layer.block_ids)} does not match block_hashes "
                             f"{len(layer.block_hashes)} for layer {layer.layer_name}")
        saves = [LayerSave(l.layer_name, list(l.block_ids), list(l.block_hashes)) for l in req.saves]
        try:
            self.engine.batch_save_kv_blocks(req.instance_id, req.tp_rank, req.pp_rank,
                                             req.device_id, saves)
        except Exception as exc:
            raise _map_engine_error(exc)
        return SaveResponse(status=_ok())

    # -- Load (service.rs:439-541) ------------------------------------------
    def Load(self, req):
        _validate_device_id(req.device_id)
        groups = [list(g.layer_names) for g in req.groups]
        loads = []
        try:
            for load in req.loads:
                lease = lease_from_bytes(load.lease)
                by_group = [[t.block_id if t.HasField("block_id") else None for t in ids.targets]
                            for ids in load.block_ids_by_group]
                loads.append((lease, by_group))
        except ValueError as exc:
            raise _Abort(grpc.StatusCode.INVALID_ARGUMENT, str(exc))
        state = None
        try:
            if req.load_state_shm:
                state = LoadState(attach_to=req.load_state_shm)
            task = self.engine.batch_load_multi(req.instance_id, req.tp_rank, req.device_id, groups,
                                                loads, state)
            # The transfer completes on the load worker and is reported through
            # the LoadState; the RPC only submits it (lib.rs:880-898).
            with self._pending_lock:
                self._pending.append(task)
            self._reap()
        except Exception as exc:
            raise _map_engine_error(exc)
        finally:
            if state is not None:
                state.close()
        return LoadResponse(status=_ok())

    # -- QueryPrefetch (service.rs:543-736) ----------------------------------
    def QueryPrefetch(self, req):
        if not req.req_id:
            raise _Abort(grpc.StatusCode.INVALID_ARGUMENT, "req_id must not be empty")
        hashes = list(req.block_hashes)
        try:
            if req.group_id > 0:
                # membership and lease in one step: what is reported present is
                # what the lease pins (service.rs:606-636)
                present, lease_id = self.engine.query_group_lease(
                    req.instance_id, req.group_id, hashes, require_all=req.wait_for_full_prefix)
                positions = [i for i, hit in enumerate(present) if hit]
                if req.wait_for_full_prefix and len(positions) != len(hashes):
                    # all-or-nothing want-set: a short answer carries no lease
                    ready = QueryReadyMsg(num_hit_blocks=len(positions), lease=b"",
                                       hit_positions=list(range(len(positions))))
                    return QueryResponse(ready=ready)
                lease = lease_to_bytes(lease_id) if positions else b""
                return QueryResponse(ready=QueryReadyMsg(num_hit_blocks=len(positions), lease=lease,
                                                      hit_positions=positions))
            hits, lease = self.engine.query_prefix(req.instance_id, hashes)
        except Exception as exc:
            raise _map_engine_error(exc)
        return QueryResponse(ready=QueryReadyMsg(num_hit_blocks=hits,
                                              lease=lease_to_bytes(lease) if hits else b""))

    # -- Release (service.rs:738-766) -----------------------------------------
    def Release(self, req):
        try:
            lease = lease_from_bytes(req.lease)
        except ValueError as exc:
            raise _Abort(grpc.StatusCode.INVALID_ARGUMENT, str(exc))
        try:
            self.engine.release_query_lease(lease)
        except _lib.PegaHipError:
            raise _Abort(grpc.StatusCode.FAILED_PRECONDITION, "query lease is unknown or expired")
        return ReleaseResponse()

    # -- UnregisterContext (service.rs:768-809) -------------------------------
    def UnregisterContext(self, req):
        try:
            # the workers stop before their view of the tensors goes away
            self.engine.unregister_instance(req.instance_id)
        except Exception as exc:
            self.registry.drop_instance(req.instance_id)
            raise _map_engine_error(exc)
        self.registry.drop_instance(req.instance_id)
        return UnregisterResponse(status=_ok())

    def Health(self, req):
        return HealthResponse(status=_ok())

    # -- Session (service.rs:1017-1072, session.rs) ------------------------------
    def Session(self, req, context):
        """Server-streaming and silent: it lasts as long as the worker holds it.
        When the stream ends (the worker closed it, or died and its socket
        closed) the instance's mapped tensors and registrations are dropped,
        unless a newer session has taken the instance over."""
        if not req.instance_id:
            context.abort(grpc.StatusCode.INVALID_ARGUMENT, "instance_id must not be empty")
        with self._sessions_lock:
            self._next_session += 1
            token = self._next_session
            self._sessions[req.instance_id] = token
        ended = threading.Event()
        context.add_callback(ended.set)
        while not ended.wait(0.05):
            if self.shutdown_requested.is_set() or not context.is_active():
                break
        with self._sessions_lock:
            owned = self._sessions.get(req.instance_id) == token
            if owned:
                del self._sessions[req.instance_id]
        if owned:
            self.cleanup_instance(req.instance_id)
        return
        yield SessionEvent()  # pragma: no cover -- makes this a generator (a stream with no events)

    def cleanup_instance(self, instance_id: str) -> None:
        """service.rs cleanup_instance: what UnregisterContext does, without a caller
        to report to."""
        try:
            self.engine.unregister_instance(instance_id)
        except _lib.PegaHipError:
            pass
        self.registry.drop_instance(instance_id)

    def Shutdown(self, req):
        self.shutdown_requested.set()
        return ShutdownResponse(status=_ok())

    # -- plumbing -----------------------------------------------------------------
    def generic_handler(self):
        handlers = {}
        for name, (req_cls, resp_cls) in METHODS.items():
            fn = getattr(self, name)

            def behavior(request, context, fn=fn):
                try:
                    return fn(request)
                except _Abort as a:
                    context.abort(a.code, a.message)

            handlers[name] = grpc.unary_unary_rpc_method_handler(
                behavior, request_deserializer=req_cls.FromString,
                response_serializer=resp_cls.SerializeToString)
        handlers["Session"] = grpc.unary_stream_rpc_method_handler(
            self.Session, request_deserializer=SessionRequest.FromString,
            response_serializer=SessionEvent.SerializeToString)
        return grpc.method_handlers_generic_handler(SERVICE, handlers)


def serve(engine: PegaEngine, address: str = DEFAULT_ENDPOINT, registry: TensorRegistry | None = None,
          max_workers: int = 32):
    """Start a server; returns (grpc.Server, EngineService, bound port).  An open
    Session occupies one of the `max_workers` threads for as long as it lasts,
    so keep `max_workers` well above the number of worker processes."""
    service = EngineService(engine, registry)
    server = grpc.server(futures.ThreadPoolExecutor(max_workers=max_workers),
                         options=[("grpc.max_receive_message_length", 256 << 20),
                                  ("grpc.max_send_message_length", 256 << 20)])
    server.add_generic_rpc_handlers((service.generic_handler(),))
    port = server.add_insecure_port(address)
    server.start()
    return server, service, port


class PegaFlowError(RuntimeError):
    """The server is unavailable or failed internally."""

    def __init__(self, message: str, code: str = "UNKNOWN"):
        super().__init__(message)
        self.code = code


class RpcRejected(ValueError):
    """The server refused the request (INVALID_ARGUMENT or FAILED_PRECONDITION);
    ``code`` is the gRPC status name, the text is the server's message."""

    def __init__(self, message: str, code: str):
        super().__init__(message)
        self.code = code


class QueryLoading:
    """The query's backing fetch is still in progress (python/pegaflow/pegaflow.pyi:55-56)."""

    def __repr__(self) -> str:
        return "QueryLoading()"


class QueryReady:
    """pegaflow.pyi:58-67: the hit count, the lease over the hit blocks (empty on
    0 hits) and, for membership queries, the hit positions."""

    def __init__(self, num_hit_blocks: int, lease: bytes, hit_positions: Sequence[int] = ()):
        self.num_hit_blocks = int(num_hit_blocks)
        self.lease = bytes(lease)
        self.hit_positions = list(hit_positions)

    def __repr__(self) -> str:
        return (f"QueryReady(num_hit_blocks={self.num_hit_blocks}, lease={self.lease.hex()}, "
                f"hit_positions={self.hit_positions})")


class EngineRpcClient:
    """Client with the method names, argument order and return values of the
    reference's ``EngineRpcClient`` (python/pegaflow/pegaflow.pyi:69-300)."""

    def __init__(self, endpoint: str | None = None):
        self._endpoint = endpoint or ("http://" + DEFAULT_ENDPOINT)
        target = self._endpoint.split("://", 1)[-1]
        self._channel = grpc.insecure_channel(
            target, options=[("grpc.max_receive_message_length", 256 << 20),
                             ("grpc.max_send_message_length", 256 << 20)])
        self._calls = {
            name: self._channel.unary_unary(f"/{SERVICE}/{name}",
                                            request_serializer=req.SerializeToString,
                                            response_deserializer=resp.FromString)
            for name, (req, resp) in METHODS.items()}

    def endpoint(self) -> str:
        return self._endpoint

    def close(self) -> None:
        self.stop_session_watcher()
        self._channel.close()

    def start_session_watcher(self, instance_id: str, namespace: str, tp_size: int,
                              world_size: int) -> None:
        """Open the liveness stream and hold it for the life of this client (or
        process): when it ends, the server drops the instance.  Calling again
        replaces the previous stream (pegaflow.pyi:290-315)."""
        self.stop_session_watcher()
        call = self._channel.unary_stream(
            f"/{SERVICE}/Session", request_serializer=SessionRequest.SerializeToString,
            response_deserializer=SessionEvent.FromString)(
                SessionRequest(instance_id=instance_id, namespace=namespace, tp_size=tp_size,
                               world_size=world_size))

        def drain():
            try:
                for _event in call:
                    pass
            except grpc.RpcError:
                pass

        thread = threading.Thread(target=drain, name="pegaflow-session", daemon=True)
        thread.start()
        self._session = (call, thread)

    def stop_session_watcher(self) -> None:
        session = getattr(self, "_session", None)
        if session is not None:
            session[0].cancel()
            session[1].join(timeout=5)
            self._session = None

    def _call(self, name, request):
        try:
            return self._calls[name](request, timeout=120)
        except grpc.RpcError as err:
            code, detail = err.code(), err.details()
            if code in (grpc.StatusCode.INVALID_ARGUMENT, grpc.StatusCode.FAILED_PRECONDITION):
                raise RpcRejected(detail, code.name) from None
            raise PegaFlowError(f"{code.name}: {detail}", code.name) from None

    def health(self) -> tuple[bool, str]:
        r = self._call("Health", HealthRequest())
        return r.status.ok, r.status.message

    def register_context_batch(self, instance_id: str, namespace: str, tp_rank: int, pp_rank: int,
                               tp_size: int, world_size: int, device_id: int,
                               layer_names: Sequence[str], wrapper_bytes_list: Sequence[bytes],
                               num_blocks_list: Sequence[int], bytes_per_block_list: Sequence[int],
                               kv_stride_bytes_list: Sequence[int], segments_list: Sequence[int],
                               transfer_backend: str, page_first: bool,
                               layer_group_ids: Sequence[int] | None = None) -> tuple[bool, str]:
        mode = TransferMode.from_name(transfer_backend)
        req = RegisterContextRequest(
            instance_id=instance_id, namespace=namespace, tp_rank=tp_rank, tp_size=tp_size,
            world_size=world_size, device_id=device_id, layer_names=list(layer_names),
            wrapper_bytes=list(wrapper_bytes_list), num_blocks=list(num_blocks_list),
            bytes_per_block=list(bytes_per_block_list), kv_stride_bytes=list(kv_stride_bytes_list),
            segments=list(segments_list), pp_rank=pp_rank, client_version=PROTOCOL_VERSION,
            transfer_mode=1 if mode == TransferMode.KERNEL else 0, page_first=page_first,
            layer_group_ids=list(layer_group_ids or []))
        r = self._call("RegisterContextBatch", req)
        return r.status.ok, r.status.message

    def save(self, instance_id: str, tp_rank: int, pp_rank: int, device_id: int,
             saves: Sequence[tuple[str, Sequence[int], Sequence[bytes]]]) -> tuple[bool, str]:
        req = SaveRequest(instance_id=instance_id, tp_rank=tp_rank, device_id=device_id,
                          pp_rank=pp_rank,
                          saves=[SaveLayer(layer_name=n, block_ids=list(ids), block_hashes=list(h))
                                 for n, ids, h in saves])
        r = self._call("Save", req)
        return r.status.ok, r.status.message

    def load(self, instance_id: str, tp_rank: int, device_id: int, load_state_shm: str,
             layer_groups: Sequence[Sequence[str]],
             loads: Sequence[tuple[bytes, Sequence[Sequence[int | None]]]]) -> tuple[bool, str]:
        req = LoadRequest(instance_id=instance_id, tp_rank=tp_rank, device_id=device_id,
                          load_state_shm=load_state_shm,
                          groups=[LoadGroup(layer_names=list(g)) for g in layer_groups])
        for lease, by_group in loads:
            ll = req.loads.add(lease=lease)
            for ids in by_group:
                group = ll.block_ids_by_group.add()
                for b in ids:
                    target = group.targets.add()
                    if b is not None:
                        target.block_id = int(b)
        r = self._call("Load", req)
        return r.status.ok, r.status.message

    def query_prefetch(self, instance_id: str, block_hashes: Sequence[bytes], req_id: str,
                       wait_for_full_prefix: bool = False, group_id: int = 0):
        """-> QueryLoading or QueryReady."""
        r = self._call("QueryPrefetch", QueryRequest(
            instance_id=instance_id, block_hashes=list(block_hashes), req_id=req_id,
            wait_for_full_prefix=wait_for_full_prefix, group_id=group_id))
        if r.WhichOneof("outcome") == "loading":
            return QueryLoading()
        return QueryReady(r.ready.num_hit_blocks, bytes(r.ready.lease), list(r.ready.hit_positions))

    def release(self, lease: bytes) -> None:
        self._call("Release", ReleaseRequest(lease=lease))

    def unregister_context(self, instance_id: str) -> tuple[bool, str]:
        r = self._call("UnregisterContext", UnregisterRequest(instance_id=instance_id))
        return r.status.ok, r.status.message

    def shutdown(self) -> tuple[bool, str]:
        r = self._call("Shutdown", ShutdownRequest())
        return r.status.ok, r.status.message
