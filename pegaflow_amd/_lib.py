"""ctypes binding of ``libpegahip.so`` (declared in ``include/pegahip.h``).

The library is the product: if it is missing this module raises, there is no
Python or CPU fallback for anything that moves bytes.
"""

from __future__ import annotations

import ctypes as C
import importlib.util
import os
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpegahip.so")

PF_OK = 0
PF_ERR_INVALID_ARGUMENT = -1
PF_ERR_STORAGE = -2
PF_ERR_DEVICE_INIT = -3
PF_ERR_WORKER_MISSING = -4
PF_ERR_INSTANCE_MISSING = -5
PF_ERR_BUFFER_TOO_SMALL = -6

PF_HOST_REGULAR = 0
PF_HOST_HIP_ALLOC = 1
PF_HOST_HUGEPAGES = 2

PF_MODE_DIRECT = 0
PF_MODE_KERNEL = 1
PF_MODE_ZEROCOPY = 2

PF_PATH_AUTO = 0
PF_PATH_ZEROCOPY = 1
PF_PATH_STAGED = 2

PF_TASK_PATH_STAGED = 1
PF_TASK_PATH_ZEROCOPY = 2
PF_TASK_PATH_DESCRIPTORS = 4

u64 = C.c_uint64
u32 = C.c_uint32
vp = C.c_void_p


class PfHostMem(C.Structure):
    _fields_ = [("host", vp), ("device", u64), ("size", u64), ("strategy", C.c_int32),
                ("numa_node", C.c_int32)]


class PfKvLayout(C.Structure):
    _fields_ = [
        ("data_ptr", u64), ("size_bytes", u64), ("num_blocks", u64), ("block_stride_bytes", u64),
        ("segment_bytes", u64), ("segments", u64), ("padded_segment_bytes", u64),
        ("kv_stride_bytes", u64), ("split", u32), ("reserved", u32),
    ]


class PfBlockCopy(C.Structure):
    _fields_ = [("addr", u64), ("bytes", u64)]


class PfCopyDesc(C.Structure):
    _fields_ = [("device", u64), ("host", vp), ("host_device", u64), ("size", u64),
                ("device_allocation", u64), ("host_allocation", u64)]


class PfMergedRange(C.Structure):
    _fields_ = [("device", u64), ("host", vp), ("size", u64)]


class PfHostBlock(C.Structure):
    _fields_ = [("seg_host", vp * 2), ("seg_device", u64 * 2), ("seg_alloc", u64 * 2),
                ("seg_size", u64 * 2), ("num_segments", u32), ("reserved", u32),
                ("host_offset", u64)]


class PfLayerTransfer(C.Structure):
    _fields_ = [("layer_name", C.c_char_p), ("layout", PfKvLayout),
                ("block_idx", C.POINTER(u64)), ("blocks", C.POINTER(PfHostBlock)),
                ("n_blocks", u64)]


class PfLayerBlocks(C.Structure):
    _fields_ = [
        ("layer_name", C.c_char_p), ("layout", PfKvLayout), ("block_ids", C.POINTER(u32)),
        ("n_blocks", u64), ("host", vp * 2), ("host_device", u64 * 2), ("host_len", u64 * 2),
        ("host_stride", u64), ("page_host", C.POINTER(u64)), ("page_host_device", C.POINTER(u64)),
        ("page_offset", u64), ("page_len", u64),
    ]


class PfXferConfig(C.Structure):
    _fields_ = [("staging_slot_bytes", u64), ("staging_slots", u32),
                ("zerocopy_max_workgroups", u32), ("auto_staged_min_bytes", u64),
                ("tile_unroll", u32), ("copy_stream", u32),
                ("auto_staged_min_call_bytes", u64), ("staged_group_bytes", u64)]


class PfFillUnit(C.Structure):
    _fields_ = [("layer", u64), ("first", u64), ("count", u64), ("slot_offset", u64), ("fill", u64)]


class PfAllocRegion(C.Structure):
    _fields_ = [("offset_bytes", u64), ("size_bytes", u64), ("token", u64)]


class PfPoolConfig(C.Structure):
    _fields_ = [("capacity", u64), ("num_shards", u32), ("use_hugepages", u32),
                ("ssd_enabled", u32), ("n_numa_nodes", u32), ("numa_nodes", C.POINTER(C.c_int32)),
                ("unit_size_hint", u64)]


class PfAllocation(C.Structure):
    _fields_ = [("handle", u64), ("host", vp), ("device", u64), ("size", u64)]


class PfWorkerLayers(C.Structure):
    _fields_ = [("device_id", C.c_int32), ("tp_rank", u32), ("pp_rank", u32), ("n_layers", u32),
                ("layer_names", C.POINTER(C.c_char_p)), ("layouts", C.POINTER(PfKvLayout)),
                ("group_ids", C.POINTER(u32))]


class PfTaskResult(C.Structure):
    _fields_ = [("status", C.c_int32), ("done", C.c_int32), ("bytes", u64),
                ("elapsed_ms", C.c_double), ("paths", u32), ("staged_groups", u32),
                ("zero_copy_launches", u32), ("link_copies", u32),
                ("resolve_ms", C.c_double), ("queue_ms", C.c_double), ("convert_ms", C.c_double),
                ("plan_ms", C.c_double), ("staging_alloc_ms", C.c_double),
                ("enqueue_ms", C.c_double), ("sync_ms", C.c_double),
                ("device_first_ms", C.c_double), ("device_ms", C.c_double)]


class PfWorkerPoolConfig(C.Structure):
    _fields_ = [("device_id", C.c_int32), ("numa_node", C.c_int32), ("transfer_mode", C.c_int32),
                ("use_descriptor_backends", u32), ("staging_slot_bytes", u64),
                ("auto_staged_min_bytes", u64), ("lazy_staging", u32), ("side_copy_streams", u32)]


class PfEngineConfig(C.Structure):
    _fields_ = [("pool_size", u64), ("use_hugepages", u32), ("numa_aware", u32),
                ("pool_shards", u32), ("blockwise_alloc", u32), ("ssd_enabled", u32),
                ("use_descriptor_backends", u32), ("unit_size_hint", u64),
                ("lease_ttl_ms", u64), ("auto_staged_min_bytes", u64),
                ("staging_slot_bytes", u64), ("lazy_staging", u32),
                ("kernel_mode_zerocopy", u32), ("side_copy_streams", u32), ("reserved", u32)]


class PfIpcTensor(C.Structure):
    _fields_ = [("handle", C.c_uint8 * 64), ("alloc_size", u64), ("offset", u64),
                ("size_bytes", u64), ("device_uuid", C.c_uint8 * 16)]


class PfLayerSave(C.Structure):
    _fields_ = [("layer_name", C.c_char_p), ("block_ids", C.POINTER(u64)),
                ("block_hashes", C.POINTER(C.POINTER(C.c_uint8))),
                ("block_hash_lens", C.POINTER(u32)), ("n_blocks", u64)]


class PfLoadRequest(C.Structure):
    _fields_ = [("lease", u64), ("dest_block_ids", C.POINTER(C.POINTER(C.c_int64))),
                ("n_blocks", u64)]


class PfSaveProfile(C.Structure):
    _fields_ = [("validate_ms", C.c_double), ("filter_ms", C.c_double), ("alloc_ms", C.c_double),
                ("assemble_ms", C.c_double), ("transfer_ms", C.c_double),
                ("publish_ms", C.c_double), ("total_ms", C.c_double), ("bytes", u64)]


# name -> (restype, argtypes).  Every symbol include/pegahip.h declares.
PROTOTYPES = {
    "pf_last_error": (C.c_char_p, []),
    "pf_version": (C.c_char_p, []),
    "pf_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "pf_set_device": (C.c_int, [C.c_int]),
    "pf_get_device": (C.c_int, [C.POINTER(C.c_int)]),
    "pf_device_synchronize": (C.c_int, []),
    "pf_device_numa_node": (C.c_int, [C.c_int, C.POINTER(C.c_int)]),
    "pf_device_name": (C.c_int, [C.c_int, C.c_char_p, C.c_size_t]),
    "pf_stream_create": (C.c_int, [C.POINTER(vp)]),
    "pf_stream_wrap": (C.c_int, [vp, C.POINTER(vp)]),
    "pf_stream_destroy": (C.c_int, [vp]),
    "pf_stream_synchronize": (C.c_int, [vp]),
    "pf_streams_run_concurrently": (C.c_int, [vp, vp, C.POINTER(C.c_int)]),
    "pf_stream_wait_event": (C.c_int, [vp, vp]),
    "pf_stream_native": (vp, [vp]),
    "pf_event_create": (C.c_int, [C.c_int, C.POINTER(vp)]),
    "pf_event_destroy": (C.c_int, [vp]),
    "pf_event_record": (C.c_int, [vp, vp]),
    "pf_event_synchronize": (C.c_int, [vp]),
    "pf_event_query": (C.c_int, [vp, C.POINTER(C.c_int)]),
    "pf_event_elapsed_ms": (C.c_int, [vp, vp, C.POINTER(C.c_float)]),
    "pf_host_alloc": (C.c_int, [u64, C.c_int, C.c_int, C.POINTER(PfHostMem)]),
    "pf_host_free": (C.c_int, [C.POINTER(PfHostMem)]),
    "pf_touch_threads": (u64, [u64]),
    "pf_huge_page_size": (u64, []),
    "pf_dev_malloc": (C.c_int, [u64, C.POINTER(u64)]),
    "pf_dev_free": (C.c_int, [u64]),
    "pf_dev_memset": (C.c_int, [u64, C.c_int, u64]),
    "pf_dev_copy_from_host": (C.c_int, [u64, vp, u64]),
    "pf_dev_copy_to_host": (C.c_int, [vp, u64, u64]),
    "pf_memcpy_h2d_async": (C.c_int, [u64, vp, u64, vp]),
    "pf_memcpy_d2h_async": (C.c_int, [vp, u64, u64, vp]),
    "pf_layout_new": (C.c_int, [u64, u64, u64, u64, u64, u64, C.POINTER(PfKvLayout)]),
    "pf_layout_with_block_stride": (C.c_int, [C.POINTER(PfKvLayout), u64]),
    "pf_layout_with_ssd_padding": (C.c_int, [C.POINTER(PfKvLayout), u64]),
    "pf_layout_block_copies": (C.c_int, [C.POINTER(PfKvLayout), u64, C.POINTER(PfBlockCopy),
                                         C.POINTER(u32)]),
    "pf_layout_padded_block_bytes": (u64, [C.POINTER(PfKvLayout)]),
    "pf_layout_block_bytes": (u64, [C.POINTER(PfKvLayout)]),
    "pf_merge_copies": (C.c_int, [C.POINTER(PfCopyDesc), u64, C.POINTER(PfMergedRange),
                                  C.POINTER(u64)]),
    "pf_backend_create": (C.c_int, [C.c_int, C.POINTER(vp)]),
    "pf_backend_destroy": (C.c_int, [vp]),
    "pf_backend_name": (C.c_char_p, [vp]),
    "pf_backend_h2d": (C.c_int, [vp, C.POINTER(PfCopyDesc), u64, vp]),
    "pf_backend_d2h": (C.c_int, [vp, C.POINTER(PfCopyDesc), u64, vp]),
    "pf_desc_copy_noalloc": (C.c_int, [C.POINTER(PfCopyDesc), u64, C.c_int, vp]),
    "pf_desc_copy_noalloc_max": (u64, []),
    "pf_transfer_mode_from_name": (C.c_int, [C.c_char_p, C.POINTER(C.c_int)]),
    "pf_build_copy_descs": (C.c_int, [C.POINTER(PfLayerTransfer), u64, C.POINTER(PfCopyDesc), u64,
                                      C.POINTER(u64), C.POINTER(u64)]),
    "pf_xfer_create": (C.c_int, [C.POINTER(PfXferConfig), C.POINTER(vp)]),
    "pf_xfer_destroy": (C.c_int, [vp]),
    "pf_xfer_save": (C.c_int, [vp, C.POINTER(PfLayerBlocks), u64, C.c_int, vp]),
    "pf_xfer_load": (C.c_int, [vp, C.POINTER(PfLayerBlocks), u64, C.c_int, vp]),
    "pf_xfer_set_layer_events": (C.c_int, [vp, C.POINTER(vp), u64]),
    "pf_xfer_last_path": (C.c_int, [vp]),
    "pf_xfer_last_kernel_ms": (C.c_int, [vp, C.POINTER(C.c_float), C.POINTER(u32)]),
    "pf_xfer_set_kernel_timing": (C.c_int, [vp, C.c_int]),
    "pf_plan_staged_fills": (C.c_int, [C.POINTER(u64), C.POINTER(u64), u64, u64, u64, u32,
                                       C.POINTER(PfFillUnit), u64, C.POINTER(u64), C.POINTER(u64)]),
    "pf_plain_copy": (C.c_int, [u64, u64, u64, u32, vp]),
    "pf_allocator_create": (C.c_int, [u64, u64, u32, C.POINTER(vp)]),
    "pf_allocator_destroy": (C.c_int, [vp]),
    "pf_allocator_allocate": (C.c_int, [vp, u64, C.POINTER(PfAllocRegion)]),
    "pf_allocator_free": (C.c_int, [vp, C.POINTER(PfAllocRegion)]),
    "pf_allocator_report": (C.c_int, [vp, C.POINTER(u64), C.POINTER(u64), C.POINTER(u64),
                                      C.POINTER(u64)]),
    "pf_pool_compute_unit_size": (u64, [u64, u64]),
    "pf_pool_create": (C.c_int, [C.POINTER(PfPoolConfig), C.POINTER(vp)]),
    "pf_pool_destroy": (C.c_int, [vp]),
    "pf_pool_allocate": (C.c_int, [vp, u64, C.c_int, C.POINTER(PfAllocation)]),
    "pf_pool_free": (C.c_int, [C.POINTER(PfAllocation)]),
    "pf_pool_usage": (C.c_int, [vp, C.POINTER(u64), C.POINTER(u64)]),
    "pf_pool_largest_free": (C.c_int, [vp, C.c_int, C.POINTER(u64)]),
    "pf_pool_is_numa": (C.c_int, [vp]),
    "pf_numa_format_cpu_list": (C.c_int, [C.POINTER(u64), u64, C.c_char_p, C.c_size_t]),
    "pf_numa_parse_cpulist": (C.c_int, [C.c_char_p, C.POINTER(u64), u64, C.POINTER(u64)]),
    "pf_numa_pin_thread": (C.c_int, [C.c_int]),
    "pf_numa_node_count": (C.c_int, []),
    "pf_numa_query_pages": (C.c_int, [C.POINTER(vp), u64, C.POINTER(C.c_int)]),
    "pf_numa_node_of_pci": (C.c_int, [C.c_char_p, C.c_char_p]),
    "pf_build_page_layout": (C.c_int, [C.POINTER(u64), C.POINTER(u64), u64, u64, C.POINTER(u64),
                                       C.POINTER(u64), C.POINTER(u64), C.POINTER(u64),
                                       C.POINTER(u64), C.POINTER(u64)]),
    "pf_topology_seal": (C.c_int, [C.POINTER(PfWorkerLayers), u32, u32, C.c_int, C.POINTER(vp)]),
    "pf_topology_destroy": (C.c_int, [vp]),
    "pf_topology_num_layers": (u64, [vp]),
    "pf_topology_total_slots": (u64, [vp]),
    "pf_topology_num_groups": (u64, [vp]),
    "pf_topology_group_of_layer": (C.c_int, [vp, u64, C.POINTER(u32)]),
    "pf_topology_group_total_slots": (C.c_int, [vp, u32, C.POINTER(u64)]),
    "pf_topology_is_page_first": (C.c_int, [vp]),
    "pf_topology_layer_id": (C.c_int, [vp, C.c_char_p, C.POINTER(u64)]),
    "pf_topology_slot_index": (C.c_int, [vp, u64, u64, C.POINTER(u64)]),
    "pf_topology_page_placement": (C.c_int, [vp, u64, C.POINTER(u64), C.POINTER(u64)]),
    "pf_topology_shard_page_size": (C.c_int, [vp, u64, C.POINTER(u64)]),
    "pf_topology_shard_layer_count": (C.c_int, [vp, u64, C.POINTER(u64)]),
    "pf_load_state_create": (C.c_int, [C.POINTER(vp)]),
    "pf_load_state_attach": (C.c_int, [C.c_char_p, C.POINTER(vp)]),
    "pf_load_state_destroy": (C.c_int, [vp]),
    "pf_load_state_name": (C.c_char_p, [vp]),
    "pf_load_state_get": (C.c_int64, [vp]),
    "pf_load_state_set": (C.c_int, [vp, C.c_int64]),
    "pf_worker_pool_spawn": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(vp)]),
    "pf_worker_pool_spawn_ex": (C.c_int, [C.POINTER(PfWorkerPoolConfig), C.POINTER(vp)]),
    "pf_worker_pool_staging_bytes": (u64, [vp]),
    "pf_worker_pool_destroy": (C.c_int, [vp]),
    "pf_worker_submit_load": (C.c_int, [vp, C.POINTER(PfLayerTransfer), u64, C.c_char_p,
                                        C.POINTER(vp)]),
    "pf_worker_submit_save": (C.c_int, [vp, C.POINTER(PfLayerTransfer), u64, C.POINTER(vp)]),
    "pf_worker_pool_queue_clashes": (u64, [vp]),
    "pf_worker_stream_report": (C.c_int, [C.c_int, C.POINTER(u64), C.POINTER(u64),
                                          C.POINTER(u64)]),
    "pf_task_wait": (C.c_int, [vp, C.c_int, C.POINTER(PfTaskResult)]),
    "pf_task_destroy": (C.c_int, [vp]),
    "pf_engine_create": (C.c_int, [C.POINTER(PfEngineConfig), C.POINTER(vp)]),
    "pf_engine_destroy": (C.c_int, [vp]),
    "pf_engine_register_context_layer_batch": (C.c_int, [
        vp, C.c_char_p, C.c_char_p, C.c_int, u64, u64, u64, u64, u64, C.POINTER(C.c_char_p),
        C.POINTER(u64), C.POINTER(u64), C.POINTER(u64), C.POINTER(u64), C.POINTER(u64),
        C.POINTER(u64), C.POINTER(u64), C.POINTER(u32), C.c_int, C.c_int]),
    "pf_engine_unregister_instance": (C.c_int, [vp, C.c_char_p]),
    "pf_engine_batch_save": (C.c_int, [vp, C.c_char_p, u64, u64, C.c_int, C.POINTER(PfLayerSave),
                                       u64]),
    "pf_engine_query_prefix": (C.c_int, [vp, C.c_char_p, C.POINTER(C.POINTER(C.c_uint8)),
                                         C.POINTER(u32), u64, C.POINTER(u64), C.POINTER(u64)]),
    "pf_engine_release_lease": (C.c_int, [vp, u64]),
    "pf_engine_batch_load": (C.c_int, [vp, C.c_char_p, u64, C.c_int, u64,
                                       C.POINTER(C.POINTER(C.c_char_p)), C.POINTER(u64), u64,
                                       C.POINTER(C.POINTER(C.c_int64)), u64, C.c_char_p,
                                       C.POINTER(vp)]),
    "pf_engine_last_save_profile": (C.c_int, [vp, C.POINTER(PfSaveProfile)]),
    "pf_engine_last_load_profile": (C.c_int, [vp, C.POINTER(PfTaskResult)]),
    "pf_engine_staging_bytes": (u64, [vp]),
    "pf_engine_batch_load_multi": (C.c_int, [vp, C.c_char_p, u64, C.c_int, u64,
                                             C.POINTER(C.POINTER(C.c_char_p)), C.POINTER(u64),
                                             C.POINTER(PfLoadRequest), u64, C.c_char_p,
                                             C.POINTER(vp)]),
    "pf_engine_query_group_membership": (C.c_int, [vp, C.c_char_p, u32,
                                                   C.POINTER(C.POINTER(C.c_uint8)),
                                                   C.POINTER(u32), u64, C.POINTER(C.c_uint8)]),
    "pf_engine_create_group_lease": (C.c_int, [vp, C.c_char_p, u32,
                                               C.POINTER(C.POINTER(C.c_uint8)), C.POINTER(u32),
                                               u64, C.POINTER(u64)]),
    "pf_engine_query_group_lease": (C.c_int, [vp, C.c_char_p, u32,
                                              C.POINTER(C.POINTER(C.c_uint8)), C.POINTER(u32),
                                              u64, C.c_int, C.POINTER(C.c_uint8),
                                              C.POINTER(u64)]),
    "pf_engine_pool_usage": (C.c_int, [vp, C.POINTER(u64), C.POINTER(u64)]),
    "pf_engine_cached_blocks": (u64, [vp]),
    "pf_engine_inflight_blocks": (u64, [vp]),
    "pf_engine_gc_stale_inflight": (u64, [vp, u64]),
    "pf_engine_evict_all": (u64, [vp]),
    "pf_device_uuid": (C.c_int, [C.c_int, C.POINTER(C.c_uint8)]),
    "pf_device_from_uuid": (C.c_int, [C.POINTER(C.c_uint8), C.POINTER(C.c_int)]),
    "pf_ipc_export": (C.c_int, [u64, u64, C.POINTER(PfIpcTensor)]),
    "pf_registry_create": (C.c_int, [C.POINTER(vp)]),
    "pf_registry_destroy": (C.c_int, [vp]),
    "pf_registry_register_layers": (C.c_int, [vp, C.c_char_p, C.c_int, u64, C.POINTER(C.c_char_p),
                                              C.POINTER(PfIpcTensor), C.POINTER(u64),
                                              C.POINTER(u64)]),
    "pf_registry_drop_context": (u64, [vp, C.c_char_p]),
    "pf_registry_drop_instance": (u64, [vp, C.c_char_p]),
    "pf_registry_clear": (u64, [vp]),
    "pf_registry_context_count": (u64, [vp]),
    "pf_server_register_context_batch": (C.c_int, [
        vp, vp, C.c_char_p, C.c_char_p, C.c_int, u64, u64, u64, u64, u64, C.POINTER(C.c_char_p),
        C.POINTER(PfIpcTensor), C.POINTER(u64), C.POINTER(u64), C.POINTER(u64), C.POINTER(u64),
        C.POINTER(u32), C.c_int, C.c_int]),
    "pf_engine_sweep_expired_leases": (u64, [vp]),
    "pf_engine_live_leases": (u64, [vp]),
}


class PegaHipError(RuntimeError):
    """A non-zero status from libpegahip; ``code`` > 0 is a hipError_t."""

    def __init__(self, code: int, message: str):
        super().__init__(f"[pegahip {code}] {message}")
        self.code = code
        self.message = message


class InvalidArgument(PegaHipError, ValueError):
    pass


class StorageError(PegaHipError):
    pass


class InstanceMissing(PegaHipError):
    pass


class WorkerMissing(PegaHipError):
    pass


_lib = None


def _bind_to_pytorch_hip_runtime() -> None:
    """PyTorch's ROCm wheels carry their own libamdhip64 (same SONAME as the
    system one).  Two HIP runtimes in one process do not both get the GPU, and
    which one a process ends up with would depend on import order.  When such
    a wheel is installed and PyTorch is not loaded yet, load its runtime first
    so that libpegahip binds to the copy PyTorch will use.  Set
    PEGAHIP_SYSTEM_HIP_RUNTIME=1 to keep the system runtime instead."""
    if "torch" in sys.modules or os.environ.get("PEGAHIP_SYSTEM_HIP_RUNTIME") == "1":
        return
    try:
        spec = importlib.util.find_spec("torch")
    except (ImportError, ValueError):
        return
    if spec is None or not spec.submodule_search_locations:
        return
    bundled = os.path.join(list(spec.submodule_search_locations)[0], "lib", "libamdhip64.so")
    if os.path.exists(bundled):
        try:
            C.CDLL(bundled, mode=C.RTLD_GLOBAL)
        except OSError:
            pass


def load():
    """Load libpegahip.so and set every prototype.  Raises if it is absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C pegaflow_amd/csrc` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`). "
            "pegaflow_amd has no fallback path.")
    _bind_to_pytorch_hip_runtime()
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status: int) -> None:
    if status == PF_OK:
        return
    msg = load().pf_last_error().decode(errors="replace")
    if status == PF_ERR_INVALID_ARGUMENT:
        raise InvalidArgument(status, msg)
    if status == PF_ERR_STORAGE:
        raise StorageError(status, msg)
    if status == PF_ERR_INSTANCE_MISSING:
        raise InstanceMissing(status, msg)
    if status == PF_ERR_WORKER_MISSING:
        raise WorkerMissing(status, msg)
    raise PegaHipError(status, msg)
