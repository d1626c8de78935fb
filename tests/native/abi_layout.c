/*
 * The layout of every struct that crosses the C ABI of libpegahip, pinned from
 * plain C: size and the offset of each field on LP64 (x86-64 Linux, the only
 * target), checked at compile time against include/pegahip.h.  A change of the
 * header that moves a field stops this file from compiling; a binding in
 * another language (the Rust `#[repr(C)]` mirrors, the ctypes mirrors of
 * pegaflow_amd/_lib.py) is correct when it reproduces exactly these numbers.
 * Run, the program prints them as JSON for such a comparison.
 *
 * Needs no HIP: gcc -std=c11 -pedantic -Werror -I. tests/native/abi_layout.c
 */
#include <stddef.h>
#include <stdio.h>

#include "include/pegahip.h"

static int first_struct = 1, first_field = 1;

#define BEGIN(type, bytes)                                                  \
  _Static_assert(sizeof(type) == (bytes), "sizeof(" #type ")");             \
  printf("%s\n  \"" #type "\": {\"size\": %zu, \"fields\": {", first_struct ? "" : ",", \
         sizeof(type));                                                     \
  first_struct = 0;                                                         \
  first_field = 1
#define FIELD(type, field, at)                                              \
  _Static_assert(offsetof(type, field) == (at), #type "." #field);          \
  printf("%s\"" #field "\": %zu", first_field ? "" : ", ", offsetof(type, field)); \
  first_field = 0
#define END() printf("}}")

int main(void) {
  printf("{");

  BEGIN(pf_host_mem, 32);
  FIELD(pf_host_mem, host, 0);
  FIELD(pf_host_mem, device, 8);
  FIELD(pf_host_mem, size, 16);
  FIELD(pf_host_mem, strategy, 24);
  FIELD(pf_host_mem, numa_node, 28);
  END();

  BEGIN(pf_kv_layout, 72);
  FIELD(pf_kv_layout, data_ptr, 0);
  FIELD(pf_kv_layout, size_bytes, 8);
  FIELD(pf_kv_layout, num_blocks, 16);
  FIELD(pf_kv_layout, block_stride_bytes, 24);
  FIELD(pf_kv_layout, segment_bytes, 32);
  FIELD(pf_kv_layout, segments, 40);
  FIELD(pf_kv_layout, padded_segment_bytes, 48);
  FIELD(pf_kv_layout, kv_stride_bytes, 56);
  FIELD(pf_kv_layout, split, 64);
  FIELD(pf_kv_layout, reserved, 68);
  END();

  BEGIN(pf_block_copy, 16);
  FIELD(pf_block_copy, addr, 0);
  FIELD(pf_block_copy, bytes, 8);
  END();

  /* transfer/mod.rs:36-44 of the reference: device, host, host_device, size,
   * device_allocation, host_allocation, eight bytes each. */
  BEGIN(pf_fill_unit, 40);
  FIELD(pf_fill_unit, layer, 0);
  FIELD(pf_fill_unit, first, 8);
  FIELD(pf_fill_unit, count, 16);
  FIELD(pf_fill_unit, slot_offset, 24);
  FIELD(pf_fill_unit, fill, 32);
  END();

  BEGIN(pf_copy_desc, 48);
  FIELD(pf_copy_desc, device, 0);
  FIELD(pf_copy_desc, host, 8);
  FIELD(pf_copy_desc, host_device, 16);
  FIELD(pf_copy_desc, size, 24);
  FIELD(pf_copy_desc, device_allocation, 32);
  FIELD(pf_copy_desc, host_allocation, 40);
  END();

  BEGIN(pf_merged_range, 24);
  FIELD(pf_merged_range, device, 0);
  FIELD(pf_merged_range, host, 8);
  FIELD(pf_merged_range, size, 16);
  END();

  BEGIN(pf_host_block, 80);
  FIELD(pf_host_block, seg_host, 0);
  FIELD(pf_host_block, seg_device, 16);
  FIELD(pf_host_block, seg_alloc, 32);
  FIELD(pf_host_block, seg_size, 48);
  FIELD(pf_host_block, num_segments, 64);
  FIELD(pf_host_block, reserved, 68);
  FIELD(pf_host_block, host_offset, 72);
  END();

  BEGIN(pf_layer_transfer, 104);
  FIELD(pf_layer_transfer, layer_name, 0);
  FIELD(pf_layer_transfer, layout, 8);
  FIELD(pf_layer_transfer, block_idx, 80);
  FIELD(pf_layer_transfer, blocks, 88);
  FIELD(pf_layer_transfer, n_blocks, 96);
  END();

  BEGIN(pf_layer_blocks, 184);
  FIELD(pf_layer_blocks, layer_name, 0);
  FIELD(pf_layer_blocks, layout, 8);
  FIELD(pf_layer_blocks, block_ids, 80);
  FIELD(pf_layer_blocks, n_blocks, 88);
  FIELD(pf_layer_blocks, host, 96);
  FIELD(pf_layer_blocks, host_device, 112);
  FIELD(pf_layer_blocks, host_len, 128);
  FIELD(pf_layer_blocks, host_stride, 144);
  FIELD(pf_layer_blocks, page_host, 152);
  FIELD(pf_layer_blocks, page_host_device, 160);
  FIELD(pf_layer_blocks, page_offset, 168);
  FIELD(pf_layer_blocks, page_len, 176);
  END();

  BEGIN(pf_xfer_config, 48);
  FIELD(pf_xfer_config, staging_slot_bytes, 0);
  FIELD(pf_xfer_config, staging_slots, 8);
  FIELD(pf_xfer_config, zerocopy_max_workgroups, 12);
  FIELD(pf_xfer_config, auto_staged_min_bytes, 16);
  FIELD(pf_xfer_config, tile_unroll, 24);
  FIELD(pf_xfer_config, copy_stream, 28);
  FIELD(pf_xfer_config, auto_staged_min_call_bytes, 32);
  FIELD(pf_xfer_config, staged_group_bytes, 40);
  END();

  BEGIN(pf_alloc_region, 24);
  FIELD(pf_alloc_region, offset_bytes, 0);
  FIELD(pf_alloc_region, size_bytes, 8);
  FIELD(pf_alloc_region, token, 16);
  END();

  BEGIN(pf_pool_config, 40);
  FIELD(pf_pool_config, capacity, 0);
  FIELD(pf_pool_config, num_shards, 8);
  FIELD(pf_pool_config, use_hugepages, 12);
  FIELD(pf_pool_config, ssd_enabled, 16);
  FIELD(pf_pool_config, n_numa_nodes, 20);
  FIELD(pf_pool_config, numa_nodes, 24);
  FIELD(pf_pool_config, unit_size_hint, 32);
  END();

  BEGIN(pf_allocation, 32);
  FIELD(pf_allocation, handle, 0);
  FIELD(pf_allocation, host, 8);
  FIELD(pf_allocation, device, 16);
  FIELD(pf_allocation, size, 24);
  END();

  BEGIN(pf_worker_layers, 40);
  FIELD(pf_worker_layers, device_id, 0);
  FIELD(pf_worker_layers, tp_rank, 4);
  FIELD(pf_worker_layers, pp_rank, 8);
  FIELD(pf_worker_layers, n_layers, 12);
  FIELD(pf_worker_layers, layer_names, 16);
  FIELD(pf_worker_layers, layouts, 24);
  FIELD(pf_worker_layers, group_ids, 32);
  END();

  BEGIN(pf_task_result, 112);
  FIELD(pf_task_result, status, 0);
  FIELD(pf_task_result, done, 4);
  FIELD(pf_task_result, bytes, 8);
  FIELD(pf_task_result, elapsed_ms, 16);
  FIELD(pf_task_result, paths, 24);
  FIELD(pf_task_result, staged_groups, 28);
  FIELD(pf_task_result, zero_copy_launches, 32);
  FIELD(pf_task_result, link_copies, 36);
  FIELD(pf_task_result, resolve_ms, 40);
  FIELD(pf_task_result, queue_ms, 48);
  FIELD(pf_task_result, convert_ms, 56);
  FIELD(pf_task_result, plan_ms, 64);
  FIELD(pf_task_result, staging_alloc_ms, 72);
  FIELD(pf_task_result, enqueue_ms, 80);
  FIELD(pf_task_result, sync_ms, 88);
  FIELD(pf_task_result, device_first_ms, 96);
  FIELD(pf_task_result, device_ms, 104);
  END();

  BEGIN(pf_worker_pool_config, 40);
  FIELD(pf_worker_pool_config, device_id, 0);
  FIELD(pf_worker_pool_config, numa_node, 4);
  FIELD(pf_worker_pool_config, transfer_mode, 8);
  FIELD(pf_worker_pool_config, use_descriptor_backends, 12);
  FIELD(pf_worker_pool_config, staging_slot_bytes, 16);
  FIELD(pf_worker_pool_config, auto_staged_min_bytes, 24);
  FIELD(pf_worker_pool_config, lazy_staging, 32);
  FIELD(pf_worker_pool_config, side_copy_streams, 36);
  END();

  BEGIN(pf_engine_config, 80);
  FIELD(pf_engine_config, pool_size, 0);
  FIELD(pf_engine_config, use_hugepages, 8);
  FIELD(pf_engine_config, numa_aware, 12);
  FIELD(pf_engine_config, pool_shards, 16);
  FIELD(pf_engine_config, blockwise_alloc, 20);
  FIELD(pf_engine_config, ssd_enabled, 24);
  FIELD(pf_engine_config, use_descriptor_backends, 28);
  FIELD(pf_engine_config, unit_size_hint, 32);
  FIELD(pf_engine_config, lease_ttl_ms, 40);
  FIELD(pf_engine_config, auto_staged_min_bytes, 48);
  FIELD(pf_engine_config, staging_slot_bytes, 56);
  FIELD(pf_engine_config, lazy_staging, 64);
  FIELD(pf_engine_config, kernel_mode_zerocopy, 68);
  FIELD(pf_engine_config, side_copy_streams, 72);
  FIELD(pf_engine_config, reserved, 76);
  END();

  BEGIN(pf_layer_save, 40);
  FIELD(pf_layer_save, layer_name, 0);
  FIELD(pf_layer_save, block_ids, 8);
  FIELD(pf_layer_save, block_hashes, 16);
  FIELD(pf_layer_save, block_hash_lens, 24);
  FIELD(pf_layer_save, n_blocks, 32);
  END();

  BEGIN(pf_save_profile, 64);
  FIELD(pf_save_profile, validate_ms, 0);
  FIELD(pf_save_profile, filter_ms, 8);
  FIELD(pf_save_profile, alloc_ms, 16);
  FIELD(pf_save_profile, assemble_ms, 24);
  FIELD(pf_save_profile, transfer_ms, 32);
  FIELD(pf_save_profile, publish_ms, 40);
  FIELD(pf_save_profile, total_ms, 48);
  FIELD(pf_save_profile, bytes, 56);
  END();

  BEGIN(pf_load_request, 24);
  FIELD(pf_load_request, lease, 0);
  FIELD(pf_load_request, dest_block_ids, 8);
  FIELD(pf_load_request, n_blocks, 16);
  END();

  BEGIN(pf_ipc_tensor, 104);
  FIELD(pf_ipc_tensor, handle, 0);
  FIELD(pf_ipc_tensor, alloc_size, 64);
  FIELD(pf_ipc_tensor, offset, 72);
  FIELD(pf_ipc_tensor, size_bytes, 80);
  FIELD(pf_ipc_tensor, device_uuid, 88);
  END();

  printf("\n}\n");
  return 0;
}
