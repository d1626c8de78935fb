"""Writes ``reference_kats.json``: the known-answer vectors the reference's own
unit tests hold for the KV block transfer path, transcribed as DATA (inputs and
expected outputs) by reading those test files.  Nothing is imported or run
from the reference; every group cites the file and lines it was read from
(paths relative to the reference checkout).

Run:  python tests/golden/make_kats.py
"""

from __future__ import annotations

import json
import os

K = 1024

KATS = {
    # ------------------------------------------------------------------
    # pegaflow-core/src/layout.rs:288-474
    # args = [data_ptr, size_bytes, num_blocks, segment_bytes, kv_stride, segments]
    # ------------------------------------------------------------------
    "layout": [
        {
            "name": "dense_layout_addresses", "cite": "layout.rs:300-307",
            "new": [0x1000, K * K, 100, K, 0, 1],
            "expect": {"is_split": False, "padded_block_bytes": K,
                       "copies": {"0": [[0x1000, K]], "5": [[0x1000 + 5 * K, K]]},
                       "out_of_range": [100]},
        },
        {
            "name": "split_layout_addresses", "cite": "layout.rs:310-323",
            "new": [0x1000, 200 * K, 100, K, 100 * K, 2],
            "expect": {"is_split": True,
                       "copies": {"3": [[0x1000 + 3 * K, K], [0x1000 + 103 * K, K]]}},
        },
        {
            "name": "adjacent_kv_collapses_to_contiguous", "cite": "layout.rs:326-336",
            "new": [0x1000, 200 * K, 100, K, K, 2],
            "expect": {"is_split": False,
                       "copies": {"0": [[0x1000, 2 * K]], "1": [[0x1000 + 2 * K, 2 * K]]}},
        },
        {
            "name": "overlapping_kv_stride_rejected", "cite": "layout.rs:338-342",
            "new": [0x1000, 200 * K, 100, K, 512, 2],
            "expect": {"error_contains": "overlap"},
        },
        {
            "name": "split_kv_regions_must_not_overlap", "cite": "layout.rs:344-348",
            "new": [0x1000, 200 * K, 100, K, 2 * K, 2],
            "expect": {"error_contains": "overlaps blocks 2 apart"},
        },
        {
            "name": "sparse_split_layout_can_have_interleaved_disjoint_segments",
            "cite": "layout.rs:350-371",
            "new": [0x1000, 1600, 2, 100, 500, 2], "with_block_stride": 1000,
            "expect": {"is_split": True,
                       "copies": {"0": [[0x1000, 100], [0x1000 + 500, 100]],
                                  "1": [[0x1000 + 1000, 100], [0x1000 + 1500, 100]]}},
        },
        {
            "name": "adjacent_kv_default_stride_keeps_blocks_disjoint", "cite": "layout.rs:373-387",
            "new": [0x1000, 200 * K, 100, K, K, 2],
            "expect": {"is_split": False,
                       "copies": {"0": [[0x1000, 2 * K]], "1": [[0x1000 + 2 * K, 2 * K]]}},
        },
        {
            "name": "block_stride_decouples_step_from_copy_size", "cite": "layout.rs:389-408",
            "new": [0x10000, 8 * 16384, 8, 8192, 0, 1], "with_block_stride": 16384,
            "expect": {"is_split": False,
                       "copies": {"3": [[0x10000 + 3 * 16384, 8192]],
                                  "7": [[0x10000 + 7 * 16384, 8192]]}},
        },
        {
            "name": "block_stride_smaller_than_block_rejected", "cite": "layout.rs:415-421",
            "new": [0x1000, K * K, 100, K, 0, 1], "with_block_stride": 512,
            "expect": {"stride_error_contains": "blocks would overlap"},
        },
        {
            "name": "strided_layout_exceeds_region", "cite": "layout.rs:423-429",
            "new": [0x1000, 8 * K, 8, K, 0, 1], "with_block_stride": 4096,
            "expect": {"stride_error_contains": "too small"},
        },
        {
            "name": "split_overlaps_again_when_stride_grows", "cite": "layout.rs:431-438",
            "new": [0x1000, 200 * K, 100, K, 100 * K, 2], "with_block_stride": 2048,
            "expect": {"stride_error_contains": "overlaps blocks 50 apart"},
        },
        {
            "name": "null_pointer_rejected", "cite": "layout.rs:441-444",
            "new": [0, K, 10, 64, 0, 1],
            "expect": {"error_contains": "null"},
        },
        {
            "name": "memory_too_small_rejected", "cite": "layout.rs:446-450",
            "new": [0x1000, 5120, 10, K, 0, 1],
            "expect": {"error_contains": "too small"},
        },
        {
            "name": "ssd_padding_unaligned", "cite": "layout.rs:452-459",
            "new": [0x1000, 10_000_000, 100, 8848, 0, 1], "with_ssd_padding": 512,
            "expect": {"padded_segment_bytes": 9216, "padded_block_bytes": 9216},
        },
        {
            "name": "ssd_padding_aligned", "cite": "layout.rs:461-466",
            "new": [0x1000, K * K, 100, K, 0, 1], "with_ssd_padding": 512,
            "expect": {"padded_segment_bytes": K, "padded_block_bytes": K},
        },
        {
            "name": "ssd_padding_split", "cite": "layout.rs:468-473",
            "new": [0x1000, 10_000_000, 100, 8848, 900_000, 2], "with_ssd_padding": 512,
            "expect": {"is_split": True, "padded_segment_bytes": 9216,
                       "padded_block_bytes": 9216 * 2},
        },
    ],
    # ------------------------------------------------------------------
    # pegaflow-core/src/transfer/memcpy.rs:104-139
    # desc = [device, host_offset, size, device_allocation, host_allocation]
    # ------------------------------------------------------------------
    "merge": [
        {"name": "contiguous_same_allocations_merge", "cite": "memcpy.rs:124-133",
         "descs": [[100, 0, 4, 1, 2], [104, 4, 4, 1, 2]], "expect_sizes": [8]},
        {"name": "different_device_allocation", "cite": "memcpy.rs:135-137",
         "descs": [[100, 0, 4, 1, 2], [104, 4, 4, 3, 2]], "expect_sizes": [4, 4]},
        {"name": "different_host_allocation", "cite": "memcpy.rs:135-137",
         "descs": [[100, 0, 4, 1, 2], [104, 4, 4, 1, 4]], "expect_sizes": [4, 4]},
    ],
    # ------------------------------------------------------------------
    # pegaflow-core/src/instance/tests.rs:160-214 (build_page_layout) and
    # :125-158, :222-265 (sorted-name ids, page placement through registration)
    # ------------------------------------------------------------------
    "page_layout": [
        {"name": "single_shard_replica", "cite": "instance/tests.rs:163-172",
         "sets": [[0, 1, 2], [0, 1, 2]], "n_layers": 3, "padded": [512, 1024, 2048],
         "expect": {"shard_page_sizes": [3584], "layer_shard": [0, 0, 0],
                    "layer_offsets": [0, 512, 1536], "layer_bytes": [512, 1024, 2048]}},
        {"name": "layer_split_partitions_into_shards", "cite": "instance/tests.rs:179-193",
         "sets": [[0, 2], [1, 3]], "n_layers": 4, "padded": [512, 1024, 1536, 2048],
         "expect": {"layer_shard": [0, 1, 0, 1], "shard_page_sizes": [2048, 3072],
                    "layer_offsets": [0, 0, 512, 1024], "layer_bytes": [512, 1024, 1536, 2048]}},
        {"name": "rejects_overlapping_shards", "cite": "instance/tests.rs:197-203",
         "sets": [[0, 1], [1, 2]], "n_layers": 3, "padded": [512, 512, 512],
         "expect": {"error_contains": "claimed by shards"}},
        {"name": "rejects_uncovered_layer", "cite": "instance/tests.rs:208-214",
         "sets": [[0], [1]], "n_layers": 3, "padded": [512, 512, 512],
         "expect": {"error_contains": "no shard owner"}},
    ],
    "topology": [
        {"name": "single_worker_registration_seals_topology", "cite": "instance/tests.rs:76-120",
         "page_first": False, "tp_size": 1,
         "workers": [{"tp_rank": 0, "layers": ["layer_b", "layer_a", "layer_d", "layer_c"],
                      "segment_bytes": 1024}],
         "expect": {"num_layers": 4, "layer_id": {"layer_a": 0, "layer_d": 3},
                    "missing": ["layer_x"], "slot_index": [[2, 0, 2]], "total_slots": 4}},
        {"name": "page_first_collapses_slots_and_lays_out_page",
         "cite": "instance/tests.rs:125-158", "page_first": True, "tp_size": 1,
         "workers": [{"tp_rank": 0, "layers": ["layer_b", "layer_a", "layer_c"],
                      "segment_bytes": 1024}],
         "expect": {"num_layers": 3, "total_slots": 1,
                    "slot_index": [[0, 0, 0], [1, 0, 0], [2, 0, 0]],
                    "shard_page_size": {"0": 3072}, "shard_layer_count": {"0": 3},
                    "page_placement": {"0": [0, 1024], "1": [1024, 1024], "2": [2048, 1024]}}},
        {"name": "page_first_layer_split_seals_per_shard_slots",
         "cite": "instance/tests.rs:222-265", "page_first": True, "tp_size": 1,
         "workers": [{"tp_rank": 0, "layers": ["layer_a", "layer_c"], "segment_bytes": 1024},
                     {"tp_rank": 0, "layers": ["layer_b"], "segment_bytes": 1024}],
         "expect": {"num_layers": 3, "total_slots": 2,
                    "slot_index": [[0, 0, 0], [1, 0, 1], [2, 0, 0]],
                    "shard_page_size": {"0": 2048, "1": 1024},
                    "shard_layer_count": {"0": 2, "1": 1}}},
    ],
    # ------------------------------------------------------------------
    # pegaflow-core/src/allocator.rs:151-263 and pinned_pool.rs:722-795
    # ------------------------------------------------------------------
    "allocator": [
        {"name": "creates_allocator_with_scaled_capacity", "cite": "allocator.rs:156-168",
         "total_bytes": 10 * K * K * K, "unit": 64, "max_allocs": 128 * K,
         "expect": {"total_units": 10 * K * K * K // 64}},
        {"name": "allocate_rounds_up_to_unit_size", "cite": "allocator.rs:171-181",
         "total_bytes": 1024, "unit": 64, "max_allocs": 128 * K,
         "ops": [["alloc", 1, {"offset": 0, "size": 64}],
                 ["report", {"free": 960, "largest": 960}]]},
        {"name": "capacity_is_rounded_down_to_unit_size", "cite": "allocator.rs:184-202",
         "total_bytes": K * K * K + 123 * K * K, "unit": 256 * K * K, "max_allocs": 128 * K,
         "expect": {"total_units": 4, "total_bytes": K * K * K},
         "ops": [["report", {"free": K * K * K, "largest": K * K * K}]]},
        {"name": "does_not_allocate_past_unaligned_capacity", "cite": "allocator.rs:205-225",
         "total_bytes": K * K * K + 123 * K * K, "unit": 256 * K * K, "max_allocs": 128 * K,
         "ops": [["alloc", 256 * K * K, {"offset": 0, "size": 256 * K * K}],
                 ["alloc", 256 * K * K, {"offset": 256 * K * K, "size": 256 * K * K}],
                 ["alloc", 256 * K * K, {"offset": 512 * K * K, "size": 256 * K * K}],
                 ["alloc", 256 * K * K, {"offset": 768 * K * K, "size": 256 * K * K}],
                 ["alloc", 1, None]]},
        {"name": "reuse_after_free_merges_neighboring_regions", "cite": "allocator.rs:227-239",
         "total_bytes": 256, "unit": 64, "max_allocs": 128 * K,
         "ops": [["alloc", 64, {"name": "a"}], ["alloc", 64, {"name": "b"}],
                 ["free", "a"], ["free", "b"],
                 ["alloc", 128, {"offset": 0, "size": 128}]]},
        {"name": "rejects_unreasonably_large_requests", "cite": "allocator.rs:242-255",
         "total_bytes": K * K, "unit": 1, "max_allocs": 128 * K,
         "ops": [["alloc_error", 2 * 0xFFFFFFFF, "overflows u32 backing allocator"]]},
        {"name": "rejects_invalid_unit_size", "cite": "allocator.rs:258-262",
         "total_bytes": 1024, "unit": 0, "max_allocs": 128 * K,
         "expect": {"create_error_contains": "unit size must be greater than zero"}},
    ],
    "pool": [
        {"name": "numa_largest_free_for_node_is_not_global_min", "cite": "pinned_pool.rs:726-776",
         "pool_bytes": 4096, "unit_hint": 512, "alloc": 3584,
         "expect": {"largest_after": 512, "largest_untouched": 4096}},
    ],
    # ------------------------------------------------------------------
    # python/tests/test_worker_kv_layout.py:27-217
    # tensor = [shape, stride, element_size]
    # ------------------------------------------------------------------
    "kv_registration": [
        {"name": "mla_blocks_first_physical_rows_are_grouped", "cite": "test_worker_kv_layout.py:27-44",
         "tensor": [[6, 64, 576], [64 * 576, 576, 1], 2], "logical_block_size": 128, "is_mla": True,
         "expect": {"layout": "blocks-first", "num_blocks": 3, "bytes_per_block": 2 * 64 * 576 * 2,
                    "kv_stride_bytes": 0, "segments": 1, "physical_blocks_per_logical_block": 2}},
        {"name": "non_mla_kv_first_uses_legacy_block_stride", "cite": "test_worker_kv_layout.py:46-61",
         "tensor": [[2, 6, 64, 4, 8], [6 * 64 * 4 * 8, 64 * 4 * 8, 4 * 8, 8, 1], 2],
         "logical_block_size": 128,
         "expect": {"layout": "KV-first", "num_blocks": 6, "bytes_per_block": 64 * 4 * 8 * 2,
                    "kv_stride_bytes": 6 * 64 * 4 * 8 * 2, "segments": 2,
                    "physical_blocks_per_logical_block": 1}},
        {"name": "mla_prefers_blocks_first_when_first_dimension_is_two",
         "cite": "test_worker_kv_layout.py:64-80",
         "tensor": [[2, 64, 576], [64 * 576, 576, 1], 2], "logical_block_size": 128, "is_mla": True,
         "expect": {"layout": "blocks-first", "num_blocks": 1, "bytes_per_block": 2 * 64 * 576 * 2,
                    "kv_stride_bytes": 0, "segments": 1, "physical_blocks_per_logical_block": 2}},
        {"name": "mla_equal_physical_and_logical_block_size_is_unchanged",
         "cite": "test_worker_kv_layout.py:83-96",
         "tensor": [[3, 128, 576], [128 * 576, 576, 1], 2], "logical_block_size": 128,
         "is_mla": True,
         "expect": {"num_blocks": 3, "bytes_per_block": 128 * 576 * 2,
                    "physical_blocks_per_logical_block": 1}},
        {"name": "recurrent_state_uses_one_page_per_logical_block",
         "cite": "test_worker_kv_layout.py:99-116",
         "tensor": [[2, 1, 4096], [4096, 4096, 1], 2], "logical_block_size": 1536, "is_mla": True,
         "is_recurrent_state": True,
         "expect": {"layout": "blocks-first", "num_blocks": 2, "bytes_per_block": 4096 * 2,
                    "kv_stride_bytes": 0, "segments": 1, "physical_blocks_per_logical_block": 1}},
        {"name": "non_mla_cross_layer_layout_uses_legacy_block_stride",
         "cite": "test_worker_kv_layout.py:119-139",
         "tensor": [[6, 93, 2, 64, 1, 128],
                    [93 * 2 * 64 * 128, 2 * 64 * 128, 64 * 128, 128, 128, 1], 2],
         "logical_block_size": 128,
         "expect": {"layout": "blocks-first", "num_blocks": 6,
                    "bytes_per_block": 93 * 2 * 64 * 1 * 128 * 2,
                    "physical_blocks_per_logical_block": 1}},
        {"name": "logical_block_size_must_be_multiple_of_physical_block_size",
         "cite": "test_worker_kv_layout.py:142-152",
         "tensor": [[3, 96, 576], [96 * 576, 576, 1], 2], "logical_block_size": 128, "is_mla": True,
         "expect": {"error_match": "logical block size"}},
        {"name": "logical_block_size_must_be_positive", "cite": "test_worker_kv_layout.py:155-165",
         "tensor": [[3, 128, 576], [128 * 576, 576, 1], 2], "logical_block_size": 0, "is_mla": True,
         "expect": {"error_match": "logical block size must be > 0"}},
        {"name": "physical_block_count_must_be_positive", "cite": "test_worker_kv_layout.py:168-178",
         "tensor": [[0, 128, 576], [128 * 576, 576, 1], 2], "logical_block_size": 128,
         "is_mla": True, "expect": {"error_match": "physical block count must be > 0"}},
        {"name": "physical_block_size_must_be_positive", "cite": "test_worker_kv_layout.py:181-191",
         "tensor": [[3, 0, 576], [0, 576, 1], 2], "logical_block_size": 128, "is_mla": True,
         "expect": {"error_match": "physical block size must be > 0"}},
        {"name": "physical_block_count_must_be_divisible_by_split_ratio",
         "cite": "test_worker_kv_layout.py:194-204",
         "tensor": [[5, 64, 576], [64 * 576, 576, 1], 2], "logical_block_size": 128, "is_mla": True,
         "expect": {"error_match": "physical block count"}},
        {"name": "bytes_per_block_must_be_nonzero", "cite": "test_worker_kv_layout.py:207-217",
         "tensor": [[3, 128, 576], [0, 576, 1], 2], "logical_block_size": 128, "is_mla": True,
         "expect": {"error_match": "Invalid bytes_per_block"}},
    ],
    # ------------------------------------------------------------------
    # pegaflow-common/src/numa.rs:499-635
    # ------------------------------------------------------------------
    "numa": {
        "cite": "numa.rs:504-603",
        "format_cpu_list": [[[], ""], [[0], "0"], [[0, 1, 2, 3], "0-3"], [[0, 2, 4], "0,2,4"],
                            [[0, 1, 2, 4, 5], "0-2,4-5"], [[0, 1, 2, 4, 6, 7, 8], "0-2,4,6-8"]],
        "parse_cpulist": [["0-3", [0, 1, 2, 3]], ["0,4,8", [0, 4, 8]],
                          ["0-2,8,16-17", [0, 1, 2, 8, 16, 17]], ["", []], ["5", [5]]],
        "parse_cpulist_hyperthreading": {"input": "0-15,32-47", "len": 32, "first": 0,
                                         "at15": 15, "at16": 32, "last": 47},
        "display": [[0, "NUMA0"], [7, "NUMA7"], [-1, "UNKNOWN"]],
        "gpu_numa_nodes": {"map": {"0": 3, "1": 3, "2": -1, "3": 0, "4": 5},
                           "expect": [0, 3, 5]},
    },
    # ------------------------------------------------------------------
    # Closed-form byte patterns the reference's GPU tests fill buffers with.
    # ------------------------------------------------------------------
    "patterns": {
        "kernel_test": {"cite": "transfer/kernel.rs:203-221", "n": 257, "seg": 4112,
                        "byte": "(i*31+7) & 0xFF"},
        "block_fill": {"cite": "tests/common/helpers.rs:79-89", "byte": "(block % 251) + 1"},
        "shuffle": {"cite": "benches/transfer_h2d.rs:301-315", "seed": 0x9E3779B97F4A7C15,
                    "rule": "xorshift64 (13,7,17) Fisher-Yates, j = next() % (i+1), i = n-1..1"},
    },
    # ------------------------------------------------------------------
    # Engine round-trips whose expected bytes the reference states explicitly.
    # ------------------------------------------------------------------
    "engine": [
        {"name": "hybrid_groups_load_to_distinct_block_ids", "cite": "tests/engine_basic.rs:62-124",
         "layers": [{"name": "full_attention", "num_blocks": 4, "block_bytes": 1024,
                     "overwrite": 0, "save_ids": [0, 1], "load_ids": [2, 3]},
                    {"name": "gdn", "num_blocks": 4, "block_bytes": 1024,
                     "overwrite": 0x40, "save_ids": [2, 3], "load_ids": [None, 0]}],
         "expect": {"full_attention": {"2": 1, "3": 2}, "gdn": {"0": 4 + 0x40}}},
        {"name": "page_first_multi_layer_roundtrip", "cite": "tests/engine_basic.rs:32-58",
         "page_first": True,
         "layers": [{"name": "layer_a", "num_blocks": 4, "block_bytes": 512, "overwrite": 0},
                    {"name": "layer_b", "num_blocks": 4, "block_bytes": 1024, "overwrite": 0x40},
                    {"name": "layer_c", "num_blocks": 4, "block_bytes": 1536, "overwrite": 0x80}],
         "expect": {"page_offsets": [0, 512, 1536], "page_size": 3072}},
    ],
}


def main() -> None:
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_kats.json")
    with open(out, "w") as f:
        json.dump(KATS, f, indent=1, sort_keys=True)
        f.write("\n")
    print(f"wrote {out}")


if __name__ == "__main__":
    main()
