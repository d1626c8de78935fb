// Launch interface of the gfx950 copy kernels (implemented in pf_kernels.hip).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace pf {

// One unit of block-ID work, read by the kernel from device memory.
// "near" is the paged KV cache in HBM; "far" is the other side: mapped pinned
// host memory (zero-copy) or a device staging buffer (staged).
//
// Fragment f = (segment s, list position i) covers
//   near: near_base + ids[i]*block_stride + s*kv_stride          [frag_bytes]
//   far : far_table ? far_table[i] + far_table_off + s*frag_bytes
//                   : far_base[s] + i*far_stride                 [frag_bytes]
struct BlockUnit {
  uint64_t near_base;
  uint64_t block_stride;
  uint64_t kv_stride;
  uint64_t frag_bytes;
  uint64_t far_base[2];
  uint64_t far_stride;
  const uint32_t* ids;        // device pointer, n_blocks entries
  const uint64_t* far_table;  // device pointer or null
  const uint32_t* order;      // device pointer or null: list position visited by row y
  uint64_t far_table_off;
  uint32_t n_blocks;
  uint32_t n_seg;             // fragments per block: 1 or 2
  uint32_t tiles_per_frag;    // ceil(frag_bytes / tile_bytes)
  uint32_t vec_ok;            // every address and stride is 16-byte aligned
  uint32_t ids16;             // the id list holds 16-bit ids (zero-copy form only)
  uint32_t reserved;
};

// Bytes one workgroup moves per tile for the given unroll (256 lanes x 16 B x U).
constexpr uint32_t tile_bytes(int unroll) { return static_cast<uint32_t>(unroll) * 256u * 16u; }

// Unroll factors the kernels are instantiated for.
bool unroll_supported(int unroll);

// Launch the zero-copy block-ID kernel over the `n_units` units starting at
// `units` (device).  `max_tiles` is the largest tile count of any of them;
// `max_workgroups_x` (0 = no cap) is the number of workgroups of the launch.
// With units of at least that many tiles there is one row of workgroups: all of
// them walk the units in order and stride over each unit's tiles.  Smaller
// units get several rows, each walking every rows-th unit.
// to_far: true = gather near -> far (save), false = scatter far -> near (load).
int launch_block_units(const BlockUnit* units, uint32_t n_units, uint64_t max_tiles, bool to_far,
                       int unroll, uint32_t max_workgroups_x, hipStream_t s);

// A slab small enough to travel in the arguments of a launch (the limit for all
// arguments of a kernel is 4 KiB): units first, then id lists and page tables,
// with the units' `ids` / `far_table` holding byte offsets into the slab.
constexpr uint32_t kArgSlabBytes = 3840;
struct ArgSlab {
  uint64_t words[kArgSlabBytes / 8];
};
// Units [first_unit, first_unit + n_units) of the slab.
int launch_block_units_args(const ArgSlab& slab, uint32_t first_unit, uint32_t n_units,
                            uint64_t max_tiles, bool to_far, int unroll, uint32_t max_workgroups_x,
                            hipStream_t s);

// Limits of one block_tiles launch (grid.y and grid.z are 16-bit).
constexpr uint32_t kMaxTileBlocks = 65535;
constexpr uint32_t kRowsLaunchUnits = 8;  // units one launch_block_tiles_rows call takes
constexpr uint64_t kStagedTileBytes = 2048;  // bytes one workgroup of the staged kernels moves
constexpr uint32_t kMaxTileUnits = 32767;

// Launch the one-tile-per-workgroup form over `n_units` units: the HBM-bound
// kernel of the staged path.  Every unit needs n_blocks <= kMaxTileBlocks;
// max_seg (1 or 2) is the largest n_seg among the units.  A unit's `order`
// (a permutation of 0..n_blocks-1) makes row y handle list position order[y].
// Measured on MI355X at the Llama shape with shuffled ids: a scatter whose
// rows ascend in destination block id runs at 6.1-6.2 TB/s against 5.7 in
// list order (and a plain copy at 6.5-6.7): writes want to be sequential,
// reads tolerate the shuffle (the same trick on the gather, sequential reads
// and shuffled writes, is slower: 5.8 against 6.4).
int launch_block_tiles(const BlockUnit* units, uint32_t n_units, uint32_t max_blocks,
                       uint64_t max_frag_bytes, uint32_t max_seg, bool to_far, hipStream_t s);

// Up to eight units of any lengths in one launch with no idle workgroups: the
// rows of all units laid end to end along grid.y (`host_units` is the host
// copy of `units`, read for the row counts).  *launched = false when the launch
// does not fit this form (more than eight units):
// nothing was enqueued and the caller uses launch_block_tiles.
int launch_block_tiles_rows(const BlockUnit* units, const BlockUnit* host_units, uint32_t n_units,
                            bool to_far, hipStream_t s, bool* launched);

// The same for a single unit, handed over by value (its `ids` / `order` are
// device addresses as usual).
int launch_block_tiles_one(const BlockUnit& unit, bool to_far, hipStream_t s);

// Plain device copy kernel of the same tile shape, for calibrating counters
// and measuring the HBM copy ceiling: copies `bytes` (multiple of 16).
// unroll 0 selects the one-tile-per-workgroup form, 1/2/4/8 the grid-stride form.
int launch_plain_copy(void* dst, const void* src, uint64_t bytes, int unroll, hipStream_t s);

// Do kernels of stream `a` and stream `b` run at the same time?  The runtime
// multiplexes a process's streams onto a few hardware queues, and two streams
// that share one execute their kernels strictly one after the other.  A
// one-lane kernel on `a` waits (for at most ~2 ms of the device's constant
// clock, then gives up) for a word that a one-lane kernel on `b` writes; seeing
// it proves the two ran concurrently.  Both streams are idle afterwards.
int streams_run_concurrently(hipStream_t a, hipStream_t b, bool* out);

}  // namespace pf
