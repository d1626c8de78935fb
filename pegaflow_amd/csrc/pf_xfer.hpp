// Block-ID gather / scatter engine (implementation in pf_xfer.cpp).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "../../include/pegahip.h"
#include "pf_common.hpp"
#include "pf_kernels.hpp"
#include "pf_layout.hpp"
#include "pf_transfer.hpp"

namespace pf {

struct LayerPlan;

// Measured on MI355X (Llama-3.1-8B shape, 327 MB per layer): slots smaller than
// a layer cost cross-stream hand-offs between DMA copies (16 MiB slots reach
// ~25 GB/s on saves, 64 MiB ~40-55 GB/s and unstable, 256 MiB 56.3 GB/s,
// 512 MiB 56.7 GB/s of a 57.3 GB/s link), so a slot holds a whole layer.
constexpr uint64_t kDefaultSlotBytes = 512ull << 20;
constexpr uint32_t kDefaultSlots = 2;
// PF_PATH_AUTO stages a dense layer (or a page-packed call) from this size on.
// Measured on MI355X, one call then a synchronise, nothing else running: the
// zero-copy kernel saves faster than the staged path up to 32 MiB (4 MiB:
// 41.0 against 33.9 GB/s; 32 MiB: 52.3 against 52.1) and slower from 64 MiB
// on (53.2 against 53.9; 128 MiB: 54.0 against 55.1); many small layers in
// one call favour it even more (8 x 4 MiB: 50.3 against 37.3).  Loads are
// faster zero-copy at every size (128 MiB: 56.9 against 55.1 GB/s), but a
// long zero-copy transfer slows kernels that run beside it, which a staged
// one does not, so large loads are staged as well.  What it costs them
// decides the threshold: a back-to-back stream of 2048^3 bf16 GEMMs (23 us
// each) runs at 104-109 TFLOP/s beside a 16-workgroup zero-copy transfer and
// at 687-713 beside a staged one (591 alone, launch-bound), a 1024^3 stream at
// 28 against 110; a staged layer costs 10-30 us beyond its bytes (through the
// engine's workers, 32 layers: 16 MiB per layer 50.0 / 52.0 GB/s staged
// against 54.1 / 56.0 zero-copy, 32 MiB 51.3 / 53.0 against 53.9 / 56.1, 4 MiB
// 44.7 / 46.4 against 51.0 / 54.7, 1 MiB 29.1 / 32.6 against 42.5 / 49.6).  From
// 16 MiB per layer on a transfer outlasts 280 us and gives up less than a
// tenth of its rate by staging.
constexpr uint64_t kDefaultAutoStagedMin = 16ull << 20;
// Staged units that follow one another share a staging slot, and one gather or
// scatter launch, while together they fit the slot (plan_staged_fills; at most kStagedGroupUnits
// of them, enough for every layer of an 80-layer model: a task of 32 layers x
// 256 KiB took 238 us in two groups of 16 and takes one gather and one link
// copy as one group): a launch pays ~6 us of ramp and tail whatever its size, so fewer,
// larger launches move more bytes per microsecond (fp8 shape, 256 MiB layers:
// one layer per launch 5.93 TB/s, two 6.12, four 6.18; Llama shape with 1 GiB
// slots, three layers per launch: 6.1-6.28 against 5.97), and the layers of a
// group complete together.  A caller that asked for a completion event per
// layer wants them apart: then only small layers are grouped, up to
// kStagedGroupBytes, whose copies still take well under a millisecond.
// Layers below this size stay with the zero-copy kernel even in a call that
// is staged for its total size.
constexpr uint64_t kMinStagedLayerBytes = 32ull << 10;
// Staged loads of layers from this size on scatter in ascending destination id
// (an HBM-rate matter); below it the order array's upload costs more than the
// scatter could gain.
constexpr uint64_t kRowOrderFromBytes = 4ull << 20;
constexpr uint64_t kStagedGroupBytes = 32ull << 20;
constexpr size_t kStagedGroupUnits = 128;
// A layer is split between two fills only into pieces of at least this size.
constexpr uint64_t kMinSplitBytes = 16ull << 20;

// How the layers of one call are cut into units (runs of list positions of one
// layer) and the units packed into staging-slot fills: one gather or scatter
// launch and its link copies per fill.  Pure arithmetic.
//
// A fill takes whole layers while they fit and then, when `may_split`, the
// head of the next one, whose tail opens the following fill: every launch but
// the last then moves a slot's worth of bytes whatever the size of a layer (a
// launch costs ~6 us beyond its bytes; Llama shape, 327 MB layers in 512 MiB
// slots: 537 MB per launch instead of 327).  A piece of a layer is at least
// kMinSplitBytes, or the layer is left whole for the next fill.  Without
// `may_split` (the caller wants a completion event per layer, or set a group
// size) layers stay whole and share a fill up to `group_cap` bytes; a layer
// larger than a slot always takes several fills.  No unit has more than
// `max_unit_blocks` positions (one grid extent) and no fill more than
// kStagedGroupUnits units.  A layer with block_bytes == 0 is not staged: it
// closes the current fill and gets one unit of its own outside any fill.
struct FillLayer {
  uint64_t n_blocks;
  uint64_t block_bytes;  // payload of one list position (all segments); 0 = not staged
};
struct FillUnit {
  size_t layer;
  uint64_t first;     // first list position
  uint64_t count;
  uint64_t slot_off;  // byte offset inside the fill's slot (256-byte aligned)
  size_t fill_end;    // first unit of a fill: one past its last unit; otherwise 0
};
struct FillPlan {
  std::vector<FillUnit> units;
  uint64_t max_fill_bytes = 0;
  size_t fills = 0;
};
FillPlan plan_staged_fills(const std::vector<FillLayer>& layers, uint64_t slot_bytes,
                           uint64_t group_cap, bool may_split, uint64_t max_unit_blocks);
constexpr int kDefaultUnroll = 4;
// Zero-copy launches are capped to a few workgroups: the host link, not the
// GPU, is the bound, and every workgroup that stays resident for the length of
// the transfer takes its compute unit away from kernels that need a whole one.
// Measured on MI355X, Llama shape (32 KiB fragments, 32 layers per launch),
// GB/s save / load alone, then a back-to-back 4096^3 bf16 GEMM stream next to
// the load / the save (1210 TFLOP/s alone):
//     4 workgroups  56.6 / 45.0    772 / 776
//     8             56.3 / 57.1    779 / 779
//    16             56.8 / 57.3    765 / 752
//    32             57.1 / 56.6    720 / 576
//    64             57.1 / 57.3    557 / 405
//   128             56.9 / 57.4    309 / 488
// (~775 is what that GEMM runs at next to ONE resident workgroup of any kind:
// its 256 workgroups of 512 registers per lane need every compute unit.)
// Sixteen workgroups of full 16 KiB tiles keep 256 KiB in flight, twice the
// link's bandwidth-delay product; fragments smaller than a tile get
// proportionally more workgroups, up to 64.
constexpr uint32_t kZeroCopyWorkgroupsFullTiles = 16;
constexpr uint32_t kZeroCopyWorkgroupsMax = 64;

// Where the time of the calls since reset_profile() went, and which way their
// bytes crossed the link.  The device figures need enable_profile() and are
// filled by read_profile() once the stream has been synchronised.
struct XferProfile {
  double plan_ms = 0;           // validation, unit and slab layout
  double staging_alloc_ms = 0;  // hipMalloc / hipFree of staging slots inside a call
  double enqueue_ms = 0;        // issuing copies and launches (row-order sort included)
  uint32_t staged_groups = 0;
  uint32_t zero_copy_launches = 0;
  uint32_t link_copies = 0;
  uint32_t staging_allocs = 0;
  double device_first_ms = 0;   // first command -> first slot filled / drained (or first kernel)
  double device_ms = 0;         // first command -> last command
};

class Xfer {
 public:
  explicit Xfer(const pf_xfer_config* cfg) {
    if (cfg) {
      if (cfg->staging_slot_bytes) slot_bytes_ = cfg->staging_slot_bytes;
      if (cfg->staging_slots) n_slots_ = cfg->staging_slots;
      if (cfg->zerocopy_max_workgroups) zc_max_wg_ = cfg->zerocopy_max_workgroups;
      if (cfg->auto_staged_min_bytes) auto_min_ = cfg->auto_staged_min_bytes;
      call_min_ = cfg->auto_staged_min_call_bytes;
      if (cfg->tile_unroll) unroll_ = static_cast<int>(cfg->tile_unroll);
      if (cfg->copy_stream) copy_stream_ = cfg->copy_stream;
      if (cfg->staged_group_bytes) group_bytes_ = cfg->staged_group_bytes;
    }
  }

  ~Xfer() {
    if (side_ && side_owned_) {
      (void)hipStreamSynchronize(side_);
      (void)hipStreamDestroy(side_);
    }
    for (auto& sl : slots_) {
      if (sl.ready) (void)hipEventDestroy(sl.ready);
      if (sl.freed) (void)hipEventDestroy(sl.freed);
      if (sl.buf) (void)hipFree(sl.buf);
    }
    if (fork_) (void)hipEventDestroy(fork_);
    if (join_) (void)hipEventDestroy(join_);
    for (auto& p : timing_pool_) {
      (void)hipEventDestroy(p.first);
      (void)hipEventDestroy(p.second);
    }
    for (hipEvent_t e : {prof_begin_, prof_first_, prof_end_}) {
      if (e) (void)hipEventDestroy(e);
    }
    (void)hipGetLastError();
  }

  int init() {
    if (!unroll_supported(unroll_)) {
      return fail(PF_ERR_INVALID_ARGUMENT, "tile_unroll must be 1, 2, 4 or 8, got %d", unroll_);
    }
    if (n_slots_ < 2 || n_slots_ > 16) {
      return fail(PF_ERR_INVALID_ARGUMENT, "staging_slots must be in [2, 16], got %u", n_slots_);
    }
    hipError_t e = hipGetDevice(&device_);
    if (e != hipSuccess) {
      fail_hip(e, "hipGetDevice");
      return fail(PF_ERR_DEVICE_INIT, "transfer engine init failed: %s", last_error().c_str());
    }
    // The side stream is created when a call first needs it: an engine whose
    // link copies stay on the caller's stream never takes a hardware queue.
    PF_HIP(hipEventCreateWithFlags(&fork_, hipEventDisableTiming));
    PF_HIP(hipEventCreateWithFlags(&join_, hipEventDisableTiming));
    slots_.resize(n_slots_);
    for (auto& sl : slots_) {
      PF_HIP(hipEventCreateWithFlags(&sl.ready, hipEventDisableTiming));
      PF_HIP(hipEventCreateWithFlags(&sl.freed, hipEventDisableTiming));
    }
    return PF_OK;
  }

  // Construct and initialise on the current device; nullptr (and the thread's
  // error message set) on failure.
  static std::unique_ptr<Xfer> create(const pf_xfer_config* cfg) {
    std::unique_ptr<Xfer> x(new Xfer(cfg));
    if (x->init() != PF_OK) return nullptr;
    return x;
  }
  int ensure_side_stream(hipStream_t s);
  // Whether the last reserve_staging() or call failed for want of device memory.
  bool staging_out_of_memory() const { return staging_oom_; }

  // The stream the link copies of the staged path run on when they do not run
  // on the caller's (copy_stream 0 / 1): a stream of the caller's, which stays
  // the caller's to destroy, instead of one this engine creates and places on
  // first use.  Not while a call is in flight.
  void set_side_stream(hipStream_t side) {
    if (side == side_) return;
    if (side_ && side_owned_) {
      (void)hipStreamSynchronize(side_);
      (void)hipStreamDestroy(side_);
    }
    side_ = side;
    side_owned_ = side == nullptr;
  }

  int run(const pf_layer_blocks* layers, uint64_t n_layers, int path, bool save, hipStream_t s);
  int run_impl(const pf_layer_blocks* layers, uint64_t n_layers, int path, bool save,
               hipStream_t s);
  int save(const pf_layer_blocks* layers, uint64_t n_layers, int path, hipStream_t s) {
    return run(layers, n_layers, path, true, s);
  }
  int load(const pf_layer_blocks* layers, uint64_t n_layers, int path, hipStream_t s) {
    return run(layers, n_layers, path, false, s);
  }

  void set_layer_events(pf_event_t* events, uint64_t n) {
    layer_events_.clear();
    if (events) {
      for (uint64_t i = 0; i < n; ++i) layer_events_.push_back(native(events[i]));
    }
  }
  int last_path() const { return last_path_; }
  // 0 = off; 1 = time every launch alone (the link copies share the kernels'
  // stream meanwhile) and restart the figures with every call; 2 = time the
  // launches where they run, leaving the streams as they are, and add up over
  // calls until last_kernel_ms() is read.
  void set_timing(int mode) {
    timing_ = mode != 0;
    timing_in_place_ = mode == 2;
    timing_used_ = 0;
  }
  int last_kernel_ms(float* out_ms, uint32_t* out_launches);

  // Allocate every staging slot at its configured size now (and one table
  // slab), so that no call pays for it: hipMalloc of a slot inside a task
  // lengthens that task.  The worker pools call this when they are spawned.
  int reserve_staging();
  uint64_t staging_bytes() const {
    uint64_t total = 0;
    for (const auto& sl : slots_) total += sl.cap;
    return total;
  }
  // Three timing events bracket the device side of the calls of a profile
  // window (begin, first slot ready, end); off unless enabled.
  int enable_profile();
  void reset_profile() {
    prof_ = XferProfile();
    prof_begin_set_ = prof_first_set_ = prof_end_set_ = false;
  }
  // Call after the stream of the profiled calls has been synchronised.
  XferProfile read_profile();

 private:
  struct Slot {
    void* buf = nullptr;
    uint64_t cap = 0;
    hipEvent_t ready = nullptr;  // contents complete (gather done / fill done)
    hipEvent_t freed = nullptr;  // contents consumed (drain done / scatter done)
    bool used = false;
  };

  // Whole-page packing of page-first layers (see plan_page_pack).
  struct PagePack {
    uint64_t lo = 0;          // first covered byte of a page
    uint64_t page_bytes = 0;  // covered bytes per page
    std::vector<std::pair<uint64_t, uint64_t>> runs;  // (first position, count) of adjacent pages
  };
  bool plan_page_pack(const std::vector<LayerPlan>& plans, bool save, PagePack* out);
  int run_page_pack(std::vector<LayerPlan>& plans, const PagePack& pack, uint64_t n_layers,
                    bool save, hipStream_t s);
  int plan_layer(const pf_layer_blocks& in, size_t index, int path, LayerPlan* out, bool* skip);
  int ensure_slot(Slot& sl, uint64_t bytes);
  // Zero-copy form: grid-stride kernel over `n_units` units, capped grid.
  int launch_strided(const BlockUnit* dev_units, uint32_t n_units, uint64_t max_tiles,
                     uint64_t min_frag_bytes, bool to_far, hipStream_t s);
  // Workgroups of a zero-copy launch whose smallest fragment is `min_frag_bytes`.
  uint32_t zero_copy_workgroups(uint64_t min_frag_bytes) const {
    if (zc_max_wg_ != 0) return zc_max_wg_;
    const uint64_t tile = tile_bytes(unroll_);
    if (min_frag_bytes == 0 || min_frag_bytes >= tile) return kZeroCopyWorkgroupsFullTiles;
    const uint64_t scaled = kZeroCopyWorkgroupsFullTiles * ((tile + min_frag_bytes - 1) / min_frag_bytes);
    return static_cast<uint32_t>(scaled < kZeroCopyWorkgroupsMax ? scaled : kZeroCopyWorkgroupsMax);
  }
  // The same with the slab in the launch's arguments (short lists).
  int launch_strided_args(const ArgSlab& slab, uint32_t first_unit, uint32_t n_units,
                          uint64_t max_tiles, uint64_t min_frag_bytes, bool to_far, hipStream_t s);
  // Staged form: one tile per workgroup over one unit.
  int launch_tiles(const BlockUnit* dev_unit, const BlockUnit& host_unit, bool to_far,
                   hipStream_t s);
  int timing_begin(hipStream_t s);
  int timing_end(hipStream_t s);

  int device_ = 0;
  uint64_t slot_bytes_ = kDefaultSlotBytes;
  uint32_t n_slots_ = kDefaultSlots;
  uint32_t zc_max_wg_ = 0;  // 0 = by fragment size (zero_copy_workgroups)
  uint64_t auto_min_ = kDefaultAutoStagedMin;
  uint64_t call_min_ = 0;  // PF_PATH_AUTO: stage every dense layer of a call that moves this much (0 = off)
  int unroll_ = kDefaultUnroll;
  bool staging_oom_ = false;         // the current call failed to allocate a staging slot
  bool staging_oom_logged_ = false;
  uint64_t group_bytes_ = 0;  // 0 = fill the slot (kStagedGroupBytes while layer events are set)

  hipStream_t side_ = nullptr;
  bool side_owned_ = true;  // created by ensure_side_stream, destroyed with the engine
  hipEvent_t fork_ = nullptr;
  hipEvent_t join_ = nullptr;
  std::vector<Slot> slots_;
  uint32_t next_slot_ = 0;
  SlabPool slabs_;
  std::vector<hipEvent_t> layer_events_;
  int last_path_ = 0;

  bool timing_ = false;
  bool timing_in_place_ = false;
  bool began_ = false;  // the current call has enqueued work
  uint32_t copy_stream_ = 0;  // 0 = by unit count, 1 = side stream, 2 = caller's stream
  // A second stream pays off only when the copy of one unit can overlap the
  // gather of the next.  Measured on MI355X (Llama layer shape, one call then
  // a synchronise): a single unit of 4 / 16 / 64 / 312 MiB moves at 33.6 /
  // 48.7 / 54.3 / 56.0 GB/s in order on the caller's stream against 24.8 /
  // 44.4 / 52.8 / 55.6 GB/s with the hand-off to a side stream; from two
  // units on the side stream wins (56.6 against 55.8 GB/s at 32 units).
  bool use_side_stream(size_t staged_units) const {
    if ((timing_ && !timing_in_place_) || copy_stream_ == 2) return false;
    if (copy_stream_ == 1) return true;
    return staged_units > 1;
  }
  std::vector<std::pair<hipEvent_t, hipEvent_t>> timing_pool_;
  size_t timing_used_ = 0;

  XferProfile prof_;
  bool profiling_ = false;
  hipEvent_t prof_begin_ = nullptr, prof_first_ = nullptr, prof_end_ = nullptr;
  bool prof_begin_set_ = false, prof_first_set_ = false, prof_end_set_ = false;
  void prof_mark_begin(hipStream_t s) {
    if (profiling_ && !prof_begin_set_) prof_begin_set_ = hipEventRecord(prof_begin_, s) == hipSuccess;
  }
  void prof_mark_first(hipStream_t s) {
    if (profiling_ && !prof_first_set_) prof_first_set_ = hipEventRecord(prof_first_, s) == hipSuccess;
  }
  void prof_mark_end(hipStream_t s) {
    if (profiling_) prof_end_set_ = hipEventRecord(prof_end_, s) == hipSuccess;
  }
};


}  // namespace pf
