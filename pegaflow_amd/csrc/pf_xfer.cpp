// Block-ID gather / scatter engine: the MI355X fast path of the KV transfer.
//
// It moves the same bytes as descriptor construction + a transfer backend
// (pegaflow-core/src/gpu_worker.rs:353-423 + transfer/{memcpy,kernel}.rs in
// the reference) without a per-fragment descriptor: per layer it uploads the
// block-id list once and the kernels derive every address from
// `data_ptr + id*block_stride (+ kv_stride)`.
//
// Two ways across the host link, chosen per layer:
//   zero-copy : one kernel reads/writes the mapped pinned host image directly;
//   staged    : a gather kernel packs the selected blocks into a device staging
//               slot (HBM-bound, microseconds), then one DMA copy per segment
//               drains the slot to the host image on a side stream while the
//               next slot is being packed (and the mirror image for loads).
#include <algorithm>
#include <chrono>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "pf_common.hpp"
#include "pf_kernels.hpp"
#include "pf_layout.hpp"
#include "pf_transfer.hpp"
#include "pf_xfer.hpp"

namespace pf {

namespace {

bool aligned16(uint64_t v) { return (v & 15ull) == 0; }

using Clock = std::chrono::steady_clock;
double ms_since(Clock::time_point t) {
  return std::chrono::duration<double, std::milli>(Clock::now() - t).count();
}

}  // namespace

struct LayerPlan {
  std::string name;
  KVCacheLayout layout;
  uint64_t frag_bytes = 0;
  uint32_t n_seg = 0;
  uint64_t n_blocks = 0;
  const uint32_t* ids = nullptr;
  uint8_t* host[2] = {nullptr, nullptr};
  uint64_t host_dev[2] = {0, 0};
  uint64_t host_stride = 0;
  const uint64_t* page_dev = nullptr;  // device-visible page bases, host array
  const uint64_t* page_host = nullptr; // host addresses of the same pages
  uint64_t page_offset = 0;
  bool staged = false;
  bool dense = false;           // uniform host image at the fragment's own stride
  bool vec_ok = false;
  uint64_t ids_slab_off = 0;    // byte offset of the id list inside the slab
  uint64_t table_slab_off = 0;  // byte offset of the page table inside the slab
  uint64_t order_slab_off = 0;  // byte offset of the row order inside the slab (staged loads)
  std::vector<std::pair<uint64_t, uint64_t>> units;  // (first position, count) of each staged unit
  bool ordered = false;
  bool order_owner = false;     // this plan fills the order region
  bool order_shared = false;    // another plan's order region serves this one
  uint64_t layer_bytes = 0;
  size_t src_index = 0;         // index in the caller's layer array
};


int Xfer::ensure_slot(Slot& sl, uint64_t bytes) {
  if (sl.cap >= bytes) return PF_OK;
  const Clock::time_point t0 = Clock::now();
  struct Account {
    XferProfile& prof;
    Clock::time_point t0;
    ~Account() {
      prof.staging_alloc_ms += ms_since(t0);
      ++prof.staging_allocs;
    }
  } account{prof_, t0};
  if (sl.buf) {
    // Grow-only: the old buffer may still be in flight.
    if (sl.used) PF_HIP(hipEventSynchronize(sl.freed));
    PF_HIP(hipFree(sl.buf));
    sl.buf = nullptr;
    sl.cap = 0;
    sl.used = false;
  }
  uint64_t cap = std::max(bytes, slot_bytes_);
  const hipError_t e = hipMalloc(&sl.buf, cap);
  if (e != hipSuccess) {
    sl.buf = nullptr;
    if (e == hipErrorOutOfMemory) staging_oom_ = true;  // run() may take the zero-copy path instead
    return fail_hip(e, "hipMalloc of a staging slot");
  }
  sl.cap = cap;
  return PF_OK;
}

int Xfer::reserve_staging() {
  staging_oom_ = false;
  for (auto& sl : slots_) {
    const int st = ensure_slot(sl, slot_bytes_);
    if (st != PF_OK) return st;
  }
  SlabPool::Slab* slab = nullptr;
  const int st = slabs_.acquire(64 * 1024, &slab);  // stays in the pool, not in flight
  prof_ = XferProfile();  // what was allocated here belongs to no call
  return st;
}

int Xfer::enable_profile() {
  if (profiling_) return PF_OK;
  PF_HIP(hipEventCreate(&prof_begin_));
  PF_HIP(hipEventCreate(&prof_first_));
  PF_HIP(hipEventCreate(&prof_end_));
  profiling_ = true;
  return PF_OK;
}

XferProfile Xfer::read_profile() {
  XferProfile out = prof_;
  float ms = 0.f;
  if (prof_begin_set_ && prof_end_set_ &&
      hipEventElapsedTime(&ms, prof_begin_, prof_end_) == hipSuccess) {
    out.device_ms = ms;
  }
  if (prof_begin_set_ && prof_first_set_ &&
      hipEventElapsedTime(&ms, prof_begin_, prof_first_) == hipSuccess) {
    out.device_first_ms = ms;
  }
  (void)hipGetLastError();
  return out;
}

// The side stream carries the link copies next to the gather / scatter kernels
// on the caller's stream `s`; on one hardware queue the two would simply take
// turns.  Created on first use and, when the caller's stream is idle at that
// moment (the check synchronises both streams), swapped for a fresh one while
// kernels of the two do not overlap.
int Xfer::ensure_side_stream(hipStream_t s) {
  if (side_ != nullptr) return PF_OK;
  PF_HIP(hipStreamCreateWithFlags(&side_, hipStreamNonBlocking));
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &capture) != hipSuccess || capture != hipStreamCaptureStatusNone ||
      hipStreamQuery(s) != hipSuccess) {
    (void)hipGetLastError();
    return PF_OK;
  }
  std::vector<hipStream_t> rejected;
  for (int attempt = 0; attempt < 4; ++attempt) {
    bool concurrent = false;
    if (streams_run_concurrently(side_, s, &concurrent) != PF_OK || concurrent) break;
    hipStream_t fresh = nullptr;
    if (hipStreamCreateWithFlags(&fresh, hipStreamNonBlocking) != hipSuccess) break;
    rejected.push_back(side_);
    side_ = fresh;
  }
  for (hipStream_t r : rejected) (void)hipStreamDestroy(r);
  (void)hipGetLastError();
  return PF_OK;
}

int Xfer::timing_begin(hipStream_t s) {
  if (!timing_) return PF_OK;
  if (timing_used_ == timing_pool_.size()) {
    hipEvent_t a = nullptr, b = nullptr;
    PF_HIP(hipEventCreate(&a));
    PF_HIP(hipEventCreate(&b));
    timing_pool_.emplace_back(a, b);
  }
  PF_HIP(hipEventRecord(timing_pool_[timing_used_].first, s));
  return PF_OK;
}

int Xfer::timing_end(hipStream_t s) {
  if (!timing_) return PF_OK;
  PF_HIP(hipEventRecord(timing_pool_[timing_used_].second, s));
  ++timing_used_;
  return PF_OK;
}

int Xfer::launch_strided(const BlockUnit* dev_units, uint32_t n_units, uint64_t max_tiles,
                         uint64_t min_frag_bytes, bool to_far, hipStream_t s) {
  int st = timing_begin(s);
  if (st != PF_OK) return st;
  st = launch_block_units(dev_units, n_units, max_tiles, to_far, unroll_,
                          zero_copy_workgroups(min_frag_bytes), s);
  if (st != PF_OK) return st;
  return timing_end(s);
}

int Xfer::launch_strided_args(const ArgSlab& slab, uint32_t first_unit, uint32_t n_units,
                              uint64_t max_tiles, uint64_t min_frag_bytes, bool to_far,
                              hipStream_t s) {
  int st = timing_begin(s);
  if (st != PF_OK) return st;
  st = launch_block_units_args(slab, first_unit, n_units, max_tiles, to_far, unroll_,
                               zero_copy_workgroups(min_frag_bytes), s);
  if (st != PF_OK) return st;
  return timing_end(s);
}

int Xfer::launch_tiles(const BlockUnit* dev_unit, const BlockUnit& host_unit, bool to_far,
                       hipStream_t s) {
  int st = timing_begin(s);
  if (st != PF_OK) return st;
  (void)dev_unit;
  st = launch_block_tiles_one(host_unit, to_far, s);
  if (st != PF_OK) return st;
  return timing_end(s);
}

int Xfer::last_kernel_ms(float* out_ms, uint32_t* out_launches) {
  float total = 0.f;
  for (size_t i = 0; i < timing_used_; ++i) {
    PF_HIP(hipEventSynchronize(timing_pool_[i].second));
    float ms = 0.f;
    PF_HIP(hipEventElapsedTime(&ms, timing_pool_[i].first, timing_pool_[i].second));
    total += ms;
  }
  *out_ms = total;
  *out_launches = static_cast<uint32_t>(timing_used_);
  if (timing_in_place_) timing_used_ = 0;
  return PF_OK;
}

int Xfer::plan_layer(const pf_layer_blocks& in, size_t index, int path, LayerPlan* out,
                     bool* skip) {
  LayerPlan& p = *out;
  p.src_index = index;
  p.name = in.layer_name ? in.layer_name : ("#" + std::to_string(index));
  *skip = false;
  std::string cause;
  if (!KVCacheLayout::from_c(in.layout, &p.layout, &cause)) {
    return fail(PF_ERR_STORAGE, "layer %s: %s", p.name.c_str(), cause.c_str());
  }
  if (in.n_blocks == 0) {
    *skip = true;
    return PF_OK;
  }
  if (!in.block_ids) {
    return fail(PF_ERR_INVALID_ARGUMENT, "layer %s: block_ids must not be null", p.name.c_str());
  }
  if (in.n_blocks > 0xFFFFFFFFull) {
    return fail(PF_ERR_INVALID_ARGUMENT, "layer %s: too many blocks (%llu)", p.name.c_str(),
                static_cast<unsigned long long>(in.n_blocks));
  }
  p.n_blocks = in.n_blocks;
  p.ids = in.block_ids;
  const uint64_t num_blocks = p.layout.num_blocks();
  for (uint64_t i = 0; i < p.n_blocks; ++i) {
    if (p.ids[i] >= num_blocks) {
      // Same wording as KVCacheLayout::block_copies wrapped by the worker
      // (layout.rs:232-237, gpu_worker.rs:363-366).
      return fail(PF_ERR_STORAGE, "layer %s: block %u out of range (%llu blocks)", p.name.c_str(),
                  p.ids[i], static_cast<unsigned long long>(num_blocks));
    }
  }
  p.frag_bytes = p.layout.fragment_bytes();
  p.n_seg = p.layout.fragments_per_block();
  p.layer_bytes = p.frag_bytes * p.n_seg * p.n_blocks;

  const bool paged = in.page_host != nullptr || in.page_host_device != nullptr;
  bool far_aligned = true;
  if (paged) {
    if (!in.page_host || !in.page_host_device) {
      return fail(PF_ERR_INVALID_ARGUMENT,
                  "layer %s: page_host and page_host_device must both be set", p.name.c_str());
    }
    uint64_t need = 0;
    if (__builtin_add_overflow(in.page_offset, p.frag_bytes * p.n_seg, &need) ||
        need > in.page_len) {
      return fail(PF_ERR_INVALID_ARGUMENT,
                  "layer %s: page slice [%llu, +%llu) exceeds page length %llu", p.name.c_str(),
                  static_cast<unsigned long long>(in.page_offset),
                  static_cast<unsigned long long>(p.frag_bytes * p.n_seg),
                  static_cast<unsigned long long>(in.page_len));
    }
    for (uint64_t i = 0; i < p.n_blocks; ++i) {
      if (in.page_host[i] == 0 || in.page_host_device[i] == 0) {
        return fail(PF_ERR_INVALID_ARGUMENT, "layer %s: page %llu has a null base",
                    p.name.c_str(), static_cast<unsigned long long>(i));
      }
      far_aligned = far_aligned && aligned16(in.page_host_device[i]);
    }
    far_aligned = far_aligned && aligned16(in.page_offset);
    p.page_dev = in.page_host_device;
    p.page_host = in.page_host;
    p.page_offset = in.page_offset;
  } else {
    if (in.host_stride < p.frag_bytes) {
      return fail(PF_ERR_INVALID_ARGUMENT,
                  "layer %s: host_stride %llu < fragment size %llu: host images would overlap",
                  p.name.c_str(), static_cast<unsigned long long>(in.host_stride),
                  static_cast<unsigned long long>(p.frag_bytes));
    }
    p.host_stride = in.host_stride;
    for (uint32_t sgm = 0; sgm < p.n_seg; ++sgm) {
      if (!in.host[sgm] || in.host_device[sgm] == 0) {
        return fail(PF_ERR_INVALID_ARGUMENT, "layer %s: host segment %u is null", p.name.c_str(),
                    sgm);
      }
      uint64_t need = 0;
      if (__builtin_mul_overflow(p.n_blocks - 1, in.host_stride, &need) ||
          __builtin_add_overflow(need, p.frag_bytes, &need)) {
        return fail(PF_ERR_INVALID_ARGUMENT, "layer %s: host image size overflows", p.name.c_str());
      }
      if (need > in.host_len[sgm]) {
        return fail(PF_ERR_INVALID_ARGUMENT,
                    "layer %s: host segment %u needs %llu bytes, has %llu", p.name.c_str(), sgm,
                    static_cast<unsigned long long>(need),
                    static_cast<unsigned long long>(in.host_len[sgm]));
      }
      p.host[sgm] = static_cast<uint8_t*>(in.host[sgm]);
      p.host_dev[sgm] = in.host_device[sgm];
      far_aligned = far_aligned && aligned16(in.host_device[sgm]);
    }
    far_aligned = far_aligned && aligned16(in.host_stride);
  }
  const bool near_aligned = aligned16(p.layout.data_ptr()) &&
                            aligned16(p.layout.block_stride_bytes()) &&
                            aligned16(p.layout.kv_stride_bytes());
  // A fragment size that is not a multiple of 16 is fine for the vector path
  // (the kernel copies the tail bytewise) as long as every fragment START is
  // aligned, which the stride checks above guarantee.
  p.vec_ok = near_aligned && far_aligned && (p.n_seg == 1 || !paged || aligned16(p.frag_bytes));

  const bool dense = !paged && in.host_stride == p.frag_bytes;
  p.dense = dense;
  switch (path) {
    case PF_PATH_ZEROCOPY:
      p.staged = false;
      break;
    case PF_PATH_STAGED:
      if (paged) {
        p.staged = false;  // run() decides: whole-page packing or an error
        break;
      }
      if (!dense) {
        return fail(PF_ERR_INVALID_ARGUMENT,
                    "layer %s: the staged path needs a dense host image (host_stride == fragment "
                    "size, no page table)",
                    p.name.c_str());
      }
      p.staged = true;
      break;
    case PF_PATH_AUTO:
      p.staged = dense && p.layer_bytes >= auto_min_;
      break;  // run() may still stage it: see the call-size rule there
    default:
      return fail(PF_ERR_INVALID_ARGUMENT, "unknown transfer path %d", path);
  }
  return PF_OK;
}

// Can this call be served by packing whole pages?  Needs: every layer paged over
// the same pages and the same block list, one fragment per block, slices that
// do not overlap and (for saves) cover their common range without gaps, and
// pages laid back to back in runs.
bool Xfer::plan_page_pack(const std::vector<LayerPlan>& plans, bool save, PagePack* out) {
  const LayerPlan& first = plans.front();
  const uint64_t n = first.n_blocks;
  uint64_t lo = UINT64_MAX, hi = 0, covered = 0;
  for (const LayerPlan& p : plans) {
    if (p.page_dev == nullptr || p.n_seg != 1 || p.n_blocks != n) return false;
    if (p.page_dev != first.page_dev &&
        std::memcmp(p.page_dev, first.page_dev, n * sizeof(uint64_t)) != 0) {
      return false;
    }
    if (p.ids != first.ids && std::memcmp(p.ids, first.ids, n * sizeof(uint32_t)) != 0) {
      return false;
    }
    lo = std::min(lo, p.page_offset);
    hi = std::max(hi, p.page_offset + p.frag_bytes);
    covered += p.frag_bytes;
  }
  // Overlap check: sort the slices.
  std::vector<std::pair<uint64_t, uint64_t>> slices;
  for (const LayerPlan& p : plans) slices.emplace_back(p.page_offset, p.frag_bytes);
  std::sort(slices.begin(), slices.end());
  for (size_t i = 1; i < slices.size(); ++i) {
    if (slices[i - 1].first + slices[i - 1].second > slices[i].first) return false;
  }
  const uint64_t page_bytes = hi - lo;
  if (save) {
    // A whole-page drain writes every byte of [lo, hi): all of it must be payload.
    if (covered != page_bytes) return false;
  } else if (covered * 10 < page_bytes * 9) {
    return false;  // loading a small part of each page: do not drag the rest over the link
  }
  // Runs of pages that sit back to back, host and device side alike.
  out->runs.clear();
  uint64_t start = 0;
  for (uint64_t i = 1; i <= n; ++i) {
    const bool adjacent = i < n && first.page_dev[i] == first.page_dev[i - 1] + page_bytes &&
                          first.page_host[i] == first.page_host[i - 1] + page_bytes;
    if (!adjacent) {
      out->runs.emplace_back(start, i - start);
      start = i;
    }
  }
  // Many short runs mean many small copies: not worth staging.
  if (out->runs.size() * 8 > n && n > 8) return false;
  out->lo = lo;
  out->page_bytes = page_bytes;
  return true;
}

namespace {
// For every unit-sized range of the list: the positions of the range, relative
// to its start, in ascending order of their block id (equal ids keep their
// order in the list).  This runs on the submitting thread, so it has to stay
// well below the transfer time of the range: a comparison sort of 65536 ids
// takes as long as moving 65536 4 KiB blocks over the link (5 ms), the radix
// passes below a fifth of that.
void fill_row_order(const uint32_t* ids, uint64_t n, uint64_t per_unit, uint32_t* out) {
  constexpr uint32_t kDigitBits = 11;
  constexpr uint32_t kBuckets = 1u << kDigitBits;
  std::vector<uint64_t> keys;
  std::vector<uint32_t> spare;
  std::vector<uint32_t> counts;
  for (uint64_t first = 0; first < n; first += per_unit) {
    const uint64_t count = std::min(per_unit, n - first);
    const uint32_t* unit_ids = ids + first;
    uint32_t* unit_out = out + first;
    bool ascending = true;
    uint32_t max_id = 0;
    for (uint64_t i = 0; i < count; ++i) {
      if (i != 0 && unit_ids[i] < unit_ids[i - 1]) ascending = false;
      max_id = std::max(max_id, unit_ids[i]);
    }
    if (ascending) {
      for (uint64_t i = 0; i < count; ++i) unit_out[i] = static_cast<uint32_t>(i);
      continue;
    }
    if (count < 2048) {
      keys.resize(count);
      for (uint64_t i = 0; i < count; ++i) keys[i] = (static_cast<uint64_t>(unit_ids[i]) << 32) | i;
      std::sort(keys.begin(), keys.end());
      for (uint64_t i = 0; i < count; ++i) unit_out[i] = static_cast<uint32_t>(keys[i]);
      continue;
    }
    // Stable least-significant-digit radix sort of the positions by id.
    uint32_t passes = 1;
    while (passes * kDigitBits < 32 && (max_id >> (passes * kDigitBits)) != 0) ++passes;
    spare.resize(count);
    counts.resize(kBuckets);
    // An even number of hand-overs ends in `unit_out`.
    uint32_t* from = (passes % 2 == 0) ? unit_out : spare.data();
    uint32_t* to = (passes % 2 == 0) ? spare.data() : unit_out;
    for (uint64_t i = 0; i < count; ++i) from[i] = static_cast<uint32_t>(i);
    for (uint32_t pass = 0; pass < passes; ++pass) {
      const uint32_t shift = pass * kDigitBits;
      std::fill(counts.begin(), counts.end(), 0u);
      for (uint64_t i = 0; i < count; ++i) ++counts[(unit_ids[i] >> shift) & (kBuckets - 1)];
      uint32_t running = 0;
      for (uint32_t b = 0; b < kBuckets; ++b) {
        const uint32_t c = counts[b];
        counts[b] = running;
        running += c;
      }
      for (uint64_t i = 0; i < count; ++i) {
        const uint32_t pos = from[i];
        to[counts[(unit_ids[pos] >> shift) & (kBuckets - 1)]++] = pos;
      }
      std::swap(from, to);
    }
  }
}
}  // namespace

int Xfer::run_page_pack(std::vector<LayerPlan>& plans, const PagePack& pack, uint64_t n_layers,
                        bool save, hipStream_t s) {
  const LayerPlan& first = plans.front();
  const uint64_t n = first.n_blocks;
  const size_t n_plans = plans.size();
  uint64_t per_unit = std::max<uint64_t>(slot_bytes_ / pack.page_bytes, 1);
  per_unit = std::min<uint64_t>(per_unit, kMaxTileBlocks);
  if (n_plans > kMaxTileUnits) {
    return fail(PF_ERR_INVALID_ARGUMENT, "too many layers in one page-packed call: %zu", n_plans);
  }
  struct Chunk {
    uint64_t first, count;
  };
  std::vector<Chunk> chunks;
  for (const auto& run : pack.runs) {
    for (uint64_t off = 0; off < run.second; off += per_unit) {
      chunks.push_back({run.first + off, std::min(per_unit, run.second - off)});
    }
  }
  uint64_t max_chunk_bytes = 0;
  for (const Chunk& c : chunks) max_chunk_bytes = std::max(max_chunk_bytes, c.count * pack.page_bytes);
  for (auto& sl : slots_) {
    int st = ensure_slot(sl, max_chunk_bytes);
    if (st != PF_OK) return st;
  }
  // Slab: one BlockUnit per (chunk, layer), then the shared id list.
  const uint64_t units_bytes = (chunks.size() * n_plans * sizeof(BlockUnit) + 255) & ~255ull;
  const uint64_t ids_bytes = (n * sizeof(uint32_t) + 255) & ~255ull;
  // Loads visit the pages of a chunk in ascending destination id (launch_block_tiles).
  const uint64_t slab_bytes = units_bytes + ids_bytes + (save ? 0 : ids_bytes);
  SlabPool::Slab* slab = nullptr;
  int st = slabs_.acquire(slab_bytes, &slab);
  if (st != PF_OK) return st;
  uint8_t* slab_host = static_cast<uint8_t*>(slab->host);
  const uint64_t slab_dev = reinterpret_cast<uint64_t>(slab->dev);
  std::memcpy(slab_host + units_bytes, first.ids, n * sizeof(uint32_t));
  if (!save) {
    uint32_t* order_host = reinterpret_cast<uint32_t*>(slab_host + units_bytes + ids_bytes);
    for (const Chunk& c : chunks) fill_row_order(first.ids + c.first, c.count, c.count, order_host + c.first);
  }
  BlockUnit* units_host = reinterpret_cast<BlockUnit*>(slab_host);
  const BlockUnit* units_dev = reinterpret_cast<const BlockUnit*>(slab_dev);
  // The units of a chunk in descending slice size, and cut into runs that one
  // launch serves: its grid gives every unit the tiles of the largest slice, so
  // slices of unlike size (72 KiB latent and 8 KiB indexer rows in one page)
  // would leave most workgroups of the small ones without a tile.  A run ends
  // where less than three quarters of its grid would be busy.
  std::vector<size_t> plan_order(n_plans);
  for (size_t pi = 0; pi < n_plans; ++pi) plan_order[pi] = pi;
  auto tiles_of_plan = [&](size_t pi) {
    return (plans[pi].frag_bytes + kStagedTileBytes - 1) / kStagedTileBytes;
  };
  std::stable_sort(plan_order.begin(), plan_order.end(),
                   [&](size_t a, size_t b) { return tiles_of_plan(a) > tiles_of_plan(b); });
  struct UnitRun {
    size_t begin, count;
    uint64_t max_frag;
  };
  std::vector<UnitRun> unit_runs;
  for (size_t k = 0; k < n_plans;) {
    const uint64_t run_tiles = tiles_of_plan(plan_order[k]);  // the largest: sorted
    uint64_t useful = 0;
    size_t e = k;
    while (e < n_plans && e - k < kMaxTileUnits) {
      const uint64_t with = useful + tiles_of_plan(plan_order[e]);
      if (e > k && with * 4 < (e - k + 1) * run_tiles * 3) break;
      useful = with;
      ++e;
    }
    unit_runs.push_back({k, e - k, plans[plan_order[k]].frag_bytes});
    k = e;
  }
  std::vector<uint32_t> chunk_slot(chunks.size());
  for (size_t ci = 0; ci < chunks.size(); ++ci) {
    chunk_slot[ci] = next_slot_;
    next_slot_ = (next_slot_ + 1) % n_slots_;
    const uint64_t base = reinterpret_cast<uint64_t>(slots_[chunk_slot[ci]].buf);
    for (size_t k = 0; k < n_plans; ++k) {
      const LayerPlan& p = plans[plan_order[k]];
      BlockUnit& u = units_host[ci * n_plans + k];
      std::memset(&u, 0, sizeof(u));
      u.near_base = p.layout.data_ptr();
      u.block_stride = p.layout.block_stride_bytes();
      u.kv_stride = 0;
      u.frag_bytes = p.frag_bytes;
      u.far_base[0] = base + (p.page_offset - pack.lo);
      u.far_stride = pack.page_bytes;
      u.ids = reinterpret_cast<const uint32_t*>(slab_dev + units_bytes) + chunks[ci].first;
      if (!save && chunks[ci].count > 1) {
        u.order = reinterpret_cast<const uint32_t*>(slab_dev + units_bytes + ids_bytes) +
                  chunks[ci].first;
      }
      u.n_blocks = static_cast<uint32_t>(chunks[ci].count);
      u.n_seg = 1;
      u.tiles_per_frag = 1;
      u.vec_ok = aligned16(p.layout.data_ptr()) && aligned16(p.layout.block_stride_bytes()) &&
                 aligned16(p.page_offset - pack.lo) && aligned16(pack.page_bytes);
    }
  }

  // Before anything of this call is on `s`: the check wants the stream idle.
  if (use_side_stream(chunks.size())) {
    const int side_status = ensure_side_stream(s);
    if (side_status != PF_OK) return side_status;
  }
  began_ = true;
  const Clock::time_point t_enqueue = Clock::now();
  prof_mark_begin(s);
  PF_HIP(hipMemcpyAsync(slab->dev, slab->host, slab_bytes, hipMemcpyHostToDevice, s));
  hipStream_t side = use_side_stream(chunks.size()) ? side_ : s;
  if (side != s) {
    PF_HIP(hipEventRecord(fork_, s));
    PF_HIP(hipStreamWaitEvent(side, fork_, 0));
  }
  for (size_t ci = 0; ci < chunks.size(); ++ci) {
    const Chunk& c = chunks[ci];
    Slot& sl = slots_[chunk_slot[ci]];
    uint8_t* host_ptr = reinterpret_cast<uint8_t*>(first.page_host[c.first] + pack.lo);
    const uint64_t bytes = c.count * pack.page_bytes;
    auto launch = [&](bool to_far) -> int {
      int rc = timing_begin(s);
      if (rc != PF_OK) return rc;
      for (const UnitRun& run : unit_runs) {
        rc = launch_block_tiles(units_dev + ci * n_plans + run.begin,
                                static_cast<uint32_t>(run.count), static_cast<uint32_t>(c.count),
                                run.max_frag, 1, to_far, s);
        if (rc != PF_OK) return rc;
      }
      return timing_end(s);
    };
    if (save) {
      if (sl.used) PF_HIP(hipStreamWaitEvent(s, sl.freed, 0));
      st = launch(true);
      if (st != PF_OK) return st;
      PF_HIP(hipEventRecord(sl.ready, s));
      PF_HIP(hipStreamWaitEvent(side, sl.ready, 0));
      PF_HIP(hipMemcpyAsync(host_ptr, sl.buf, bytes, hipMemcpyDeviceToHost, side));
      PF_HIP(hipEventRecord(sl.freed, side));
      prof_mark_first(side);
    } else {
      if (sl.used) PF_HIP(hipStreamWaitEvent(side, sl.freed, 0));
      PF_HIP(hipMemcpyAsync(sl.buf, host_ptr, bytes, hipMemcpyHostToDevice, side));
      PF_HIP(hipEventRecord(sl.ready, side));
      prof_mark_first(side);
      PF_HIP(hipStreamWaitEvent(s, sl.ready, 0));
      st = launch(false);
      if (st != PF_OK) return st;
      PF_HIP(hipEventRecord(sl.freed, s));
    }
    sl.used = true;
    ++prof_.staged_groups;
    ++prof_.link_copies;
  }
  if (save && side != s) {
    PF_HIP(hipEventRecord(join_, side));
    PF_HIP(hipStreamWaitEvent(s, join_, 0));
  }
  // Every layer of a page lands together: all per-layer events fire at the end.
  if (!layer_events_.empty()) {
    for (uint64_t li = 0; li < n_layers; ++li) PF_HIP(hipEventRecord(layer_events_[li], s));
  }
  prof_mark_end(s);
  prof_.enqueue_ms += ms_since(t_enqueue);
  return slabs_.release_after(slab, s);
}

int Xfer::run(const pf_layer_blocks* layers, uint64_t n_layers, int path, bool save,
              hipStream_t s) {
  began_ = false;
  staging_oom_ = false;
  int st = run_impl(layers, n_layers, path, save, s);
  if (st != PF_OK && !began_ && staging_oom_ && path == PF_PATH_AUTO) {
    // The device has no memory left for a staging slot (slots allocated on
    // first use, or grown for an oversized block).  Nothing is enqueued yet,
    // and the zero-copy path moves the same bytes without device memory: a
    // slower neighbour for the model's kernels beats a failed transfer.  The
    // next AUTO call tries to allocate again.
    if (!staging_oom_logged_) {
      staging_oom_logged_ = true;
      log_line(LogLevel::Info,
               "no device memory for a staging slot (%s): this transfer, and later ones while "
               "that lasts, take the zero-copy path", last_error().c_str());
    }
    (void)hipGetLastError();
    began_ = false;
    st = run_impl(layers, n_layers, PF_PATH_ZEROCOPY, save, s);
  }
  if (st != PF_OK && began_) {
    // Something was already enqueued, possibly on the side stream, which the
    // caller's synchronise of `s` would not cover: drain both before the
    // caller learns of the failure and releases its buffers.
    const std::string message = last_error();
    if (side_ != nullptr) (void)hipStreamSynchronize(side_);
    (void)hipStreamSynchronize(s);
    (void)hipGetLastError();
    last_error() = message;
  }
  return st;
}

FillPlan plan_staged_fills(const std::vector<FillLayer>& layers, uint64_t slot_bytes,
                           uint64_t group_cap, bool may_split, uint64_t max_unit_blocks) {
  FillPlan plan;
  constexpr size_t kNone = static_cast<size_t>(-1);
  size_t fill_start = kNone;
  uint64_t used = 0;
  auto close_fill = [&]() {
    if (fill_start == kNone) return;
    plan.units[fill_start].fill_end = plan.units.size();
    plan.max_fill_bytes = std::max(plan.max_fill_bytes, used);
    ++plan.fills;
    fill_start = kNone;
    used = 0;
  };
  for (size_t li = 0; li < layers.size(); ++li) {
    const FillLayer& layer = layers[li];
    if (layer.block_bytes == 0) {
      close_fill();
      plan.units.push_back({li, 0, layer.n_blocks, 0, 0});
      continue;
    }
    const uint64_t block_bytes = layer.block_bytes;
    const uint64_t slot_blocks =
        std::min<uint64_t>(std::max<uint64_t>(slot_bytes / block_bytes, 1), max_unit_blocks);
    uint64_t pos = 0;
    while (pos < layer.n_blocks) {
      const uint64_t remaining = layer.n_blocks - pos;
      uint64_t take = 0;
      if (fill_start == kNone) {
        // A fresh fill takes up to a whole slot of this layer.
        take = std::min(remaining, slot_blocks);
      } else {
        // A layer that opened the fill may go on to the end of the slot (it came
        // back here only because a unit is capped at one grid extent); behind
        // other layers the fill ends at the group size.
        const uint64_t cap = plan.units[fill_start].layer == li ? slot_bytes : group_cap;
        const uint64_t room = cap > used ? (cap - used) / block_bytes : 0;
        const bool full = plan.units.size() - fill_start >= kStagedGroupUnits;
        if (!full && room >= remaining) {
          take = remaining;  // the rest of the layer fits
        } else if (!full && may_split && room * block_bytes >= kMinSplitBytes &&
                   (remaining - room) * block_bytes >= kMinSplitBytes) {
          take = room;       // its head fills the slot, its tail opens the next fill
        } else {
          close_fill();
          continue;
        }
        // A unit is one grid extent at most; what is left of the layer follows
        // as another unit, in this fill while there is room.
        take = std::min(take, max_unit_blocks);
      }
      if (fill_start == kNone) fill_start = plan.units.size();
      plan.units.push_back({li, pos, take, used, 0});
      used += (take * block_bytes + 255) & ~255ull;
      pos += take;
    }
  }
  close_fill();
  return plan;
}

int Xfer::run_impl(const pf_layer_blocks* layers, uint64_t n_layers, int path, bool save,
                   hipStream_t s) {
  if (!timing_in_place_) timing_used_ = 0;
  if (n_layers == 0) return PF_OK;
  if (!layers) return fail(PF_ERR_INVALID_ARGUMENT, "layers must not be null");
  const Clock::time_point t_call = Clock::now();
  const double alloc_before = prof_.staging_alloc_ms;
  if (!layer_events_.empty() && layer_events_.size() < n_layers) {
    return fail(PF_ERR_INVALID_ARGUMENT, "%zu layer events set, call has %llu layers",
                layer_events_.size(), static_cast<unsigned long long>(n_layers));
  }

  // ---- 1. validate everything before touching the stream ----------------
  std::vector<LayerPlan> plans;
  plans.reserve(n_layers);
  for (uint64_t li = 0; li < n_layers; ++li) {
    LayerPlan p;
    bool skip = false;
    int st = plan_layer(layers[li], li, path, &p, &skip);
    if (st != PF_OK) return st;
    if (!skip) plans.push_back(std::move(p));
  }
  // A call that moves enough dense bytes is staged whatever the size of its
  // layers: what the resident zero-copy kernel costs the kernels beside it
  // grows with the length of the call, and small layers share staging slots
  // and link copies.
  if (path == PF_PATH_AUTO && call_min_ != 0) {
    uint64_t dense_bytes = 0;
    for (const LayerPlan& p : plans) dense_bytes += p.dense ? p.layer_bytes : 0;
    if (dense_bytes >= call_min_) {
      for (LayerPlan& p : plans) p.staged = p.staged || (p.dense && p.layer_bytes >= kMinStagedLayerBytes);
    }
  }
  const bool want_events = !layer_events_.empty();
  if (plans.empty()) {
    // Nothing to move: layers' events still fire so a waiter is released.
    if (want_events) {
      for (uint64_t li = 0; li < n_layers; ++li) PF_HIP(hipEventRecord(layer_events_[li], s));
    }
    return PF_OK;
  }
  // Page-first images whose layer slices tile contiguous pages are packed page
  // by page in staging and cross the link as whole pages.
  if (path != PF_PATH_ZEROCOPY && plans.front().page_dev != nullptr) {
    PagePack pack;
    if (plan_page_pack(plans, save, &pack)) {
      uint64_t total = 0;
      for (const LayerPlan& p : plans) total += p.layer_bytes;
      if (path == PF_PATH_STAGED || total >= auto_min_) {
        last_path_ = PF_PATH_STAGED;
        prof_.plan_ms += ms_since(t_call);
        return run_page_pack(plans, pack, n_layers, save, s);
      }
    } else if (path == PF_PATH_STAGED) {
      return fail(PF_ERR_INVALID_ARGUMENT,
                  "the staged path needs a dense host image (host_stride == fragment size) or "
                  "page-first layers that tile contiguous pages");
    }
  } else if (path == PF_PATH_STAGED) {
    for (const LayerPlan& p : plans) {
      if (p.page_dev != nullptr) {
        return fail(PF_ERR_INVALID_ARGUMENT,
                    "layer %s: the staged path needs a dense host image (host_stride == fragment "
                    "size, no page table)", p.name.c_str());
      }
    }
  }
  last_path_ = plans.front().staged ? PF_PATH_STAGED : PF_PATH_ZEROCOPY;

  // ---- 2. lay out the slab: units, id lists, page tables ----------------
  const uint32_t tile = tile_bytes(unroll_);
  struct UnitRef {
    size_t plan;
    uint64_t first;  // first list position
    uint64_t count;
  };
  std::vector<UnitRef> unit_refs;
  uint64_t max_unit_bytes = 0;
  // Units and staging-slot fills (plan_staged_fills).  group_end[ui] is one
  // past the last unit of the fill that starts at unit ui (0 for units inside
  // a fill and for zero-copy units); unit_slot_off[ui] is the unit's offset in
  // its slot.
  std::vector<size_t> group_end;
  std::vector<uint64_t> unit_slot_off;
  {
    std::vector<FillLayer> fill_layers(plans.size());
    for (size_t pi = 0; pi < plans.size(); ++pi) {
      const LayerPlan& p = plans[pi];
      fill_layers[pi] = {p.n_blocks, p.staged ? p.frag_bytes * p.n_seg : 0};
    }
    const uint64_t group_wish =
        group_bytes_ != 0 ? group_bytes_ : (want_events ? kStagedGroupBytes : slot_bytes_);
    const FillPlan fp =
        plan_staged_fills(fill_layers, slot_bytes_, std::min<uint64_t>(group_wish, slot_bytes_),
                          !want_events && group_bytes_ == 0, kMaxTileBlocks);
    max_unit_bytes = fp.max_fill_bytes;
    unit_refs.reserve(fp.units.size());
    for (const FillUnit& u : fp.units) {
      unit_refs.push_back({u.layer, u.first, u.count});
      group_end.push_back(u.fill_end);
      unit_slot_off.push_back(u.slot_off);
      if (plans[u.layer].staged) plans[u.layer].units.emplace_back(u.first, u.count);
    }
  }
  // The visiting orders of staged loads sit behind everything else in the slab
  // and are uploaded on their own, after the first link copy is under way:
  // `order_slab_off` is relative to that tail until the head's size is known.
  uint64_t slab_bytes = 0, order_bytes = 0;
  bool all_zero_copy = true;
  uint32_t max_id = 0;
  for (const LayerPlan& p : plans) {
    all_zero_copy = all_zero_copy && !p.staged;
    if (all_zero_copy) {
      for (uint64_t i = 0; i < p.n_blocks; ++i) max_id = std::max(max_id, p.ids[i]);
    }
  }
  auto lay_out = [&](uint64_t id_bytes) {
    slab_bytes = unit_refs.size() * sizeof(BlockUnit);
    slab_bytes = (slab_bytes + 255) & ~255ull;
    order_bytes = 0;
    for (size_t pi = 0; pi < plans.size(); ++pi) {
      LayerPlan& p = plans[pi];
      p.ordered = p.order_owner = p.order_shared = false;
      // Layers that pass the very same id array share one upload.
      bool shared = false;
      for (size_t pj = 0; pj < pi; ++pj) {
        if (plans[pj].n_blocks == p.n_blocks &&
            (plans[pj].ids == p.ids ||
             std::memcmp(plans[pj].ids, p.ids, p.n_blocks * sizeof(uint32_t)) == 0)) {
          p.ids_slab_off = plans[pj].ids_slab_off;
          shared = true;
          break;
        }
      }
      if (!shared) {
        p.ids_slab_off = slab_bytes;
        slab_bytes += (p.n_blocks * id_bytes + 255) & ~255ull;
      }
      // Staged loads visit each unit's positions in ascending destination id
      // (launch_block_tiles); layers with the same ids and unit size share it.
      if (!save && p.staged && p.n_blocks > 1 && p.layer_bytes >= kRowOrderFromBytes) {
        p.ordered = true;
        for (size_t pj = 0; pj < pi; ++pj) {
          if (plans[pj].ordered && plans[pj].ids_slab_off == p.ids_slab_off &&
              plans[pj].units == p.units) {
            p.order_slab_off = plans[pj].order_slab_off;
            p.order_shared = true;
            break;
          }
        }
        if (!p.order_shared) {
          p.order_owner = true;
          p.order_slab_off = order_bytes;
          order_bytes += (p.n_blocks * sizeof(uint32_t) + 255) & ~255ull;
        }
      }
      if (p.page_dev) {
        bool tshared = false;
        for (size_t pj = 0; pj < pi; ++pj) {
          if (plans[pj].page_dev == p.page_dev && plans[pj].n_blocks == p.n_blocks) {
            p.table_slab_off = plans[pj].table_slab_off;
            tshared = true;
            break;
          }
        }
        if (!tshared) {
          p.table_slab_off = slab_bytes;
          slab_bytes += (p.n_blocks * sizeof(uint64_t) + 255) & ~255ull;
        }
      }
    }
  };
  lay_out(sizeof(uint32_t));
  // Short lists of zero-copy layers travel in the launch's arguments (below);
  // ids below 65536 are halved in size when that is what makes them fit.
  bool ids16 = false;
  if (all_zero_copy && slab_bytes > kArgSlabBytes && max_id < 65536u) {
    lay_out(sizeof(uint16_t));
    if (slab_bytes <= kArgSlabBytes) {
      ids16 = true;
    } else {
      lay_out(sizeof(uint32_t));
    }
  }
  const uint64_t head_bytes = slab_bytes;
  slab_bytes += order_bytes;
  for (LayerPlan& p : plans) {
    if (p.ordered) p.order_slab_off += head_bytes;
  }
  // A call of zero-copy layers whose units, id lists and page tables fit the
  // argument segment of a launch carries them there: nothing to upload first.
  bool in_args = slab_bytes <= kArgSlabBytes;
  for (const LayerPlan& p : plans) in_args = in_args && !p.staged;
  ArgSlab arg_slab;
  SlabPool::Slab* slab = nullptr;
  int st = PF_OK;
  if (!in_args) {
    st = slabs_.acquire(slab_bytes, &slab);
    if (st != PF_OK) return st;
  }
  uint8_t* slab_host = in_args ? reinterpret_cast<uint8_t*>(&arg_slab) : static_cast<uint8_t*>(slab->host);
  // In the argument form the units carry offsets into the slab, not addresses.
  const uint64_t slab_dev = in_args ? 0 : reinterpret_cast<uint64_t>(slab->dev);
  for (size_t pi = 0; pi < plans.size(); ++pi) {
    LayerPlan& p = plans[pi];
    if (ids16) {
      uint16_t* narrow = reinterpret_cast<uint16_t*>(slab_host + p.ids_slab_off);
      for (uint64_t i = 0; i < p.n_blocks; ++i) narrow[i] = static_cast<uint16_t>(p.ids[i]);
      // the kernel reads whole words: the odd half of the last one must be readable
      if (p.n_blocks & 1) narrow[p.n_blocks] = 0;
    } else {
      std::memcpy(slab_host + p.ids_slab_off, p.ids, p.n_blocks * sizeof(uint32_t));
    }
    if (p.page_dev) {
      std::memcpy(slab_host + p.table_slab_off, p.page_dev, p.n_blocks * sizeof(uint64_t));
    }
  }

  // ---- 3. staging slots ---------------------------------------------------
  std::vector<uint32_t> unit_slot(unit_refs.size(), 0);
  BlockUnit* units_host = reinterpret_cast<BlockUnit*>(slab_host);
  const BlockUnit* units_dev = reinterpret_cast<const BlockUnit*>(slab_dev);
  uint32_t slot_cursor = next_slot_;
  if (max_unit_bytes != 0) {
    for (auto& sl : slots_) {
      st = ensure_slot(sl, max_unit_bytes);
      if (st != PF_OK) return st;
    }
  }
  uint32_t group_slot = 0;
  for (size_t ui = 0; ui < unit_refs.size(); ++ui) {
    const UnitRef& r = unit_refs[ui];
    const LayerPlan& p = plans[r.plan];
    BlockUnit& u = units_host[ui];
    std::memset(&u, 0, sizeof(u));
    u.near_base = p.layout.data_ptr();
    u.block_stride = p.layout.block_stride_bytes();
    u.kv_stride = p.layout.kv_stride_bytes();
    u.frag_bytes = p.frag_bytes;
    // Zero-copy units start at list position 0, so a 16-bit list starts on a word.
    u.ids = reinterpret_cast<const uint32_t*>(slab_dev + p.ids_slab_off) + (ids16 ? 0 : r.first);
    u.ids16 = ids16 ? 1 : 0;
    if (p.ordered) {
      u.order = reinterpret_cast<const uint32_t*>(slab_dev + p.order_slab_off) + r.first;
    }
    u.n_blocks = static_cast<uint32_t>(r.count);
    u.n_seg = p.n_seg;
    u.tiles_per_frag = static_cast<uint32_t>((p.frag_bytes + tile - 1) / tile);
    if (p.staged) {
      if (group_end[ui] != 0) {  // first unit of a group: the next slot
        group_slot = slot_cursor;
        slot_cursor = (slot_cursor + 1) % n_slots_;
      }
      unit_slot[ui] = group_slot;
      const uint64_t base = reinterpret_cast<uint64_t>(slots_[group_slot].buf) + unit_slot_off[ui];
      u.far_base[0] = base;
      u.far_base[1] = base + r.count * p.frag_bytes;
      u.far_stride = p.frag_bytes;
      // Staging is 256-byte aligned device memory; only the near side and the
      // fragment size decide whether 16-byte vectors are safe.
      u.vec_ok = aligned16(p.layout.data_ptr()) && aligned16(p.layout.block_stride_bytes()) &&
                 aligned16(p.layout.kv_stride_bytes()) && aligned16(p.frag_bytes);
    } else {
      if (p.page_dev) {
        u.far_table = reinterpret_cast<const uint64_t*>(slab_dev + p.table_slab_off);
        u.far_table_off = p.page_offset;
      } else {
        u.far_base[0] = p.host_dev[0];
        u.far_base[1] = p.host_dev[1];
        u.far_stride = p.host_stride;
      }
      u.vec_ok = p.vec_ok ? 1 : 0;
    }
  }
  next_slot_ = slot_cursor;

  // ---- 4. enqueue ---------------------------------------------------------
  // A second stream pays off when the link copies of one fill can overlap the
  // gather of the next: count the fills.
  size_t staged_units = 0;
  for (size_t ge : group_end) staged_units += ge != 0 ? 1 : 0;
  // Before anything of this call is on `s`: the check wants the stream idle.
  if (use_side_stream(staged_units)) {
    const int side_status = ensure_side_stream(s);
    if (side_status != PF_OK) return side_status;
  }
  began_ = true;
  prof_.plan_ms += ms_since(t_call) - (prof_.staging_alloc_ms - alloc_before);
  const Clock::time_point t_enqueue = Clock::now();
  prof_mark_begin(s);
  if (!in_args) {
    PF_HIP(hipMemcpyAsync(slab->dev, slab->host, head_bytes, hipMemcpyHostToDevice, s));
  }
  // Sorting the ids of a long list takes the submitting thread about a
  // millisecond per 64 Ki ids: do it while the first unit's link copy runs.
  bool orders_pending = order_bytes != 0;
  auto upload_orders = [&]() -> int {
    if (!orders_pending) return PF_OK;
    orders_pending = false;
    for (const LayerPlan& p : plans) {
      if (p.order_owner) {
        uint32_t* order = reinterpret_cast<uint32_t*>(slab_host + p.order_slab_off);
        for (const auto& unit : p.units) {
          fill_row_order(p.ids + unit.first, unit.second, unit.second, order + unit.first);
        }
      }
    }
    PF_HIP(hipMemcpyAsync(reinterpret_cast<void*>(slab_dev + head_bytes), slab_host + head_bytes,
                          order_bytes, hipMemcpyHostToDevice, s));
    return PF_OK;
  };
  // With kernel timing on, the DMA copies run on the caller's stream too, so
  // that every timed kernel executes alone (a measurement mode: no overlap).
  hipStream_t side = use_side_stream(staged_units) ? side_ : s;
  bool side_used = false;
  auto fork_side = [&]() -> int {
    if (side_used || side == s) return PF_OK;
    PF_HIP(hipEventRecord(fork_, s));
    PF_HIP(hipStreamWaitEvent(side, fork_, 0));
    side_used = true;
    return PF_OK;
  };
  auto tiles_of = [&](const BlockUnit& u) -> uint64_t {
    return static_cast<uint64_t>(u.n_blocks) * u.tiles_per_frag * u.n_seg;
  };
  // Skipped (empty) layers fire their event at the position of the next
  // planned layer; track the caller index we have fired up to.
  uint64_t events_fired = 0;
  auto fire_events_through = [&](uint64_t caller_index, hipStream_t on) -> int {
    if (!want_events) return PF_OK;
    for (; events_fired <= caller_index; ++events_fired) {
      PF_HIP(hipEventRecord(layer_events_[events_fired], on));
    }
    return PF_OK;
  };

  size_t ui = 0;
  while (ui < unit_refs.size()) {
    const LayerPlan& p = plans[unit_refs[ui].plan];
    if (!p.staged) {
      // Batch consecutive zero-copy layers into one launch unless the caller
      // wants a completion event per layer.
      size_t uj = ui + 1;
      uint64_t max_tiles = tiles_of(units_host[ui]);
      uint64_t min_frag = units_host[ui].frag_bytes;
      if (!want_events) {
        while (uj < unit_refs.size() && !plans[unit_refs[uj].plan].staged) {
          max_tiles = std::max(max_tiles, tiles_of(units_host[uj]));
          min_frag = std::min(min_frag, units_host[uj].frag_bytes);
          ++uj;
        }
      }
      if (in_args) {
        st = launch_strided_args(arg_slab, static_cast<uint32_t>(ui), static_cast<uint32_t>(uj - ui),
                                 max_tiles, min_frag, save, s);
      } else {
        st = launch_strided(units_dev + ui, static_cast<uint32_t>(uj - ui), max_tiles, min_frag,
                            save, s);
      }
      if (st != PF_OK) return st;
      ++prof_.zero_copy_launches;
      prof_mark_first(s);
      st = fire_events_through(plans[unit_refs[uj - 1].plan].src_index, s);
      if (st != PF_OK) return st;
      ui = uj;
      continue;
    }

    // Staged group: the units [ui, ue) share one slot.
    st = fork_side();
    if (st != PF_OK) return st;
    const size_t ue = group_end[ui];
    Slot& sl = slots_[unit_slot[ui]];
    // The link copies of the group, coalesced: pieces that follow one another
    // both in staging and in the host image cross as one copy (a copy costs
    // ~10 us beyond its bytes).  V follows K when the engine allocated a
    // layer's K and V buffers one after the other, and the next layer follows
    // when its buffers were allocated right behind: a group of small layers
    // saved by one call is then a single copy.
    struct LinkCopy {
      uint8_t* host;
      uint64_t staged;
      uint64_t bytes;
    };
    std::vector<LinkCopy> group_copies;
    for (size_t k = ui; k < ue; ++k) {
      const UnitRef& r = unit_refs[k];
      const LayerPlan& q = plans[r.plan];
      const BlockUnit& u = units_host[k];
      for (uint32_t sgm = 0; sgm < q.n_seg; ++sgm) {
        LinkCopy c{q.host[sgm] + r.first * q.host_stride, u.far_base[sgm], r.count * q.frag_bytes};
        if (!group_copies.empty() &&
            group_copies.back().host + group_copies.back().bytes == c.host &&
            group_copies.back().staged + group_copies.back().bytes == c.staged) {
          group_copies.back().bytes += c.bytes;
        } else {
          group_copies.push_back(c);
        }
      }
    }
    auto link_copies = [&](bool to_host) -> int {
      for (const LinkCopy& c : group_copies) {
        void* staged = reinterpret_cast<void*>(c.staged);
        if (to_host) {
          PF_HIP(hipMemcpyAsync(c.host, staged, c.bytes, hipMemcpyDeviceToHost, side));
        } else {
          PF_HIP(hipMemcpyAsync(staged, c.host, c.bytes, hipMemcpyHostToDevice, side));
        }
      }
      return PF_OK;
    };
    auto launch_group = [&](bool to_far) -> int {
      if (ue - ui == 1) return launch_tiles(units_dev + ui, units_host[ui], to_far, s);
      // Workgroups the one-launch form would start: the rows form (up to
      // kRowsLaunchUnits units) starts every row with the tiles of the largest
      // fragment and the segments of the widest unit; the units-inner form also
      // gives every unit the rows of the longest.
      auto tiles_of = [](const BlockUnit& u) {
        return (u.frag_bytes + kStagedTileBytes - 1) / kStagedTileBytes;
      };
      uint32_t max_blocks = 0, max_seg = 0;
      uint64_t max_frag = 0, max_tiles = 0, total_rows = 0;
      for (size_t k = ui; k < ue; ++k) {
        const BlockUnit& u = units_host[k];
        max_blocks = std::max(max_blocks, u.n_blocks);
        max_seg = std::max(max_seg, u.n_seg);
        max_frag = std::max(max_frag, u.frag_bytes);
        max_tiles = std::max(max_tiles, tiles_of(u));
        total_rows += u.n_blocks;
      }
      const size_t n_group = ue - ui;
      const bool rows_form = n_group <= kRowsLaunchUnits;
      const uint64_t started =
          (rows_form ? total_rows : static_cast<uint64_t>(max_blocks) * n_group) * max_tiles * max_seg;
      // Units too unlike for one grid leave it full of workgroups that find no
      // tile.  Those are cheap but not free (they start and end at ~6 000 per
      // microsecond), and so is every further launch (~8 us of ramp, tail and
      // hand-over): the fill is cut into runs of units that keep three quarters
      // of their grids busy, and goes out as one rows launch per run when that
      // saves more idle workgroups than the launches cost.  A task over cache
      // groups of unlike size (8 full-attention layers of 625 blocks among 40
      // sliding-window layers of 8: 82 % of the units-inner grid idle) does:
      // gather 240 -> 136 us, scatter 241 -> 140 us.  Layers of 72 KiB and of
      // 8 KiB blocks in turn (44 % idle) do not: one launch 170 us, a launch
      // per layer 242 us.
      struct Run {
        size_t begin, end;
      };
      std::vector<Run> runs;
      uint64_t runs_started = 0;
      for (size_t k = ui; k < ue;) {
        size_t e = k;
        uint64_t run_useful = 0, run_rows = 0, run_tiles = 0, run_seg = 0;
        while (e < ue && e - k < kRowsLaunchUnits) {
          const BlockUnit& u = units_host[e];
          const uint64_t nu = run_useful + static_cast<uint64_t>(u.n_blocks) * tiles_of(u) * u.n_seg;
          const uint64_t nr = run_rows + u.n_blocks;
          const uint64_t nt = std::max(run_tiles, tiles_of(u));
          const uint64_t ns = std::max<uint64_t>(run_seg, u.n_seg);
          if (e > k && nu * 4 < nr * nt * ns * 3) break;
          run_useful = nu;
          run_rows = nr;
          run_tiles = nt;
          run_seg = ns;
          ++e;
        }
        runs.push_back({k, e});
        runs_started += run_rows * run_tiles * run_seg;
        k = e;
      }
      constexpr uint64_t kIdleWorkgroupsPerUs = 6000, kLaunchUs = 8;
      const bool in_runs = runs.size() > 1 && started > runs_started &&
                           (started - runs_started) / kIdleWorkgroupsPerUs >
                               (runs.size() - 1) * kLaunchUs;
      int rc = timing_begin(s);
      if (rc != PF_OK) return rc;
      bool launched = false;
      if (in_runs) {
        for (const Run& run : runs) {
          rc = launch_block_tiles_rows(units_dev + run.begin, units_host + run.begin,
                                       static_cast<uint32_t>(run.end - run.begin), to_far, s,
                                       &launched);
          if (rc != PF_OK) return rc;
          // (Only a launch beyond the grid limits is refused; what went out
          // before it is then simply done again by the form below.)
          if (!launched) break;
        }
      } else if (rows_form) {
        rc = launch_block_tiles_rows(units_dev + ui, units_host + ui, static_cast<uint32_t>(n_group),
                                     to_far, s, &launched);
        if (rc != PF_OK) return rc;
      }
      if (!launched) {
        rc = launch_block_tiles(units_dev + ui, static_cast<uint32_t>(n_group), max_blocks, max_frag,
                                max_seg, to_far, s);
        if (rc != PF_OK) return rc;
      }
      return timing_end(s);
    };
    // The events of every layer that ends inside the group fire behind it.
    const uint64_t last_layer = plans[unit_refs[ue - 1].plan].src_index;
    const bool ends_a_layer =
        ue == unit_refs.size() || unit_refs[ue].plan != unit_refs[ue - 1].plan;
    const uint64_t fire_through = ends_a_layer ? last_layer : (last_layer == 0 ? UINT64_MAX : last_layer - 1);
    if (save) {
      if (sl.used) PF_HIP(hipStreamWaitEvent(s, sl.freed, 0));
      st = launch_group(true);
      if (st != PF_OK) return st;
      PF_HIP(hipEventRecord(sl.ready, s));
      PF_HIP(hipStreamWaitEvent(side, sl.ready, 0));
      st = link_copies(true);
      if (st != PF_OK) return st;
      PF_HIP(hipEventRecord(sl.freed, side));
      prof_mark_first(side);
      sl.used = true;
      if (fire_through != UINT64_MAX) {
        st = fire_events_through(fire_through, side);
        if (st != PF_OK) return st;
      }
    } else {
      if (sl.used) PF_HIP(hipStreamWaitEvent(side, sl.freed, 0));
      st = link_copies(false);
      if (st != PF_OK) return st;
      PF_HIP(hipEventRecord(sl.ready, side));
      prof_mark_first(side);
      st = upload_orders();
      if (st != PF_OK) return st;
      PF_HIP(hipStreamWaitEvent(s, sl.ready, 0));
      st = launch_group(false);
      if (st != PF_OK) return st;
      PF_HIP(hipEventRecord(sl.freed, s));
      sl.used = true;
      if (fire_through != UINT64_MAX) {
        st = fire_events_through(fire_through, s);
        if (st != PF_OK) return st;
      }
    }
    ++prof_.staged_groups;
    prof_.link_copies += static_cast<uint32_t>(group_copies.size());
    ui = ue;
  }
  if (side_used && save) {
    // Join: everything the side stream drained is ordered before whatever the
    // caller enqueues (or records) next on its stream.
    PF_HIP(hipEventRecord(join_, side));
    PF_HIP(hipStreamWaitEvent(s, join_, 0));
  }
  // Trailing empty layers.
  if (want_events && events_fired < n_layers) {
    st = fire_events_through(n_layers - 1, s);
    if (st != PF_OK) return st;
  }
  prof_mark_end(s);
  prof_.enqueue_ms += ms_since(t_enqueue);
  return in_args ? PF_OK : slabs_.release_after(slab, s);
}

}  // namespace pf

extern "C" {

int pf_xfer_create(const pf_xfer_config* cfg, pf_xfer_t* out) {
  PF_REQUIRE_PTR(out);
  std::unique_ptr<pf::Xfer> x(new pf::Xfer(cfg));
  int st = x->init();
  if (st != PF_OK) return st;
  *out = reinterpret_cast<pf_xfer_t>(x.release());
  return PF_OK;
}

int pf_xfer_destroy(pf_xfer_t x) {
  delete reinterpret_cast<pf::Xfer*>(x);
  return PF_OK;
}

int pf_xfer_save(pf_xfer_t x, const pf_layer_blocks* layers, uint64_t n_layers, int path,
                 pf_stream_t s) {
  PF_REQUIRE_PTR(x);
  return reinterpret_cast<pf::Xfer*>(x)->run(layers, n_layers, path, true, pf::native(s));
}

int pf_xfer_load(pf_xfer_t x, const pf_layer_blocks* layers, uint64_t n_layers, int path,
                 pf_stream_t s) {
  PF_REQUIRE_PTR(x);
  return reinterpret_cast<pf::Xfer*>(x)->run(layers, n_layers, path, false, pf::native(s));
}

int pf_xfer_set_layer_events(pf_xfer_t x, pf_event_t* events, uint64_t n) {
  PF_REQUIRE_PTR(x);
  reinterpret_cast<pf::Xfer*>(x)->set_layer_events(events, n);
  return PF_OK;
}

int pf_xfer_last_path(pf_xfer_t x) { return x ? reinterpret_cast<pf::Xfer*>(x)->last_path() : 0; }

int pf_xfer_last_kernel_ms(pf_xfer_t x, float* out_ms, uint32_t* out_launches) {
  PF_REQUIRE_PTR(x);
  PF_REQUIRE_PTR(out_ms);
  PF_REQUIRE_PTR(out_launches);
  return reinterpret_cast<pf::Xfer*>(x)->last_kernel_ms(out_ms, out_launches);
}

int pf_plan_staged_fills(const uint64_t* layer_blocks, const uint64_t* block_bytes,
                         uint64_t n_layers, uint64_t slot_bytes, uint64_t group_bytes,
                         uint32_t per_layer_events, pf_fill_unit* out, uint64_t capacity,
                         uint64_t* out_units, uint64_t* out_fills) {
  PF_REQUIRE_PTR(out_units);
  PF_REQUIRE_PTR(out_fills);
  if (n_layers != 0) {
    PF_REQUIRE_PTR(layer_blocks);
    PF_REQUIRE_PTR(block_bytes);
  }
  if (capacity != 0) PF_REQUIRE_PTR(out);
  const uint64_t slot = slot_bytes != 0 ? slot_bytes : pf::kDefaultSlotBytes;
  std::vector<pf::FillLayer> layers(n_layers);
  for (uint64_t i = 0; i < n_layers; ++i) layers[i] = {layer_blocks[i], block_bytes[i]};
  const uint64_t wish =
      group_bytes != 0 ? group_bytes : (per_layer_events ? pf::kStagedGroupBytes : slot);
  const pf::FillPlan plan =
      pf::plan_staged_fills(layers, slot, std::min<uint64_t>(wish, slot),
                            !per_layer_events && group_bytes == 0, pf::kMaxTileBlocks);
  uint64_t fill = 0;
  size_t fill_end = 0;
  bool in_fill = false;
  for (size_t ui = 0; ui < plan.units.size(); ++ui) {
    const pf::FillUnit& u = plan.units[ui];
    if (u.fill_end != 0) {
      if (in_fill) ++fill;
      in_fill = true;
      fill_end = u.fill_end;
    }
    const bool staged = in_fill && ui < fill_end;
    if (ui < capacity) {
      out[ui] = {u.layer, u.first, u.count, u.slot_off, staged ? fill : UINT64_MAX};
    }
  }
  *out_units = plan.units.size();
  *out_fills = plan.fills;
  return PF_OK;
}

int pf_plain_copy(uint64_t dst, uint64_t src, uint64_t bytes, uint32_t tile_unroll,
                  pf_stream_t s) {
  // 0 selects the one-tile-per-workgroup form the staged path uses.
  int unroll = static_cast<int>(tile_unroll);
  return pf::launch_plain_copy(reinterpret_cast<void*>(dst), reinterpret_cast<const void*>(src),
                               bytes, unroll, pf::native(s));
}

int pf_xfer_set_kernel_timing(pf_xfer_t x, int enable) {
  PF_REQUIRE_PTR(x);
  if (enable < 0 || enable > 2) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "kernel timing mode %d (expected 0, 1 or 2)", enable);
  }
  reinterpret_cast<pf::Xfer*>(x)->set_timing(enable);
  return PF_OK;
}

}  // extern "C"
