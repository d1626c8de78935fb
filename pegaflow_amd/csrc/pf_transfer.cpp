#include "pf_transfer.hpp"

#include <algorithm>
#include <cstring>

#include "pf_common.hpp"

namespace pf {

// Grid cap for descriptor-copy launches whose far side is mapped host memory.
// The host link is saturated by a few dozen workgroups; more of them only add
// outstanding small requests on the link and take compute units away from
// whatever else runs on the device for as long as the copy lasts.  Measured on
// MI355X with shuffled fragments (4 KiB x 65536, 16 KiB x 32768, 32 KiB x
// 20000), GB/s d2h / h2d: uncapped 53.0/53.8, 53.8/55.4, 54.1/55.6; 64
// workgroups 53.8/56.1, 54.6/57.2, 54.8/57.2; 16 workgroups fall to 48/32 on
// the 4 KiB shape but hold the full rate from 16 KiB fragments on.  So: 16
// workgroups for batches whose average fragment fills a 16 KiB tile, more for
// smaller fragments, at most 64.
static uint32_t host_link_workgroups(uint64_t total_bytes, uint64_t n) {
  constexpr uint64_t kTile = 16384;
  const uint64_t avg = n ? total_bytes / n : 0;
  if (avg >= kTile) return 16;
  const uint64_t scaled = 16 * ((kTile + (avg ? avg : 1) - 1) / (avg ? avg : 1));
  return static_cast<uint32_t>(scaled < 64 ? scaled : 64);
}

// ---------------------------------------------------------------------------
// merge
// ---------------------------------------------------------------------------

std::vector<MergedRange> merge(const CopyDesc* copies, uint64_t n) {
  std::vector<MergedRange> out;
  out.reserve(n);
  uint64_t run_first = 0;  // index of the descriptor that opened the current run
  for (uint64_t i = 0; i < n; ++i) {
    const CopyDesc& c = copies[i];
    if (!out.empty()) {
      MergedRange& run = out.back();
      const CopyDesc& first = copies[run_first];
      const bool same_allocations = first.device_allocation == c.device_allocation &&
                                    first.host_allocation == c.host_allocation;
      const bool device_contiguous = run.device + run.size == c.device;
      const bool host_contiguous = static_cast<uint8_t*>(run.host) + run.size == c.host;
      if (same_allocations && device_contiguous && host_contiguous) {
        run.size += c.size;
        continue;
      }
    }
    run_first = i;
    out.push_back({c.device, c.host, c.size});
  }
  return out;
}

// ---------------------------------------------------------------------------
// build_copy_descs
// ---------------------------------------------------------------------------

bool build_copy_descs(const pf_layer_transfer* layers, uint64_t n_layers,
                      std::vector<CopyDesc>* out, uint64_t* total_bytes, std::string* err) {
  out->clear();
  uint64_t total = 0;
  for (uint64_t li = 0; li < n_layers; ++li) {
    const pf_layer_transfer& layer = layers[li];
    const std::string name = layer.layer_name ? layer.layer_name : "";
    KVCacheLayout layout;
    std::string cause;
    if (!KVCacheLayout::from_c(layer.layout, &layout, &cause)) {
      *err = "layer " + name + ": " + cause;
      return false;
    }
    if (layer.n_blocks != 0 && (!layer.block_idx || !layer.blocks)) {
      *err = "layer " + name + ": block list is null";
      return false;
    }
    for (uint64_t bi = 0; bi < layer.n_blocks; ++bi) {
      const pf_host_block& hb = layer.blocks[bi];
      BlockCopies bc;
      if (!layout.block_copies(layer.block_idx[bi], &bc, &cause)) {
        *err = "layer " + name + ": " + cause;
        return false;
      }
      if (hb.num_segments == 0 || hb.num_segments > 2 || !hb.seg_host[0]) {
        *err = "layer " + name + ": host block has no segment 0";
        return false;
      }
      uint8_t* k_host = static_cast<uint8_t*>(hb.seg_host[0]) + hb.host_offset;
      uint64_t k_dev = hb.seg_device[0] + hb.host_offset;
      if (bc.n == 2) {
        // A single-segment host block holds K then V back to back
        // (gpu_worker.rs:373-379).
        const bool has_v = hb.num_segments >= 2 && hb.seg_host[1];
        uint8_t* v_host = has_v ? static_cast<uint8_t*>(hb.seg_host[1]) + hb.host_offset
                                : k_host + bc.k.bytes;
        uint64_t v_dev = has_v ? hb.seg_device[1] + hb.host_offset : k_dev + bc.k.bytes;
        uint64_t v_alloc = has_v ? hb.seg_alloc[1] : hb.seg_alloc[0];
        out->push_back({bc.k.addr, k_host, k_dev, bc.k.bytes, li, hb.seg_alloc[0]});
        out->push_back({bc.v.addr, v_host, v_dev, bc.v.bytes, li, v_alloc});
        total += bc.k.bytes + bc.v.bytes;
      } else {
        out->push_back({bc.k.addr, k_host, k_dev, bc.k.bytes, li, hb.seg_alloc[0]});
        total += bc.k.bytes;
      }
    }
  }
  if (total_bytes) *total_bytes = total;
  return true;
}

// ---------------------------------------------------------------------------
// SlabPool
// ---------------------------------------------------------------------------

SlabPool::~SlabPool() {
  for (auto& s : slabs_) {
    if (s->in_flight && s->done) (void)hipEventSynchronize(s->done);
    if (s->done) (void)hipEventDestroy(s->done);
    if (s->host) (void)hipHostFree(s->host);
    if (s->dev) (void)hipFree(s->dev);
  }
  (void)hipGetLastError();
}

int SlabPool::acquire(uint64_t bytes, Slab** out) {
  for (auto& s : slabs_) {
    if (s->cap < bytes) continue;
    if (s->in_flight) {
      hipError_t q = hipEventQuery(s->done);
      if (q == hipErrorNotReady) {
        (void)hipGetLastError();
        continue;
      }
      if (q != hipSuccess) return fail_hip(q, "hipEventQuery(slab)");
      s->in_flight = false;
    }
    *out = s.get();
    return PF_OK;
  }
  uint64_t cap = 64 * 1024;
  while (cap < bytes) cap <<= 1;
  std::unique_ptr<Slab> s(new Slab());
  PF_HIP(hipHostMalloc(&s->host, cap, hipHostMallocMapped | hipHostMallocPortable));
  hipError_t e = hipMalloc(&s->dev, cap);
  if (e == hipSuccess) e = hipEventCreateWithFlags(&s->done, hipEventDisableTiming);
  if (e != hipSuccess) {
    (void)hipHostFree(s->host);
    if (s->dev) (void)hipFree(s->dev);
    return fail_hip(e, "slab allocation");
  }
  s->cap = cap;
  *out = s.get();
  slabs_.push_back(std::move(s));
  return PF_OK;
}

int SlabPool::release_after(Slab* slab, hipStream_t s) {
  PF_HIP(hipEventRecord(slab->done, s));
  slab->in_flight = true;
  return PF_OK;
}

// Descriptor tables up to this size (4096 rows) are left in mapped host memory.
constexpr uint64_t kHostTableBytes = 96 * 1024;

// ---------------------------------------------------------------------------
// MemcpyBackend
// ---------------------------------------------------------------------------

MemcpyBackend::~MemcpyBackend() {
  if (staging_done_) {
    if (staging_used_) (void)hipEventSynchronize(staging_done_);
    (void)hipEventDestroy(staging_done_);
  }
  if (staging_) (void)hipFree(staging_);
  (void)hipGetLastError();
}

namespace {

// A merged range that keeps what the staged forms need.
struct Range {
  uint64_t device;
  uint8_t* host;
  uint64_t host_device;
  uint64_t size;
  uint64_t host_allocation;
};

// The reference's merge rule (memcpy.rs:25-55), keeping the device-visible
// host address and the host allocation of the descriptor that opened a range.
std::vector<Range> merge_ranges(const CopyDesc* copies, uint64_t n) {
  std::vector<Range> out;
  out.reserve(n);
  uint64_t run_first = 0;
  for (uint64_t i = 0; i < n; ++i) {
    const CopyDesc& c = copies[i];
    if (!out.empty()) {
      Range& run = out.back();
      const CopyDesc& first = copies[run_first];
      if (first.device_allocation == c.device_allocation &&
          first.host_allocation == c.host_allocation && run.device + run.size == c.device &&
          run.host + run.size == static_cast<uint8_t*>(c.host)) {
        run.size += c.size;
        continue;
      }
    }
    run_first = i;
    out.push_back({c.device, static_cast<uint8_t*>(c.host), c.host_device, c.size,
                   c.host_allocation});
  }
  return out;
}

hipError_t copy_range(const Range& r, bool host_is_src, hipStream_t s) {
  return host_is_src
             ? hipMemcpyHtoDAsync(reinterpret_cast<hipDeviceptr_t>(r.device), r.host, r.size, s)
             : hipMemcpyDtoHAsync(r.host, reinterpret_cast<hipDeviceptr_t>(r.device), r.size, s);
}

}  // namespace

namespace {
// A batch that failed half way may have left work on the stream that reads
// the table slab or the staging buffer: drain it, keeping the message.
int drained(int st, hipStream_t s) {
  if (st == PF_OK) return st;
  const std::string message = last_error();
  (void)hipStreamSynchronize(s);
  (void)hipGetLastError();
  last_error() = message;
  return st;
}
}  // namespace

int MemcpyBackend::submit(const CopyDesc* copies, uint64_t n, bool host_is_src, hipStream_t s) {
  return drained(submit_impl(copies, n, host_is_src, s), s);
}

// A long list that does not merge costs the submitting thread 6-7 ns per
// descriptor (merging, sorting into runs, writing the table) before anything is
// enqueued: 0.4 ms for 65 536 fragments of 4 KiB, a twelfth of their transfer.
// Such a list goes piece by piece, everything in order on the stream, so that
// the device works on one piece while the next is prepared (65 536 shuffled
// 4 KiB fragments: 48.2 -> 49.3 GiB/s).  A list whose first piece merges into
// few ranges is handed over whole: cutting it would only cut its large copies.
int MemcpyBackend::submit_impl(const CopyDesc* copies, uint64_t n, bool host_is_src,
                               hipStream_t s) {
  constexpr uint64_t kPiece = 16384;
  uint64_t done = 0;
  while (n - done > kPiece + kPiece / 2) {
    uint64_t ranges = 0;
    const int st = submit_piece(copies + done, kPiece, host_is_src, s, &ranges);
    if (st != PF_OK) return st;
    done += kPiece;
    if (ranges * 16 <= kPiece) break;
  }
  uint64_t ranges = 0;
  return done < n ? submit_piece(copies + done, n - done, host_is_src, s, &ranges) : PF_OK;
}

int MemcpyBackend::submit_piece(const CopyDesc* copies, uint64_t n, bool host_is_src,
                                hipStream_t s, uint64_t* out_ranges) {
  const std::vector<Range> ranges = merge_ranges(copies, n);
  *out_ranges = ranges.size();
  const char* what = host_is_src ? "hipMemcpyHtoDAsync" : "hipMemcpyDtoHAsync";
  if (ranges.size() <= kFewRanges) {
    for (const Range& r : ranges) {
      hipError_t e = copy_range(r, host_is_src, s);
      if (e != hipSuccess) return fail_hip(e, what);
    }
    return PF_OK;
  }

  // Sort the ranges into: large (own copy), members of a host-dense run
  // (staged), isolated small ones.  A run is a maximal sequence, in list
  // order per host allocation, of small ranges whose host sides follow one
  // another without a gap.
  struct Run {
    uint8_t* host_begin;
    uint64_t bytes;
    std::vector<uint32_t> members;  // indices into `ranges`
  };
  std::vector<Run> runs;
  std::vector<std::pair<uint64_t, size_t>> open;  // host allocation -> index of its open run
  // A batch whose small ranges add up to little is not worth the staging hop
  // (pack kernel + copy + their hand-over): when every range has a device-visible
  // host address the copy kernel moves them over the link directly, and at this
  // size it is gone before it could matter to a kernel running beside it.
  // Measured on MI355X, 4 KiB fragments shuffled, call + synchronise: 1024
  // fragments 33 GiB/s staged against 42 through the kernel, 4096 fragments 43
  // against 48.
  uint64_t small_bytes = 0;
  bool small_mapped = true;
  for (const Range& r : ranges) {
    if (r.size >= kLargeRange || r.size == 0) continue;
    small_bytes += r.size;
    small_mapped = small_mapped && r.host_device != 0;
  }
  const bool all_by_kernel = small_mapped && small_bytes <= kKernelBelowBytes;
  for (size_t i = 0; i < ranges.size(); ++i) {
    const Range& r = ranges[i];
    if (r.size >= kLargeRange || r.size == 0) continue;
    if (all_by_kernel) continue;  // listed as isolated below, without a run record each
    size_t oi = 0;
    while (oi < open.size() && open[oi].first != r.host_allocation) ++oi;
    if (oi < open.size()) {
      Run& run = runs[open[oi].second];
      if (run.host_begin + run.bytes == r.host && run.bytes + r.size <= kStagingBytes) {
        run.bytes += r.size;
        run.members.push_back(static_cast<uint32_t>(i));
        continue;
      }
      open[oi].second = runs.size();
    } else {
      if (open.size() >= 64) open.erase(open.begin());  // bound the linear search
      open.emplace_back(r.host_allocation, runs.size());
    }
    runs.push_back(Run{r.host, r.size, {static_cast<uint32_t>(i)}});
  }
  std::vector<uint32_t> isolated;
  bool isolated_mapped = true;
  uint64_t staged_pieces = 0, max_staged_piece = 0, max_run_bytes = 0;
  if (all_by_kernel) {
    isolated.reserve(ranges.size());
    for (size_t i = 0; i < ranges.size(); ++i) {
      if (ranges[i].size < kLargeRange && ranges[i].size != 0) isolated.push_back(static_cast<uint32_t>(i));
    }
  }
  for (const Run& run : runs) {
    if (run.members.size() == 1) {
      isolated.push_back(run.members[0]);
      isolated_mapped = isolated_mapped && ranges[run.members[0]].host_device != 0;
    } else {
      staged_pieces += run.members.size();
      max_run_bytes = std::max(max_run_bytes, run.bytes + 16);
      for (uint32_t m : run.members) max_staged_piece = std::max(max_staged_piece, ranges[m].size);
    }
  }
  const bool isolated_by_kernel = isolated_mapped && isolated.size() > kFewRanges;

  // Large ranges, and isolated ones that cannot use the kernel: one copy each.
  for (const Range& r : ranges) {
    if (r.size >= kLargeRange) {
      hipError_t e = copy_range(r, host_is_src, s);
      if (e != hipSuccess) return fail_hip(e, what);
    }
  }
  if (!isolated_by_kernel) {
    for (uint32_t i : isolated) {
      hipError_t e = copy_range(ranges[i], host_is_src, s);
      if (e != hipSuccess) return fail_hip(e, what);
    }
  }
  const uint64_t table_rows = staged_pieces + (isolated_by_kernel ? isolated.size() : 0);
  if (table_rows == 0) return PF_OK;
  if (table_rows > 0x7FFFFFFFull) {
    return fail(PF_ERR_INVALID_ARGUMENT, "descriptor batch of %llu exceeds the kernel limit",
                static_cast<unsigned long long>(table_rows));
  }

  if (staged_pieces != 0) {
    if (staging_done_ == nullptr) {
      PF_HIP(hipEventCreateWithFlags(&staging_done_, hipEventDisableTiming));
    }
    if (staging_cap_ < max_run_bytes) {
      // Grow-only; the last batch that used the old buffer must be through with it,
      // whichever stream it ran on.
      if (staging_) {
        if (staging_used_) PF_HIP(hipEventSynchronize(staging_done_));
        PF_HIP(hipFree(staging_));
        staging_ = nullptr;
        staging_cap_ = 0;
        staging_used_ = false;
      }
      uint64_t cap = 1ull << 20;
      while (cap < max_run_bytes) cap <<= 1;
      PF_HIP(hipMalloc(&staging_, cap));
      staging_cap_ = cap;
    }
    // A batch on another stream than the previous one is not ordered behind it
    // by the stream: make it wait until the buffer is free.
    if (staging_used_ && staging_stream_ != s) {
      PF_HIP(hipStreamWaitEvent(s, staging_done_, 0));
    }
  }

  SlabPool::Slab* slab = nullptr;
  int st = slabs_.acquire(table_rows * 3 * sizeof(uint64_t), &slab);
  if (st != PF_OK) return st;
  uint64_t* table = static_cast<uint64_t*>(slab->host);
  const uint64_t* table_dev = static_cast<const uint64_t*>(slab->dev);
  uint64_t row = 0;
  // Rows of the isolated ranges first, then run by run.
  uint64_t max_isolated = 0, isolated_bytes = 0;
  if (isolated_by_kernel) {
    for (uint32_t i : isolated) {
      const Range& r = ranges[i];
      table[3 * row + 0] = host_is_src ? r.device : r.host_device;
      table[3 * row + 1] = host_is_src ? r.host_device : r.device;
      table[3 * row + 2] = r.size;
      max_isolated = std::max(max_isolated, r.size);
      isolated_bytes += r.size;
      ++row;
    }
  }
  const uint64_t staging_base = reinterpret_cast<uint64_t>(staging_);
  for (const Run& run : runs) {
    if (run.members.size() == 1) continue;
    // Keep the host side's alignment modulo 16 so aligned pieces stay on the
    // 16-byte path of the kernel.
    const uint64_t pad = reinterpret_cast<uint64_t>(run.host_begin) & 15ull;
    for (uint32_t m : run.members) {
      const Range& r = ranges[m];
      const uint64_t in_staging = staging_base + pad + static_cast<uint64_t>(r.host - run.host_begin);
      table[3 * row + 0] = host_is_src ? r.device : in_staging;
      table[3 * row + 1] = host_is_src ? in_staging : r.device;
      table[3 * row + 2] = r.size;
      ++row;
    }
  }
  // A short table of ranges that all go through the mapped-memory kernel is
  // read where it was written (see KernelBackend::submit_impl); tables of
  // packing launches stay in device memory, where the HBM-rate kernels read them.
  if (staged_pieces == 0 && table_rows * 3 * sizeof(uint64_t) <= kHostTableBytes) {
    void* alias = nullptr;
    PF_HIP(hipHostGetDevicePointer(&alias, slab->host, 0));
    table_dev = static_cast<const uint64_t*>(alias);
  } else {
    PF_HIP(hipMemcpyAsync(slab->dev, slab->host, table_rows * 3 * sizeof(uint64_t),
                          hipMemcpyHostToDevice, s));
  }
  row = 0;
  if (isolated_by_kernel) {
    st = launch_desc_copy(table_dev, isolated.size(), max_isolated, s,
                          host_link_workgroups(isolated_bytes, isolated.size()));
    if (st != PF_OK) return st;
    row = isolated.size();
  }
  // One staging buffer, everything in stream order: pack, then copy (save),
  // or copy, then unpack (load); the next run waits for the previous one.
  for (const Run& run : runs) {
    if (run.members.size() == 1) continue;
    const uint64_t pad = reinterpret_cast<uint64_t>(run.host_begin) & 15ull;
    uint8_t* in_staging = static_cast<uint8_t*>(staging_) + pad;
    if (host_is_src) {
      PF_HIP(hipMemcpyHtoDAsync(reinterpret_cast<hipDeviceptr_t>(in_staging), run.host_begin,
                                run.bytes, s));
    }
    // Many pieces of at most one tile: two rows per workgroup, so that the second
    // row's descriptor is on its way while the first is copied (65 536 pieces of
    // 4 KiB: 92 us instead of 98).
    const uint64_t pieces = run.members.size();
    const uint32_t pack_workgroups =
        max_staged_piece <= 16384 && pieces >= 8192 ? static_cast<uint32_t>((pieces + 1) / 2) : 0;
    st = launch_desc_copy(table_dev + 3 * row, pieces, max_staged_piece, s, pack_workgroups);
    if (st != PF_OK) return st;
    if (!host_is_src) {
      PF_HIP(hipMemcpyDtoHAsync(run.host_begin, reinterpret_cast<hipDeviceptr_t>(in_staging),
                                run.bytes, s));
    }
    row += run.members.size();
  }
  if (staged_pieces != 0) {
    PF_HIP(hipEventRecord(staging_done_, s));
    staging_stream_ = s;
    staging_used_ = true;
  }
  return slabs_.release_after(slab, s);
}

// ---------------------------------------------------------------------------
// KernelBackend
// ---------------------------------------------------------------------------

int KernelBackend::submit(const CopyDesc* copies, uint64_t n, bool host_is_src, hipStream_t s) {
  return drained(submit_impl(copies, n, host_is_src, s), s);
}

int KernelBackend::submit_impl(const CopyDesc* copies, uint64_t n, bool host_is_src,
                               hipStream_t s) {
  if (n == 0) return PF_OK;  // kernel.rs:85-87
  if (n > 0x7FFFFFFFull) {
    return fail(PF_ERR_INVALID_ARGUMENT, "descriptor batch of %llu exceeds the kernel limit",
                static_cast<unsigned long long>(n));
  }
  const uint64_t bytes = n * 3 * sizeof(uint64_t);
  SlabPool::Slab* slab = nullptr;
  int st = slabs_.acquire(bytes, &slab);
  if (st != PF_OK) return st;
  uint64_t* table = static_cast<uint64_t*>(slab->host);
  uint64_t max_size = 0, total_size = 0;
  for (uint64_t i = 0; i < n; ++i) {
    const CopyDesc& c = copies[i];
    total_size += c.size;
    if (c.size != 0 && (c.device == 0 || c.host_device == 0)) {
      // The kernel dereferences both addresses; a null one would fault the GPU.
      return fail(PF_ERR_INVALID_ARGUMENT,
                  "descriptor %llu: the kernel backend needs a device address and a "
                  "device-visible host address",
                  static_cast<unsigned long long>(i));
    }
    table[3 * i + 0] = host_is_src ? c.device : c.host_device;
    table[3 * i + 1] = host_is_src ? c.host_device : c.device;
    table[3 * i + 2] = c.size;
    max_size = std::max<uint64_t>(max_size, c.size);
  }
  // A short table is read where it was written, in mapped host memory: the
  // upload would cost more than the rows' trip over the link, which the kernel
  // hides behind the copy of the row before.
  const uint64_t* table_dev = static_cast<const uint64_t*>(slab->dev);
  if (bytes <= kHostTableBytes) {
    void* alias = nullptr;
    PF_HIP(hipHostGetDevicePointer(&alias, slab->host, 0));
    table_dev = static_cast<const uint64_t*>(alias);
  } else {
    PF_HIP(hipMemcpyAsync(slab->dev, slab->host, bytes, hipMemcpyHostToDevice, s));
  }
  st = launch_desc_copy(table_dev, n, max_size, s, host_link_workgroups(total_size, n));
  if (st != PF_OK) return st;
  return slabs_.release_after(slab, s);
}

std::unique_ptr<TransferBackend> build_backend(TransferMode mode) {
  if (mode != TransferMode::Direct) return std::unique_ptr<TransferBackend>(new KernelBackend());
  return std::unique_ptr<TransferBackend>(new MemcpyBackend());
}

}  // namespace pf

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------

extern "C" {

int pf_merge_copies(const pf_copy_desc* copies, uint64_t n, pf_merged_range* out,
                    uint64_t* out_n) {
  PF_REQUIRE_PTR(out_n);
  if (n != 0) {
    PF_REQUIRE_PTR(copies);
    PF_REQUIRE_PTR(out);
  }
  auto merged = pf::merge(copies, n);
  for (size_t i = 0; i < merged.size(); ++i) out[i] = merged[i];
  *out_n = merged.size();
  return PF_OK;
}

int pf_backend_create(int mode, pf_backend_t* out) {
  PF_REQUIRE_PTR(out);
  if (mode != PF_MODE_DIRECT && mode != PF_MODE_KERNEL) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "unknown transfer mode %d", mode);
  }
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) {
    int code = pf::fail_hip(e, "hipGetDevice");
    (void)code;
    return pf::fail(PF_ERR_DEVICE_INIT, "backend init failed: %s", pf::last_error().c_str());
  }
  *out = reinterpret_cast<pf_backend_t>(
      pf::build_backend(static_cast<pf::TransferMode>(mode)).release());
  return PF_OK;
}

int pf_backend_destroy(pf_backend_t b) {
  delete reinterpret_cast<pf::TransferBackend*>(b);
  return PF_OK;
}

const char* pf_backend_name(pf_backend_t b) {
  return b ? reinterpret_cast<pf::TransferBackend*>(b)->name() : "";
}

int pf_backend_h2d(pf_backend_t b, const pf_copy_desc* copies, uint64_t n, pf_stream_t s) {
  PF_REQUIRE_PTR(b);
  if (n != 0) PF_REQUIRE_PTR(copies);
  return reinterpret_cast<pf::TransferBackend*>(b)->h2d(copies, n, pf::native(s));
}

int pf_backend_d2h(pf_backend_t b, const pf_copy_desc* copies, uint64_t n, pf_stream_t s) {
  PF_REQUIRE_PTR(b);
  if (n != 0) PF_REQUIRE_PTR(copies);
  return reinterpret_cast<pf::TransferBackend*>(b)->d2h(copies, n, pf::native(s));
}

int pf_transfer_mode_from_name(const char* name, int* out_mode) {
  PF_REQUIRE_PTR(name);
  PF_REQUIRE_PTR(out_mode);
  std::string s(name);
  size_t a = s.find_first_not_of(" \t\r\n");
  size_t b = s.find_last_not_of(" \t\r\n");
  s = a == std::string::npos ? "" : s.substr(a, b - a + 1);
  std::transform(s.begin(), s.end(), s.begin(), [](unsigned char c) { return std::tolower(c); });
  if (s == "direct") {
    *out_mode = PF_MODE_DIRECT;
    return PF_OK;
  }
  if (s == "kernel") {
    *out_mode = PF_MODE_KERNEL;
    return PF_OK;
  }
  return pf::fail(PF_ERR_INVALID_ARGUMENT,
                  "Unsupported pegaflow.transfer_backend '%s'; expected one of: direct, kernel",
                  name);
}

int pf_build_copy_descs(const pf_layer_transfer* layers, uint64_t n_layers, pf_copy_desc* out,
                        uint64_t cap, uint64_t* out_n, uint64_t* out_total_bytes) {
  PF_REQUIRE_PTR(out_n);
  if (n_layers != 0) PF_REQUIRE_PTR(layers);
  std::vector<pf::CopyDesc> descs;
  uint64_t total = 0;
  std::string err;
  if (!pf::build_copy_descs(layers, n_layers, &descs, &total, &err)) {
    return pf::fail(PF_ERR_STORAGE, "%s", err.c_str());
  }
  *out_n = descs.size();
  if (out_total_bytes) *out_total_bytes = total;
  if (descs.size() > cap) {
    return pf::fail(PF_ERR_BUFFER_TOO_SMALL, "descriptor buffer holds %llu entries, need %llu",
                    static_cast<unsigned long long>(cap),
                    static_cast<unsigned long long>(descs.size()));
  }
  if (!descs.empty()) {
    PF_REQUIRE_PTR(out);
    std::memcpy(out, descs.data(), descs.size() * sizeof(pf::CopyDesc));
  }
  return PF_OK;
}

}  // extern "C"
