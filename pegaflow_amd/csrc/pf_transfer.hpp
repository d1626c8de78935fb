// Copy descriptors, the merge rule, descriptor construction and the two
// reference-compatible transfer backends.  Follows
// pegaflow-core/src/transfer/{mod,memcpy,kernel}.rs and
// pegaflow-core/src/gpu_worker.rs:353-423 of the reference.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "../../include/pegahip.h"
#include "pf_layout.hpp"

namespace pf {

using CopyDesc = pf_copy_desc;       // transfer/mod.rs:36-44
using MergedRange = pf_merged_range; // transfer/memcpy.rs:16-20

// transfer/mod.rs:62-76.
enum class TransferMode : int {
  Direct = PF_MODE_DIRECT,
  Kernel = PF_MODE_KERNEL,
  ZeroCopy = PF_MODE_ZEROCOPY,  // worker pools only: block-ID engine pinned to the zero-copy kernel
};

// transfer/memcpy.rs:25-55: greedy left-to-right join of list-adjacent copies
// that share both allocations and are contiguous on both sides.
std::vector<MergedRange> merge(const CopyDesc* copies, uint64_t n);

// gpu_worker.rs:353-423.  Returns false with *err = "layer <name>: <cause>".
bool build_copy_descs(const pf_layer_transfer* layers, uint64_t n_layers,
                      std::vector<CopyDesc>* out, uint64_t* total_bytes, std::string* err);

// A pinned host slab with a device twin, recycled once the stream work that
// reads it has finished.  Used for descriptor tables and block-id lists.
class SlabPool {
 public:
  struct Slab {
    void* host = nullptr;
    void* dev = nullptr;
    uint64_t cap = 0;
    hipEvent_t done = nullptr;
    bool in_flight = false;
  };
  ~SlabPool();
  // A slab of at least `bytes` whose previous use (if any) has completed.
  int acquire(uint64_t bytes, Slab** out);
  // Mark the slab busy until everything enqueued on `s` so far has run.
  int release_after(Slab* slab, hipStream_t s);

 private:
  std::vector<std::unique_ptr<Slab>> slabs_;
};

// transfer/mod.rs:53-60.
class TransferBackend {
 public:
  virtual ~TransferBackend() = default;
  virtual int h2d(const CopyDesc* copies, uint64_t n, hipStream_t s) = 0;
  virtual int d2h(const CopyDesc* copies, uint64_t n, hipStream_t s) = 0;
  virtual const char* name() const = 0;
};

// transfer/memcpy.rs:57-102: DMA-style copies of the merged ranges.  A batch
// of few or large ranges is one hipMemcpyAsync per range, exactly as the
// reference.  A batch of many small ranges would pay the per-copy cost of the
// runtime on every fragment (1.6 GiB/s at 4 KiB on MI355X), so ranges whose
// host sides follow one another in memory are packed in a device staging
// buffer by one kernel and cross the link as one large copy per run; small
// ranges that are isolated on the host side go through the mapped-memory
// kernel when they carry a device-visible host address.  The bytes moved and
// the enqueue-only contract are those of the reference.
class MemcpyBackend : public TransferBackend {
 public:
  ~MemcpyBackend() override;
  int h2d(const CopyDesc* copies, uint64_t n, hipStream_t s) override {
    return submit(copies, n, true, s);
  }
  int d2h(const CopyDesc* copies, uint64_t n, hipStream_t s) override {
    return submit(copies, n, false, s);
  }
  const char* name() const override { return "direct"; }

  static constexpr uint64_t kLargeRange = 4ull << 20;   // copied on its own from this size on
  static constexpr uint64_t kFewRanges = 8;             // batches up to this size: one copy per range
  static constexpr uint64_t kStagingBytes = 256ull << 20;
  static constexpr uint64_t kKernelBelowBytes = 16ull << 20;  // small batches skip the staging hop

 private:
  int submit(const CopyDesc* copies, uint64_t n, bool host_is_src, hipStream_t s);
  int submit_impl(const CopyDesc* copies, uint64_t n, bool host_is_src, hipStream_t s);
  // One piece of a batch; *out_ranges = merged ranges it came to.
  int submit_piece(const CopyDesc* copies, uint64_t n, bool host_is_src, hipStream_t s,
                   uint64_t* out_ranges);
  SlabPool slabs_;
  // One staging buffer serves every batch.  Batches on one stream are ordered
  // by the stream; a batch on another stream first waits for `staging_done_`,
  // recorded behind the last batch that used the buffer.
  void* staging_ = nullptr;
  uint64_t staging_cap_ = 0;
  hipEvent_t staging_done_ = nullptr;
  hipStream_t staging_stream_ = nullptr;  // stream of the last batch that used staging_
  bool staging_used_ = false;
};

// transfer/kernel.rs:51-151: one kernel launch for the whole batch, host side
// addressed through its device-visible mapping.
class KernelBackend : public TransferBackend {
 public:
  int h2d(const CopyDesc* copies, uint64_t n, hipStream_t s) override {
    return submit(copies, n, true, s);
  }
  int d2h(const CopyDesc* copies, uint64_t n, hipStream_t s) override {
    return submit(copies, n, false, s);
  }
  const char* name() const override { return "kernel"; }

 private:
  int submit(const CopyDesc* copies, uint64_t n, bool host_is_src, hipStream_t s);
  int submit_impl(const CopyDesc* copies, uint64_t n, bool host_is_src, hipStream_t s);
  SlabPool slabs_;
};

// gpu_worker.rs:264-276.
std::unique_ptr<TransferBackend> build_backend(TransferMode mode);

// Launch the descriptor-table copy kernel: `table` is a device array of
// 3*n u64 words [dst, src, size].  `max_size` is the largest size in it.
// `max_workgroups` caps the grid (0 = as many as the batch has tiles).
int launch_desc_copy(const uint64_t* table, uint64_t n, uint64_t max_size, hipStream_t s,
                     uint32_t max_workgroups = 0);

}  // namespace pf
