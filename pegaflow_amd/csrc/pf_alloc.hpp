// Offset allocation for the pinned pool.
//
// OffsetAllocator: O(1) two-level-bitmap bin allocator over u32 units with
// neighbour merging on free.  The reference uses the crates.io crate
// `offset-allocator 0.2.0` (Cargo.lock:1703-1704), a port of Sebastian
// Aaltonen's OffsetAllocator; its source is not part of the reference tree,
// so this is a restatement of the published algorithm (32 top bins x 8 leaf
// bins, sizes classified as 3-bit-mantissa floats, requests rounded up to a
// bin, remainders rounded down).  The reference's own tests pin: first
// allocation at offset 0, same-size allocations at consecutive offsets,
// merge on free, exhaustion -> none.  The exact offset sequence under
// interleaved alloc/free beyond those is not pinned by anything in the
// reference tree.
//
// ScaledOffsetAllocator: bytes <-> units wrapper, follows
// pegaflow-core/src/allocator.rs:63-142.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace pf {

class OffsetAllocator {
 public:
  static constexpr uint32_t kNoSpace = 0xFFFFFFFFu;
  struct Allocation {
    uint32_t offset = kNoSpace;
    uint32_t metadata = kNoSpace;  // node index
    bool ok() const { return offset != kNoSpace; }
  };
  struct StorageReport {
    uint32_t total_free_space = 0;
    uint32_t largest_free_region = 0;
  };

  OffsetAllocator(uint32_t size, uint32_t max_allocs);
  Allocation allocate(uint32_t size);
  void free(Allocation a);
  uint32_t allocation_size(Allocation a) const;
  StorageReport storage_report() const;

  // Size classes: 5-bit exponent, 3-bit mantissa.
  static uint32_t uint_to_float_round_up(uint32_t size);
  static uint32_t uint_to_float_round_down(uint32_t size);
  static uint32_t float_to_uint(uint32_t f);

 private:
  static constexpr uint32_t kUnused = 0xFFFFFFFFu;
  static constexpr uint32_t kTopBins = 32;
  static constexpr uint32_t kBinsPerLeaf = 8;
  static constexpr uint32_t kLeafBins = kTopBins * kBinsPerLeaf;
  struct Node {
    uint32_t data_offset = 0;
    uint32_t data_size = 0;
    uint32_t bin_prev = kUnused;
    uint32_t bin_next = kUnused;
    uint32_t neighbor_prev = kUnused;
    uint32_t neighbor_next = kUnused;
    bool used = false;
  };
  uint32_t insert_node_into_bin(uint32_t size, uint32_t data_offset);
  void remove_node_from_bin(uint32_t node_index);
  uint32_t pop_free_node();
  void push_free_node(uint32_t index);
  uint32_t free_node_count() const {
    return static_cast<uint32_t>(recycled_.size()) + (max_allocs_ - fresh_);
  }

  uint32_t size_;
  uint32_t max_allocs_;
  uint32_t free_storage_ = 0;
  uint32_t used_bins_top_ = 0;
  uint8_t used_bins_[kTopBins] = {};
  uint32_t bin_indices_[kLeafBins];
  // Node records grow on demand; indices are handed out in ascending order
  // and freed ones are reused last-in-first-out, as a pre-filled stack would.
  std::vector<Node> nodes_;
  std::vector<uint32_t> recycled_;
  uint32_t fresh_ = 0;
};

// allocator.rs:7-43.
struct AllocatorError {
  enum Kind { None, InvalidUnitSize, CapacityTooLarge, RequestTooLarge } kind = None;
  uint64_t bytes = 0;
  uint64_t unit_size = 0;
  std::string to_string() const;
};

// allocator.rs:45-142.
class ScaledOffsetAllocator {
 public:
  struct Allocation {
    uint64_t offset_bytes = 0;
    uint64_t size_bytes = 0;  // rounded up to the unit
    OffsetAllocator::Allocation raw;
  };
  struct StorageReportBytes {
    uint64_t total_free_bytes = 0;
    uint64_t largest_free_allocation_bytes = 0;
  };
  static ScaledOffsetAllocator* create(uint64_t total_bytes, uint64_t unit_size, uint32_t max_allocs,
                                       AllocatorError* err);
  // Returns 1 = allocated, 0 = no space (or size 0), -1 = error (*err set).
  int allocate(uint64_t size_bytes, Allocation* out, AllocatorError* err);
  void free(const Allocation& a);
  uint64_t total_bytes() const { return unit_size_ * total_units_; }
  uint64_t unit_size() const { return unit_size_; }
  uint32_t total_units() const { return total_units_; }
  StorageReportBytes storage_report() const;

 private:
  ScaledOffsetAllocator(uint64_t unit, uint32_t units, uint32_t max_allocs)
      : unit_size_(unit), total_units_(units), inner_(units, max_allocs) {}
  uint64_t unit_size_;
  uint32_t total_units_;
  OffsetAllocator inner_;
};

}  // namespace pf
