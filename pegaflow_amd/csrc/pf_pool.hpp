// Pinned host pool: backing region + offset allocator, sharded and per-NUMA
// variants, RAII allocations.  Follows pegaflow-core/src/pinned_pool.rs:20-715
// of the reference.
#pragma once

#include <atomic>
#include <cstdint>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "pf_alloc.hpp"
#include "pf_numa.hpp"
#include "pf_pinned_mem.hpp"

namespace pf {

// pinned_pool.rs:20-52: host address and device-visible address of the same byte.
struct MappedPinnedPtr {
  uint8_t* host = nullptr;
  uint8_t* device = nullptr;
  MappedPinnedPtr add(uint64_t offset) const { return {host + offset, device + offset}; }
};

class PinnedMemoryPool;

// pinned_pool.rs:56-117: frees itself back to its pool when destroyed.
class PinnedAllocation {
 public:
  PinnedAllocation(ScaledOffsetAllocator::Allocation a, uint8_t* ptr, uint8_t* device_ptr,
                   std::shared_ptr<PinnedMemoryPool> pool)
      : allocation_(a), ptr_(ptr), device_ptr_(device_ptr), pool_(std::move(pool)) {}
  ~PinnedAllocation();
  PinnedAllocation(const PinnedAllocation&) = delete;
  PinnedAllocation& operator=(const PinnedAllocation&) = delete;

  uint8_t* as_ptr() const { return ptr_; }
  uint64_t size_bytes() const { return allocation_.size_bytes; }
  uint64_t offset_bytes() const { return allocation_.offset_bytes; }
  MappedPinnedPtr mapped_ptr() const { return {ptr_, device_ptr_}; }
  // pinned_pool.rs:86-95; false when [offset, offset+size) leaves the allocation.
  bool mapped_ptr_at(uint64_t offset, uint64_t size, MappedPinnedPtr* out) const;
  // pinned_pool.rs:97-109.
  bool mapped_ptr_for_host_range(const uint8_t* host_ptr, uint64_t size, MappedPinnedPtr* out) const;
  // Identity used to tell allocations apart when merging copies
  // (block.rs:79-81: the Arc address).
  uint64_t allocation_id() const { return reinterpret_cast<uint64_t>(this); }

 private:
  ScaledOffsetAllocator::Allocation allocation_;
  uint8_t* ptr_;
  uint8_t* device_ptr_;
  std::shared_ptr<PinnedMemoryPool> pool_;
};

// pinned_pool.rs:121-345.
class PinnedMemoryPool : public std::enable_shared_from_this<PinnedMemoryPool> {
 public:
  static constexpr uint32_t kMaxAllocs = 4000000;  // pinned_pool.rs:131
  static constexpr uint64_t kUnitAlignment = 512;  // pinned_pool.rs:133
  // pinned_pool.rs:135-141.
  static uint64_t compute_unit_size(uint64_t pool_size, uint64_t hint);
  // pinned_pool.rs:165-180 picks the strategy: hugepages flag -> HugePages,
  // else SSD enabled -> Regular, else mapped hipHostMalloc.
  static AllocStrategy pick_strategy(bool use_hugepages, bool ssd_enabled);
  static std::shared_ptr<PinnedMemoryPool> create(uint64_t pool_size, bool use_hugepages,
                                                  bool ssd_enabled, uint64_t unit_size_hint,
                                                  NumaNode node, std::string* err, int* status);
  std::shared_ptr<PinnedAllocation> allocate(uint64_t size);
  void free_internal(const ScaledOffsetAllocator::Allocation& a);
  void usage(uint64_t* used, uint64_t* total);
  uint64_t largest_free_allocation();
  void memory_region(uint8_t** ptr, uint64_t* len) const;
  uint64_t allocatable_bytes() const { return allocatable_bytes_; }

 private:
  PinnedMemoryPool() = default;
  std::unique_ptr<PinnedMemory> backing_;
  std::mutex mu_;
  std::unique_ptr<ScaledOffsetAllocator> allocator_;
  uint64_t allocatable_bytes_ = 0;
};

// pinned_pool.rs:347-456: round-robin over shards with fallback to all.
class ShardedPinnedPool {
 public:
  static std::unique_ptr<ShardedPinnedPool> create(uint64_t total_capacity, uint32_t num_shards,
                                                   bool use_hugepages, bool ssd_enabled,
                                                   uint64_t unit_size_hint, NumaNode node,
                                                   std::string* err, int* status);
  std::shared_ptr<PinnedAllocation> allocate(uint64_t size);
  void usage(uint64_t* used, uint64_t* total);
  uint64_t largest_free_allocation();
  void memory_regions(std::vector<std::pair<uint8_t*, uint64_t>>* out) const;
  size_t num_shards() const { return shards_.size(); }

 private:
  std::vector<std::shared_ptr<PinnedMemoryPool>> shards_;
  std::atomic<uint64_t> cursor_{0};
};

// pinned_pool.rs:458-597 (per-NUMA pools) and :599-715 (the facade).
class PinnedAllocator {
 public:
  static std::unique_ptr<PinnedAllocator> new_global(uint64_t capacity, uint32_t num_shards,
                                                     bool use_hugepages, bool ssd_enabled,
                                                     uint64_t unit_hint, std::string* err,
                                                     int* status);
  // Empty `numa_nodes` falls back to a global allocator (pinned_pool.rs:640-646).
  static std::unique_ptr<PinnedAllocator> new_numa(uint64_t capacity,
                                                   const std::vector<NumaNode>& numa_nodes,
                                                   uint32_t num_shards, bool use_hugepages,
                                                   bool ssd_enabled, uint64_t unit_hint,
                                                   std::string* err, int* status);
  // Global: `numa_node` ignored.  NUMA: that node's pool; UNKNOWN or a node
  // without a pool -> nullptr (pinned_pool.rs:563-571).
  std::shared_ptr<PinnedAllocation> allocate(uint64_t size, NumaNode numa_node);
  void usage(uint64_t* used, uint64_t* total);
  uint64_t largest_free_allocation_for_node(NumaNode numa_node);
  bool is_numa() const { return is_numa_; }
  void memory_regions(std::vector<std::pair<uint8_t*, uint64_t>>* out) const;

 private:
  bool is_numa_ = false;
  std::unique_ptr<ShardedPinnedPool> global_;
  std::map<uint32_t, std::unique_ptr<ShardedPinnedPool>> per_node_;
};

}  // namespace pf
