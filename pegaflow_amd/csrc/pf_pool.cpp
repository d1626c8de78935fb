#include "pf_pool.hpp"

#include "pf_common.hpp"

namespace pf {

// ---------------------------------------------------------------------------
// PinnedAllocation
// ---------------------------------------------------------------------------

PinnedAllocation::~PinnedAllocation() {
  if (pool_) pool_->free_internal(allocation_);
}

bool PinnedAllocation::mapped_ptr_at(uint64_t offset, uint64_t size, MappedPinnedPtr* out) const {
  uint64_t end = 0;
  if (__builtin_add_overflow(offset, size, &end) || end > allocation_.size_bytes) return false;
  *out = mapped_ptr().add(offset);
  return true;
}

bool PinnedAllocation::mapped_ptr_for_host_range(const uint8_t* host_ptr, uint64_t size,
                                                 MappedPinnedPtr* out) const {
  if (host_ptr < ptr_) return false;
  return mapped_ptr_at(static_cast<uint64_t>(host_ptr - ptr_), size, out);
}

// ---------------------------------------------------------------------------
// PinnedMemoryPool
// ---------------------------------------------------------------------------

uint64_t PinnedMemoryPool::compute_unit_size(uint64_t pool_size, uint64_t hint) {
  const uint64_t max_units = 0xFFFFFFFFull;
  uint64_t min_unit_for_capacity = pool_size / max_units + (pool_size % max_units ? 1 : 0);
  uint64_t base = hint ? hint : kUnitAlignment;
  uint64_t unit = base > min_unit_for_capacity ? base : min_unit_for_capacity;
  return (unit + kUnitAlignment - 1) / kUnitAlignment * kUnitAlignment;
}

AllocStrategy PinnedMemoryPool::pick_strategy(bool use_hugepages, bool ssd_enabled) {
  if (use_hugepages) return AllocStrategy::HugePages;
  if (ssd_enabled) return AllocStrategy::Regular;
  return AllocStrategy::HipHostAlloc;
}

std::shared_ptr<PinnedMemoryPool> PinnedMemoryPool::create(uint64_t pool_size, bool use_hugepages,
                                                           bool ssd_enabled,
                                                           uint64_t unit_size_hint, NumaNode node,
                                                           std::string* err, int* status) {
  if (pool_size == 0) {
    *err = "Pinned memory pool size must be greater than zero";
    *status = PF_ERR_INVALID_ARGUMENT;
    return nullptr;
  }
  std::shared_ptr<PinnedMemoryPool> pool(new PinnedMemoryPool());
  pool->backing_ =
      PinnedMemory::allocate(pool_size, pick_strategy(use_hugepages, ssd_enabled), node, err, status);
  if (!pool->backing_) {
    *err = "Failed to allocate pinned memory pool: " + *err;
    return nullptr;
  }
  const uint64_t actual = pool->backing_->size();
  const uint64_t unit = compute_unit_size(actual, unit_size_hint);
  pool->allocatable_bytes_ = actual / unit * unit;
  AllocatorError aerr;
  pool->allocator_.reset(ScaledOffsetAllocator::create(actual, unit, kMaxAllocs, &aerr));
  if (!pool->allocator_) {
    *err = "Failed to create memory allocator (size=" + std::to_string(actual) +
           ", unit=" + std::to_string(unit) + "): " + aerr.to_string();
    *status = PF_ERR_INVALID_ARGUMENT;
    return nullptr;
  }
  return pool;
}

std::shared_ptr<PinnedAllocation> PinnedMemoryPool::allocate(uint64_t size) {
  if (size == 0) return nullptr;
  ScaledOffsetAllocator::Allocation a;
  {
    std::lock_guard<std::mutex> lock(mu_);
    AllocatorError aerr;
    if (allocator_->allocate(size, &a, &aerr) != 1) return nullptr;  // exhausted or too large
  }
  uint64_t end = 0;
  if (__builtin_add_overflow(a.offset_bytes, a.size_bytes, &end) || end > backing_->size()) {
    // The allocator handed out a range outside the backing region: a bug.
    std::lock_guard<std::mutex> lock(mu_);
    allocator_->free(a);
    return nullptr;
  }
  return std::make_shared<PinnedAllocation>(a, backing_->as_ptr() + a.offset_bytes,
                                            backing_->device_ptr() + a.offset_bytes,
                                            shared_from_this());
}

void PinnedMemoryPool::free_internal(const ScaledOffsetAllocator::Allocation& a) {
  std::lock_guard<std::mutex> lock(mu_);
  allocator_->free(a);
}

void PinnedMemoryPool::usage(uint64_t* used, uint64_t* total) {
  std::lock_guard<std::mutex> lock(mu_);
  auto r = allocator_->storage_report();
  *total = allocator_->total_bytes();
  *used = *total - r.total_free_bytes;
}

uint64_t PinnedMemoryPool::largest_free_allocation() {
  std::lock_guard<std::mutex> lock(mu_);
  return allocator_->storage_report().largest_free_allocation_bytes;
}

void PinnedMemoryPool::memory_region(uint8_t** ptr, uint64_t* len) const {
  *ptr = backing_->as_ptr();
  *len = backing_->size();
}

// ---------------------------------------------------------------------------
// ShardedPinnedPool
// ---------------------------------------------------------------------------

std::unique_ptr<ShardedPinnedPool> ShardedPinnedPool::create(uint64_t total_capacity,
                                                             uint32_t num_shards,
                                                             bool use_hugepages, bool ssd_enabled,
                                                             uint64_t unit_size_hint, NumaNode node,
                                                             std::string* err, int* status) {
  if (num_shards < 1) num_shards = 1;
  const uint64_t per_shard = total_capacity / num_shards;
  std::unique_ptr<ShardedPinnedPool> sp(new ShardedPinnedPool());
  for (uint32_t i = 0; i < num_shards; ++i) {
    auto shard = PinnedMemoryPool::create(per_shard, use_hugepages, ssd_enabled, unit_size_hint,
                                          node, err, status);
    if (!shard) return nullptr;
    sp->shards_.push_back(std::move(shard));
  }
  return sp;
}

std::shared_ptr<PinnedAllocation> ShardedPinnedPool::allocate(uint64_t size) {
  const uint64_t n = shards_.size();
  const uint64_t start = cursor_.fetch_add(1, std::memory_order_relaxed) % n;
  for (uint64_t i = 0; i < n; ++i) {
    if (auto a = shards_[(start + i) % n]->allocate(size)) return a;
  }
  return nullptr;
}

void ShardedPinnedPool::usage(uint64_t* used, uint64_t* total) {
  *used = *total = 0;
  for (auto& s : shards_) {
    uint64_t u = 0, t = 0;
    s->usage(&u, &t);
    *used += u;
    *total += t;
  }
}

uint64_t ShardedPinnedPool::largest_free_allocation() {
  uint64_t best = 0;
  for (auto& s : shards_) best = std::max(best, s->largest_free_allocation());
  return best;
}

void ShardedPinnedPool::memory_regions(std::vector<std::pair<uint8_t*, uint64_t>>* out) const {
  for (auto& s : shards_) {
    uint8_t* p = nullptr;
    uint64_t len = 0;
    s->memory_region(&p, &len);
    out->emplace_back(p, len);
  }
}

// ---------------------------------------------------------------------------
// PinnedAllocator
// ---------------------------------------------------------------------------

std::unique_ptr<PinnedAllocator> PinnedAllocator::new_global(uint64_t capacity,
                                                             uint32_t num_shards,
                                                             bool use_hugepages, bool ssd_enabled,
                                                             uint64_t unit_hint, std::string* err,
                                                             int* status) {
  std::unique_ptr<PinnedAllocator> a(new PinnedAllocator());
  a->global_ = ShardedPinnedPool::create(capacity, num_shards, use_hugepages, ssd_enabled,
                                         unit_hint, NumaNode(), err, status);
  if (!a->global_) return nullptr;
  return a;
}

std::unique_ptr<PinnedAllocator> PinnedAllocator::new_numa(uint64_t capacity,
                                                           const std::vector<NumaNode>& numa_nodes,
                                                           uint32_t num_shards, bool use_hugepages,
                                                           bool ssd_enabled, uint64_t unit_hint,
                                                           std::string* err, int* status) {
  if (numa_nodes.empty()) {
    return new_global(capacity, num_shards, use_hugepages, ssd_enabled, unit_hint, err, status);
  }
  std::unique_ptr<PinnedAllocator> a(new PinnedAllocator());
  a->is_numa_ = true;
  const uint64_t per_node = capacity / numa_nodes.size();
  int device = 0;
  (void)hipGetDevice(&device);
  for (const NumaNode& node : numa_nodes) {
    if (node.is_unknown()) continue;
    std::unique_ptr<ShardedPinnedPool> pool;
    std::string build_err, numa_err;
    int build_status = PF_OK;
    // Built on a thread pinned to the node so first touch lands there
    // (pinned_pool.rs:517-531).
    bool ran = run_on_numa(node, [&] {
      (void)hipSetDevice(device);
      pool = ShardedPinnedPool::create(per_node, num_shards, use_hugepages, ssd_enabled, unit_hint,
                                       node, &build_err, &build_status);
    }, &numa_err);
    if (!ran || !pool) {
      *err = "Failed to create pool on NUMA" + std::to_string(node.id) + ": " +
             (ran ? build_err : numa_err);
      *status = ran ? build_status : PF_ERR_STORAGE;
      return nullptr;
    }
    a->per_node_[node.id] = std::move(pool);
  }
  return a;
}

std::shared_ptr<PinnedAllocation> PinnedAllocator::allocate(uint64_t size, NumaNode numa_node) {
  if (!is_numa_) return global_->allocate(size);
  if (numa_node.is_unknown()) return nullptr;
  auto it = per_node_.find(numa_node.id);
  if (it == per_node_.end()) return nullptr;
  return it->second->allocate(size);
}

void PinnedAllocator::usage(uint64_t* used, uint64_t* total) {
  if (!is_numa_) {
    global_->usage(used, total);
    return;
  }
  *used = *total = 0;
  for (auto& kv : per_node_) {
    uint64_t u = 0, t = 0;
    kv.second->usage(&u, &t);
    *used += u;
    *total += t;
  }
}

uint64_t PinnedAllocator::largest_free_allocation_for_node(NumaNode numa_node) {
  if (!is_numa_) return global_->largest_free_allocation();
  if (numa_node.is_unknown()) return 0;
  auto it = per_node_.find(numa_node.id);
  return it == per_node_.end() ? 0 : it->second->largest_free_allocation();
}

void PinnedAllocator::memory_regions(std::vector<std::pair<uint8_t*, uint64_t>>* out) const {
  if (!is_numa_) {
    global_->memory_regions(out);
    return;
  }
  for (auto& kv : per_node_) kv.second->memory_regions(out);
}

}  // namespace pf
