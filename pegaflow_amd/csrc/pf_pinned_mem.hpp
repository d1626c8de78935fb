// Pinned, device-mapped host memory in three strategies.  Follows
// pegaflow-core/src/pinned_mem.rs:100-397 of the reference:
//   Regular   : mmap + parallel NUMA-pinned pre-touch + hipHostRegister(Mapped)
//   HipAlloc  : hipHostMalloc(Mapped)
//   HugePages : mmap(MAP_HUGETLB) + pre-touch + hipHostRegister(Mapped)
#pragma once

#include <cstdint>
#include <memory>
#include <string>

#include "pf_numa.hpp"

namespace pf {

enum class AllocStrategy : int { Regular = 0, HipHostAlloc = 1, HugePages = 2 };

// pinned_mem.rs:46-60.  0 when /proc/meminfo has no usable Hugepagesize line.
uint64_t huge_page_size();
// Parse "Hugepagesize:  2048 kB" out of a meminfo text (pinned_mem.rs:48-60).
uint64_t parse_huge_page_size(const std::string& meminfo);
// pinned_mem.rs:368-376: min(ceil(size / 1 GiB), ncpu), at least 1.
uint64_t touch_threads(uint64_t size);
// pinned_mem.rs:326-360: fault in every page from threads pinned to `node`.
void parallel_pre_touch(uint8_t* ptr, uint64_t size, NumaNode node);

class PinnedMemory {
 public:
  // Returns nullptr and fills *err / *status on failure.
  static std::unique_ptr<PinnedMemory> allocate(uint64_t size, AllocStrategy strategy,
                                                NumaNode node, std::string* err, int* status);
  ~PinnedMemory();
  PinnedMemory(const PinnedMemory&) = delete;
  PinnedMemory& operator=(const PinnedMemory&) = delete;

  uint8_t* as_ptr() const { return ptr_; }
  uint8_t* device_ptr() const { return device_ptr_; }
  uint64_t size() const { return size_; }
  AllocStrategy strategy() const { return strategy_; }
  // Give up ownership: the destructor will no longer free the region.
  void disown() { ptr_ = nullptr; }

 private:
  PinnedMemory() = default;
  uint8_t* ptr_ = nullptr;
  uint8_t* device_ptr_ = nullptr;
  uint64_t size_ = 0;
  AllocStrategy strategy_ = AllocStrategy::HipHostAlloc;
};

}  // namespace pf
