#include "pf_alloc.hpp"

#include <mutex>

#include "pf_common.hpp"

namespace pf {

namespace {

constexpr uint32_t kMantissaBits = 3;
constexpr uint32_t kMantissaValue = 1u << kMantissaBits;
constexpr uint32_t kMantissaMask = kMantissaValue - 1;
constexpr uint32_t kTopShift = 3;
constexpr uint32_t kLeafMask = 7;

// Lowest set bit at position >= start, or kNoSpace.
uint32_t lowest_set_bit_from(uint32_t mask, uint32_t start) {
  if (start >= 32) return OffsetAllocator::kNoSpace;
  uint32_t after = mask & (~0u << start);
  if (after == 0) return OffsetAllocator::kNoSpace;
  return static_cast<uint32_t>(__builtin_ctz(after));
}

}  // namespace

uint32_t OffsetAllocator::uint_to_float_round_up(uint32_t size) {
  uint32_t exp = 0, mantissa = 0;
  if (size < kMantissaValue) {
    mantissa = size;  // denormal: exact
  } else {
    uint32_t highest = 31u - static_cast<uint32_t>(__builtin_clz(size));
    uint32_t start = highest - kMantissaBits;
    exp = start + 1;
    mantissa = (size >> start) & kMantissaMask;
    uint32_t low_mask = (1u << start) - 1;
    if (size & low_mask) ++mantissa;  // may carry into the exponent below
  }
  return (exp << kMantissaBits) + mantissa;
}

uint32_t OffsetAllocator::uint_to_float_round_down(uint32_t size) {
  uint32_t exp = 0, mantissa = 0;
  if (size < kMantissaValue) {
    mantissa = size;
  } else {
    uint32_t highest = 31u - static_cast<uint32_t>(__builtin_clz(size));
    uint32_t start = highest - kMantissaBits;
    exp = start + 1;
    mantissa = (size >> start) & kMantissaMask;
  }
  return (exp << kMantissaBits) | mantissa;
}

uint32_t OffsetAllocator::float_to_uint(uint32_t f) {
  uint32_t exp = f >> kMantissaBits;
  uint32_t mantissa = f & kMantissaMask;
  if (exp == 0) return mantissa;
  return (mantissa | kMantissaValue) << (exp - 1);
}

OffsetAllocator::OffsetAllocator(uint32_t size, uint32_t max_allocs)
    : size_(size), max_allocs_(max_allocs) {
  for (uint32_t i = 0; i < kLeafBins; ++i) bin_indices_[i] = kUnused;
  if (size_ > 0 && max_allocs_ > 0) insert_node_into_bin(size_, 0);
}

uint32_t OffsetAllocator::pop_free_node() {
  if (!recycled_.empty()) {
    uint32_t i = recycled_.back();
    recycled_.pop_back();
    return i;
  }
  uint32_t i = fresh_++;
  if (i >= nodes_.size()) nodes_.resize(static_cast<size_t>(i) + 1);
  return i;
}

void OffsetAllocator::push_free_node(uint32_t index) { recycled_.push_back(index); }

uint32_t OffsetAllocator::insert_node_into_bin(uint32_t size, uint32_t data_offset) {
  uint32_t bin = uint_to_float_round_down(size);
  uint32_t top = bin >> kTopShift, leaf = bin & kLeafMask;
  if (bin_indices_[bin] == kUnused) {
    used_bins_[top] |= static_cast<uint8_t>(1u << leaf);
    used_bins_top_ |= 1u << top;
  }
  uint32_t head = bin_indices_[bin];
  uint32_t index = pop_free_node();
  Node& n = nodes_[index];
  n = Node();
  n.data_offset = data_offset;
  n.data_size = size;
  n.bin_next = head;
  if (head != kUnused) nodes_[head].bin_prev = index;
  bin_indices_[bin] = index;
  free_storage_ += size;
  return index;
}

void OffsetAllocator::remove_node_from_bin(uint32_t index) {
  Node& n = nodes_[index];
  if (n.bin_prev != kUnused) {
    nodes_[n.bin_prev].bin_next = n.bin_next;
    if (n.bin_next != kUnused) nodes_[n.bin_next].bin_prev = n.bin_prev;
  } else {
    uint32_t bin = uint_to_float_round_down(n.data_size);
    uint32_t top = bin >> kTopShift, leaf = bin & kLeafMask;
    bin_indices_[bin] = n.bin_next;
    if (n.bin_next != kUnused) nodes_[n.bin_next].bin_prev = kUnused;
    if (bin_indices_[bin] == kUnused) {
      used_bins_[top] &= static_cast<uint8_t>(~(1u << leaf));
      if (used_bins_[top] == 0) used_bins_top_ &= ~(1u << top);
    }
  }
  push_free_node(index);
  free_storage_ -= n.data_size;
}

OffsetAllocator::Allocation OffsetAllocator::allocate(uint32_t size) {
  // One spare node is kept for the remainder a split produces.
  if (free_node_count() <= 1) return Allocation();
  uint32_t min_bin = uint_to_float_round_up(size);
  uint32_t min_top = min_bin >> kTopShift, min_leaf = min_bin & kLeafMask;
  uint32_t top = min_top, leaf = kNoSpace;
  if (top < kTopBins && (used_bins_top_ & (1u << top))) {
    leaf = lowest_set_bit_from(used_bins_[top], min_leaf);
  }
  if (leaf == kNoSpace) {
    top = lowest_set_bit_from(used_bins_top_, min_top + 1);
    if (top == kNoSpace) return Allocation();
    leaf = static_cast<uint32_t>(__builtin_ctz(used_bins_[top]));
  }
  uint32_t bin = (top << kTopShift) | leaf;
  uint32_t index = bin_indices_[bin];
  Node& n = nodes_[index];
  uint32_t total = n.data_size;
  n.data_size = size;
  n.used = true;
  bin_indices_[bin] = n.bin_next;
  if (n.bin_next != kUnused) nodes_[n.bin_next].bin_prev = kUnused;
  free_storage_ -= total;
  if (bin_indices_[bin] == kUnused) {
    used_bins_[top] &= static_cast<uint8_t>(~(1u << leaf));
    if (used_bins_[top] == 0) used_bins_top_ &= ~(1u << top);
  }
  uint32_t remainder = total - size;
  if (remainder > 0) {
    uint32_t data_offset = n.data_offset;
    uint32_t old_next = n.neighbor_next;
    uint32_t fresh = insert_node_into_bin(remainder, data_offset + size);  // may move nodes_
    Node& self = nodes_[index];
    if (old_next != kUnused) nodes_[old_next].neighbor_prev = fresh;
    nodes_[fresh].neighbor_prev = index;
    nodes_[fresh].neighbor_next = old_next;
    self.neighbor_next = fresh;
  }
  Allocation a;
  a.offset = nodes_[index].data_offset;
  a.metadata = index;
  return a;
}

void OffsetAllocator::free(Allocation a) {
  if (!a.ok() || a.metadata >= nodes_.size()) return;
  uint32_t index = a.metadata;
  if (!nodes_[index].used) return;  // double free: ignore
  uint32_t offset = nodes_[index].data_offset;
  uint32_t size = nodes_[index].data_size;
  uint32_t prev = nodes_[index].neighbor_prev;
  if (prev != kUnused && !nodes_[prev].used) {
    offset = nodes_[prev].data_offset;
    size += nodes_[prev].data_size;
    uint32_t prev_prev = nodes_[prev].neighbor_prev;
    remove_node_from_bin(prev);
    nodes_[index].neighbor_prev = prev_prev;
  }
  uint32_t next = nodes_[index].neighbor_next;
  if (next != kUnused && !nodes_[next].used) {
    size += nodes_[next].data_size;
    uint32_t next_next = nodes_[next].neighbor_next;
    remove_node_from_bin(next);
    nodes_[index].neighbor_next = next_next;
  }
  uint32_t neighbor_next = nodes_[index].neighbor_next;
  uint32_t neighbor_prev = nodes_[index].neighbor_prev;
  nodes_[index].used = false;
  push_free_node(index);
  uint32_t combined = insert_node_into_bin(size, offset);
  if (neighbor_next != kUnused) {
    nodes_[combined].neighbor_next = neighbor_next;
    nodes_[neighbor_next].neighbor_prev = combined;
  }
  if (neighbor_prev != kUnused) {
    nodes_[combined].neighbor_prev = neighbor_prev;
    nodes_[neighbor_prev].neighbor_next = combined;
  }
}

uint32_t OffsetAllocator::allocation_size(Allocation a) const {
  if (!a.ok() || a.metadata >= nodes_.size()) return 0;
  return nodes_[a.metadata].data_size;
}

OffsetAllocator::StorageReport OffsetAllocator::storage_report() const {
  StorageReport r;
  if (free_node_count() > 1) {
    r.total_free_space = free_storage_;
    if (used_bins_top_ != 0) {
      uint32_t top = 31u - static_cast<uint32_t>(__builtin_clz(used_bins_top_));
      uint32_t leaf = 31u - static_cast<uint32_t>(__builtin_clz(static_cast<uint32_t>(used_bins_[top])));
      r.largest_free_region = float_to_uint((top << kTopShift) | leaf);
    }
  }
  return r;
}

std::string AllocatorError::to_string() const {
  switch (kind) {
    case InvalidUnitSize:
      return "unit size must be greater than zero";
    case CapacityTooLarge:
      return "capacity " + std::to_string(bytes) + " bytes with unit " + std::to_string(unit_size) +
             " overflows u32 backing allocator";
    case RequestTooLarge:
      return "request " + std::to_string(bytes) + " bytes with unit " + std::to_string(unit_size) +
             " overflows u32 backing allocator";
    default:
      return "";
  }
}

ScaledOffsetAllocator* ScaledOffsetAllocator::create(uint64_t total_bytes, uint64_t unit_size,
                                                     uint32_t max_allocs, AllocatorError* err) {
  if (unit_size == 0) {
    if (err) *err = {AllocatorError::InvalidUnitSize, 0, 0};
    return nullptr;
  }
  uint64_t units = total_bytes / unit_size;
  if (units > 0xFFFFFFFFull) {
    if (err) *err = {AllocatorError::CapacityTooLarge, total_bytes, unit_size};
    return nullptr;
  }
  return new ScaledOffsetAllocator(unit_size, static_cast<uint32_t>(units), max_allocs);
}

int ScaledOffsetAllocator::allocate(uint64_t size_bytes, Allocation* out, AllocatorError* err) {
  if (size_bytes == 0) return 0;
  uint64_t units = size_bytes / unit_size_ + (size_bytes % unit_size_ ? 1 : 0);
  if (units > 0xFFFFFFFFull) {
    if (err) *err = {AllocatorError::RequestTooLarge, size_bytes, unit_size_};
    return -1;
  }
  OffsetAllocator::Allocation raw = inner_.allocate(static_cast<uint32_t>(units));
  if (!raw.ok()) return 0;
  out->raw = raw;
  out->offset_bytes = static_cast<uint64_t>(raw.offset) * unit_size_;
  out->size_bytes = static_cast<uint64_t>(inner_.allocation_size(raw)) * unit_size_;
  return 1;
}

void ScaledOffsetAllocator::free(const Allocation& a) { inner_.free(a.raw); }

ScaledOffsetAllocator::StorageReportBytes ScaledOffsetAllocator::storage_report() const {
  auto r = inner_.storage_report();
  return {static_cast<uint64_t>(r.total_free_space) * unit_size_,
          static_cast<uint64_t>(r.largest_free_region) * unit_size_};
}

}  // namespace pf
