// Host-side images of saved blocks.  Follows pegaflow-core/src/block.rs:62-454
// and pegaflow-common/src/block.rs:1-43 of the reference.
#pragma once

#include <chrono>
#include <cstdint>
#include <memory>
#include <string>
#include <string_view>
#include <vector>

#include "pf_pool.hpp"

namespace pf {

// pegaflow-common/src/block.rs:5-21: (namespace, hash bytes).  The namespace
// is the small integer the engine assigned to its name, and the digest of the
// pair is computed once, when the key (or a view of it) is built: a save looks
// every key up twice and inserts it once, a query looks it up once.
inline size_t block_key_digest(uint32_t ns, std::string_view hash) {
  return std::hash<std::string_view>{}(hash) ^ (static_cast<size_t>(ns) * 0x9E3779B97F4A7C15ull);
}
struct BlockKey {
  uint32_t ns = 0;
  std::string hash;  // raw bytes
  size_t digest = 0;
  BlockKey() = default;
  BlockKey(uint32_t ns_id, std::string hash_bytes)
      : ns(ns_id), hash(std::move(hash_bytes)), digest(block_key_digest(ns, hash)) {}
};
// The same without owning the bytes, for look-ups.
struct BlockKeyView {
  uint32_t ns = 0;
  std::string_view hash;
  size_t digest = 0;
  BlockKeyView(uint32_t ns_id, std::string_view hash_bytes)
      : ns(ns_id), hash(hash_bytes), digest(block_key_digest(ns, hash)) {}
};
struct BlockKeyHash {
  using is_transparent = void;
  size_t operator()(const BlockKey& k) const { return k.digest; }
  size_t operator()(const BlockKeyView& k) const { return k.digest; }
};
struct BlockKeyEqual {
  using is_transparent = void;
  template <typename A, typename B>
  bool operator()(const A& a, const B& b) const {
    return a.digest == b.digest && a.ns == b.ns && std::string_view(a.hash) == std::string_view(b.hash);
  }
};

// pegaflow-common/src/block.rs:30-43: group 0 keeps the raw hash, groups >= 1
// append the big-endian group id.
inline std::string group_hash(std::string hash, uint32_t group_id) {
  if (group_id == 0) return hash;
  hash.push_back(static_cast<char>((group_id >> 24) & 0xFF));
  hash.push_back(static_cast<char>((group_id >> 16) & 0xFF));
  hash.push_back(static_cast<char>((group_id >> 8) & 0xFF));
  hash.push_back(static_cast<char>(group_id & 0xFF));
  return hash;
}

// block.rs:62-88: one contiguous range of pinned memory; keeps its allocation alive.
class Segment {
 public:
  // False when [host_ptr, host_ptr + size) is not inside `allocation`.
  static bool create(uint8_t* host_ptr, uint64_t size, std::shared_ptr<PinnedAllocation> allocation,
                     Segment* out) {
    MappedPinnedPtr p;
    if (!allocation || !allocation->mapped_ptr_for_host_range(host_ptr, size, &p)) return false;
    out->ptr_ = p;
    out->size_ = size;
    out->allocation_ = std::move(allocation);
    return true;
  }
  MappedPinnedPtr ptr() const { return ptr_; }
  uint64_t size() const { return size_; }
  uint64_t allocation_id() const { return allocation_ ? allocation_->allocation_id() : 0; }

 private:
  MappedPinnedPtr ptr_;
  uint64_t size_ = 0;
  std::shared_ptr<PinnedAllocation> allocation_;
};

// block.rs:90-199: an ordered list of segments, layout-agnostic.  One or two
// segments (every layout on the path) live inline; more spill to the heap.
class RawBlock {
 public:
  RawBlock() = default;
  explicit RawBlock(std::vector<Segment> segments) {
    n_ = segments.size();
    for (size_t i = 0; i < segments.size(); ++i) {
      total_size_ += segments[i].size();
      if (i < 2) {
        inline_[i] = std::move(segments[i]);
      } else {
        extra_.push_back(std::move(segments[i]));
      }
    }
  }
  static RawBlock single_segment(Segment s) {
    RawBlock b;
    b.n_ = 1;
    b.total_size_ = s.size();
    b.inline_[0] = std::move(s);
    return b;
  }
  static RawBlock two_segments(Segment k, Segment v) {
    RawBlock b;
    b.n_ = 2;
    b.total_size_ = k.size() + v.size();
    b.inline_[0] = std::move(k);
    b.inline_[1] = std::move(v);
    return b;
  }
  size_t num_segments() const { return n_; }
  bool segment_mapped_ptr(size_t i, MappedPinnedPtr* out) const {
    if (i >= n_) return false;
    *out = at(i).ptr();
    return true;
  }
  uint64_t segment_allocation_id(size_t i) const { return i < n_ ? at(i).allocation_id() : 0; }
  uint64_t segment_size(size_t i) const { return i < n_ ? at(i).size() : 0; }
  uint64_t memory_footprint() const { return total_size_; }

 private:
  const Segment& at(size_t i) const { return i < 2 ? inline_[i] : extra_[i - 2]; }
  Segment inline_[2];
  std::vector<Segment> extra_;
  size_t n_ = 0;
  uint64_t total_size_ = 0;
};

// block.rs:255-330: immutable once every slot is filled.
class SealedBlock {
 public:
  explicit SealedBlock(std::vector<RawBlock> slots) : slots_(std::move(slots)) {
    for (const auto& b : slots_) footprint_ += b.memory_footprint();
  }
  const RawBlock* get_slot(size_t slot_id) const {
    return slot_id < slots_.size() ? &slots_[slot_id] : nullptr;
  }
  size_t num_slots() const { return slots_.size(); }
  uint64_t memory_footprint() const { return footprint_; }

 private:
  std::vector<RawBlock> slots_;
  uint64_t footprint_ = 0;
};

// block.rs:346-454: slots arrive one by one; seals when none remain.
class InflightBlock {
 public:
  using Clock = std::chrono::steady_clock;
  // `created` lets a save that begins thousands of blocks read the clock once.
  explicit InflightBlock(size_t total_slots, Clock::time_point created = Clock::now())
      : slots_(total_slots), remaining_(total_slots), created_(created) {}
  enum class Insert { Inserted, Completed, Duplicate };
  Insert insert_slot(size_t slot_id, RawBlock block) {
    if (slot_id >= slots_.size() || filled(slot_id)) return Insert::Duplicate;
    slots_[slot_id] = std::move(block);
    --remaining_;
    return remaining_ == 0 ? Insert::Completed : Insert::Inserted;
  }
  // The empty slot to build a block in, or null when it is taken or out of
  // range; the caller confirms with slot_filled() once the block is in place.
  RawBlock* empty_slot(size_t slot_id) {
    return slot_id >= slots_.size() || filled(slot_id) ? nullptr : &slots_[slot_id];
  }
  Insert slot_filled() {
    --remaining_;
    return remaining_ == 0 ? Insert::Completed : Insert::Inserted;
  }
  size_t total_slots() const { return slots_.size(); }
  size_t filled_count() const { return slots_.size() - remaining_; }
  bool complete() const { return remaining_ == 0; }
  // Time since the first slot arrived (write_path.rs:302-330 collects blocks
  // that stay incomplete for too long).
  Clock::duration age() const { return Clock::now() - created_; }
  std::shared_ptr<SealedBlock> seal() { return std::make_shared<SealedBlock>(std::move(slots_)); }
  // Move every filled slot of `other` into this block (slots already filled
  // here are kept: a repeated slot is a duplicate, as in insert_slot).
  Insert absorb(InflightBlock&& other) {
    Insert last = Insert::Duplicate;
    const size_t n = other.slots_.size() < slots_.size() ? other.slots_.size() : slots_.size();
    for (size_t i = 0; i < n; ++i) {
      if (!other.filled(i)) continue;
      Insert r = insert_slot(i, std::move(other.slots_[i]));
      if (r == Insert::Completed) return r;
      if (r == Insert::Inserted) last = r;
    }
    return last;
  }

 private:
  // A slot that holds a block has at least one segment.
  bool filled(size_t slot_id) const { return slots_[slot_id].num_segments() != 0; }
  std::vector<RawBlock> slots_;
  size_t remaining_;
  Clock::time_point created_;
};

}  // namespace pf
