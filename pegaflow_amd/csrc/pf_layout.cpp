#include "pf_layout.hpp"

#include "pf_common.hpp"

namespace pf {

namespace {

bool mul_ok(uint64_t a, uint64_t b, uint64_t* out) { return !__builtin_mul_overflow(a, b, out); }
bool add_ok(uint64_t a, uint64_t b, uint64_t* out) { return !__builtin_add_overflow(a, b, out); }

std::string u(uint64_t v) { return std::to_string(v); }

bool set(std::string* err, std::string msg) {
  if (err) *err = std::move(msg);
  return false;
}

}  // namespace

bool KVCacheLayout::create(uint64_t data_ptr, uint64_t size_bytes, uint64_t num_blocks,
                           uint64_t segment_bytes, uint64_t kv_stride_bytes, uint64_t segments,
                           KVCacheLayout* out, std::string* err) {
  if (data_ptr == 0) return set(err, "data_ptr must not be null");
  if (size_bytes == 0) return set(err, "size_bytes must be > 0");
  if (segment_bytes == 0 || num_blocks == 0 || segments == 0) {
    return set(err, "segment_bytes, num_blocks, and segments must be non-zero");
  }
  uint64_t end_addr = 0;
  if (!add_ok(data_ptr, size_bytes, &end_addr)) {
    return set(err, "data_ptr + size_bytes overflows the address space");
  }
  uint64_t block_bytes = 0;
  if (!mul_ok(segment_bytes, segments, &block_bytes)) return set(err, "block size overflow");

  bool split = false;
  if (segments > 1) {
    if (kv_stride_bytes == 0) return set(err, "kv_stride_bytes must be > 0 when segments > 1");
    if (kv_stride_bytes < segment_bytes) {
      return set(err, "kv_stride_bytes " + u(kv_stride_bytes) + " < segment_bytes " +
                          u(segment_bytes) + ": segments would overlap");
    }
    if (kv_stride_bytes > segment_bytes) {
      if (segments != 2) {
        return set(err, "split layout (kv_stride_bytes " + u(kv_stride_bytes) +
                            " > segment_bytes " + u(segment_bytes) +
                            ") supports exactly 2 segments, got " + u(segments));
      }
      split = true;
    }
    // kv_stride_bytes == segment_bytes: K and V adjacent, one range.
  }

  KVCacheLayout l;
  l.c_.data_ptr = data_ptr;
  l.c_.size_bytes = size_bytes;
  l.c_.num_blocks = num_blocks;
  l.c_.block_stride_bytes = split ? segment_bytes : block_bytes;
  l.c_.segment_bytes = segment_bytes;
  l.c_.segments = segments;
  l.c_.padded_segment_bytes = segment_bytes;
  l.c_.kv_stride_bytes = split ? kv_stride_bytes : 0;
  l.c_.split = split ? 1 : 0;
  if (!l.check_bounds(err)) return false;
  *out = l;
  return true;
}

bool KVCacheLayout::with_block_stride(uint64_t stride, std::string* err) {
  uint64_t min_stride = is_split() ? c_.segment_bytes : block_bytes();
  if (stride < min_stride) {
    return set(err, "block_stride " + u(stride) + " must be >= " + u(min_stride) +
                        ": blocks would overlap");
  }
  KVCacheLayout candidate = *this;
  candidate.c_.block_stride_bytes = stride;
  if (!candidate.check_bounds(err)) return false;
  *this = candidate;
  return true;
}

void KVCacheLayout::with_ssd_padding(uint64_t alignment) {
  if (alignment == 0) return;
  uint64_t rem = c_.segment_bytes % alignment;
  c_.padded_segment_bytes = rem == 0 ? c_.segment_bytes : c_.segment_bytes + (alignment - rem);
}

bool KVCacheLayout::check_bounds(std::string* err) const {
  uint64_t span = 0;  // (num_blocks - 1) * block_stride
  uint64_t end = 0;
  if (!is_split()) {
    uint64_t bb = block_bytes();
    if (c_.block_stride_bytes < bb) {
      return set(err, "block_stride " + u(c_.block_stride_bytes) + " must be >= block_bytes " +
                          u(bb) + ": blocks would overlap");
    }
    if (!mul_ok(c_.num_blocks - 1, c_.block_stride_bytes, &span) || !add_ok(span, bb, &end)) {
      return set(err, "memory layout overflow");
    }
  } else {
    if (c_.block_stride_bytes < c_.segment_bytes) {
      return set(err, "block_stride " + u(c_.block_stride_bytes) + " must be >= segment_bytes " +
                          u(c_.segment_bytes) + ": blocks would overlap");
    }
    if (!check_split_segments_disjoint(err)) return false;
    uint64_t last_seg_end = 0;
    if (!mul_ok(c_.num_blocks - 1, c_.block_stride_bytes, &span) ||
        !add_ok(span, c_.segment_bytes, &last_seg_end) ||
        !add_ok(c_.kv_stride_bytes, last_seg_end, &end)) {
      return set(err, "memory layout overflow");
    }
  }
  if (end > c_.size_bytes) {
    return set(err, "registered memory too small: need " + u(end) + " bytes, got " +
                        u(c_.size_bytes));
  }
  return true;
}

// A V segment of block b sits at b*stride + kv_stride.  It can only collide
// with the K segment of the block nearest to that offset, i.e. the blocks
// floor(kv_stride / stride) and that + 1 further on (layout.rs:206-226).
bool KVCacheLayout::check_split_segments_disjoint(std::string* err) const {
  uint64_t max_distance = c_.num_blocks - 1;
  uint64_t nearest = c_.kv_stride_bytes / c_.block_stride_bytes;
  uint64_t next = nearest == UINT64_MAX ? nearest : nearest + 1;
  const uint64_t candidates[2] = {nearest, next};
  for (uint64_t distance : candidates) {
    if (distance == 0 || distance > max_distance) continue;
    uint64_t off = 0;
    if (!mul_ok(distance, c_.block_stride_bytes, &off)) return set(err, "memory layout overflow");
    uint64_t gap = c_.kv_stride_bytes > off ? c_.kv_stride_bytes - off : off - c_.kv_stride_bytes;
    if (gap < c_.segment_bytes) {
      return set(err, "kv_stride_bytes " + u(c_.kv_stride_bytes) + " overlaps blocks " +
                          u(distance) + " apart");
    }
  }
  return true;
}

bool KVCacheLayout::block_copies(uint64_t block_idx, BlockCopies* out, std::string* err) const {
  if (block_idx >= c_.num_blocks) {
    return set(err, "block " + u(block_idx) + " out of range (" + u(c_.num_blocks) + " blocks)");
  }
  uint64_t base = c_.data_ptr + block_idx * c_.block_stride_bytes;
  if (is_split()) {
    out->n = 2;
    out->k = {base, c_.segment_bytes};
    out->v = {base + c_.kv_stride_bytes, c_.segment_bytes};
  } else {
    out->n = 1;
    out->k = {base, block_bytes()};
    out->v = {0, 0};
  }
  return true;
}

bool KVCacheLayout::from_c(const pf_kv_layout& c, KVCacheLayout* out, std::string* err) {
  // Rebuild from the primary fields, then re-apply the derived ones through
  // the validating setters so a hand-filled struct cannot bypass the checks.
  uint64_t kv = c.split ? c.kv_stride_bytes : (c.segments > 1 ? c.segment_bytes : 0);
  KVCacheLayout l;
  if (!create(c.data_ptr, c.size_bytes, c.num_blocks, c.segment_bytes, kv, c.segments, &l, err)) {
    return false;
  }
  if ((c.split != 0) != l.is_split()) return set(err, "layout struct: split flag is inconsistent");
  if (c.block_stride_bytes != l.block_stride_bytes()) {
    if (!l.with_block_stride(c.block_stride_bytes, err)) return false;
  }
  if (c.padded_segment_bytes < c.segment_bytes) {
    return set(err, "layout struct: padded_segment_bytes < segment_bytes");
  }
  l.c_.padded_segment_bytes = c.padded_segment_bytes;
  *out = l;
  return true;
}

}  // namespace pf

extern "C" {

int pf_layout_new(uint64_t data_ptr, uint64_t size_bytes, uint64_t num_blocks,
                  uint64_t segment_bytes, uint64_t kv_stride_bytes, uint64_t segments,
                  pf_kv_layout* out) {
  PF_REQUIRE_PTR(out);
  pf::KVCacheLayout l;
  std::string err;
  if (!pf::KVCacheLayout::create(data_ptr, size_bytes, num_blocks, segment_bytes, kv_stride_bytes,
                                 segments, &l, &err)) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "%s", err.c_str());
  }
  *out = l.c();
  return PF_OK;
}

int pf_layout_with_block_stride(pf_kv_layout* layout, uint64_t stride) {
  PF_REQUIRE_PTR(layout);
  pf::KVCacheLayout l;
  std::string err;
  if (!pf::KVCacheLayout::from_c(*layout, &l, &err) || !l.with_block_stride(stride, &err)) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "%s", err.c_str());
  }
  *layout = l.c();
  return PF_OK;
}

int pf_layout_with_ssd_padding(pf_kv_layout* layout, uint64_t alignment) {
  PF_REQUIRE_PTR(layout);
  if (alignment == 0) return pf::fail(PF_ERR_INVALID_ARGUMENT, "alignment must be > 0");
  pf::KVCacheLayout l;
  std::string err;
  if (!pf::KVCacheLayout::from_c(*layout, &l, &err)) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "%s", err.c_str());
  }
  l.with_ssd_padding(alignment);
  *layout = l.c();
  return PF_OK;
}

int pf_layout_block_copies(const pf_kv_layout* layout, uint64_t block_idx, pf_block_copy out[2],
                           uint32_t* out_n) {
  PF_REQUIRE_PTR(layout);
  PF_REQUIRE_PTR(out);
  PF_REQUIRE_PTR(out_n);
  pf::KVCacheLayout l;
  std::string err;
  pf::BlockCopies bc;
  if (!pf::KVCacheLayout::from_c(*layout, &l, &err) || !l.block_copies(block_idx, &bc, &err)) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "%s", err.c_str());
  }
  *out_n = bc.n;
  out[0] = {bc.k.addr, bc.k.bytes};
  out[1] = {bc.v.addr, bc.v.bytes};
  return PF_OK;
}

uint64_t pf_layout_padded_block_bytes(const pf_kv_layout* layout) {
  return layout ? layout->padded_segment_bytes * layout->segments : 0;
}

uint64_t pf_layout_block_bytes(const pf_kv_layout* layout) {
  return layout ? layout->segment_bytes * layout->segments : 0;
}

}  // extern "C"
