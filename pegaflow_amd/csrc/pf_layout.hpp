// Per-layer KV cache layout: one affine address rule
//   addr = data_ptr + block_idx * block_stride + segment_idx * kv_stride
// validated once at construction.  Semantics and error messages follow
// pegaflow-core/src/layout.rs:13-286 of the reference.
#pragma once

#include <cstdint>
#include <string>

#include "../../include/pegahip.h"

namespace pf {

struct BlockCopy {
  uint64_t addr = 0;
  uint64_t bytes = 0;
};

// layout.rs:32-38: one contiguous range, or K and V apart.
struct BlockCopies {
  uint32_t n = 0;  // 1 = contiguous, 2 = split (k, v)
  BlockCopy k;     // the only range when n == 1
  BlockCopy v;
};

class KVCacheLayout {
 public:
  // layout.rs:73-130.  On failure returns false and fills *err.
  static bool create(uint64_t data_ptr, uint64_t size_bytes, uint64_t num_blocks,
                     uint64_t segment_bytes, uint64_t kv_stride_bytes, uint64_t segments,
                     KVCacheLayout* out, std::string* err);

  // layout.rs:140-153.
  bool with_block_stride(uint64_t stride, std::string* err);
  // layout.rs:157-160.
  void with_ssd_padding(uint64_t alignment);
  // layout.rs:231-255.
  bool block_copies(uint64_t block_idx, BlockCopies* out, std::string* err) const;

  uint64_t data_ptr() const { return c_.data_ptr; }
  uint64_t size_bytes() const { return c_.size_bytes; }
  uint64_t num_blocks() const { return c_.num_blocks; }
  uint64_t block_stride_bytes() const { return c_.block_stride_bytes; }
  bool is_split() const { return c_.split != 0; }
  uint64_t kv_stride_bytes() const { return c_.kv_stride_bytes; }
  uint64_t segments() const { return c_.segments; }
  uint64_t segment_bytes() const { return c_.segment_bytes; }
  uint64_t block_bytes() const { return c_.segment_bytes * c_.segments; }
  uint64_t padded_segment_bytes() const { return c_.padded_segment_bytes; }
  uint64_t padded_block_bytes() const { return c_.padded_segment_bytes * c_.segments; }
  // Bytes one fragment moves: a segment when split, else the whole block.
  uint64_t fragment_bytes() const { return is_split() ? c_.segment_bytes : block_bytes(); }
  uint32_t fragments_per_block() const { return is_split() ? 2u : 1u; }

  const pf_kv_layout& c() const { return c_; }
  // Re-validate a C struct that came across the ABI (guards against a caller
  // that filled it by hand).
  static bool from_c(const pf_kv_layout& c, KVCacheLayout* out, std::string* err);

 private:
  bool check_bounds(std::string* err) const;
  bool check_split_segments_disjoint(std::string* err) const;
  pf_kv_layout c_{};
};

}  // namespace pf
