// Layer-id space and page-first placement of an instance.  Follows
// pegaflow-core/src/instance.rs:46-269 (LayerTopology, PageLayout,
// build_page_layout) and :488-672 (seal_topology) of the reference.
#pragma once

#include <cstdint>
#include <map>
#include <set>
#include <string>
#include <vector>

#include "pf_layout.hpp"

namespace pf {

// instance.rs:78-98.
struct PageLayout {
  std::vector<size_t> layer_shard;       // shard (storage slot) owning each layer id
  std::vector<size_t> layer_offsets;     // byte offset of each layer in its shard's page
  std::vector<size_t> layer_bytes;       // padded block bytes of each layer
  std::vector<size_t> shard_page_sizes;  // page size per shard
};

// instance.rs:107-162.  `names` only feed the error messages.
bool build_page_layout(const std::vector<std::set<size_t>>& worker_layer_sets,
                       const std::vector<std::string>& names,
                       const std::vector<size_t>& padded_bytes, PageLayout* out, std::string* err);

// What one worker (GPU) registered; the subset of GpuContext that sealing reads
// (instance.rs:293-378).
struct WorkerRegistration {
  int device_id = 0;
  size_t tp_rank = 0;
  size_t pp_rank = 0;
  std::map<std::string, KVCacheLayout> kv_caches;
  std::map<std::string, uint32_t> layer_groups;  // absent = group 0
  uint32_t group_of_layer(const std::string& name) const {
    auto it = layer_groups.find(name);
    return it == layer_groups.end() ? 0 : it->second;
  }
};

// instance.rs:46-269.
class LayerTopology {
 public:
  // instance.rs:488-672: validate and seal the id space from every worker.
  static bool seal(const std::vector<const WorkerRegistration*>& workers, size_t tp_size,
                   bool page_first, const std::string& instance_id, size_t world_size,
                   LayerTopology* out, std::string* err);

  bool layer_id(const std::string& name, size_t* out, std::string* err) const;
  size_t num_layers() const { return name_to_id_.size(); }
  bool is_page_first() const { return has_page_layout_; }
  size_t total_slots() const;
  size_t num_groups() const { return group_layer_count_.size(); }
  uint32_t group_of_layer(size_t layer_id) const { return layer_group_[layer_id]; }
  bool group_total_slots(uint32_t group, size_t* out, std::string* err) const;
  bool shard_page_size(size_t shard, size_t* out) const;
  bool shard_layer_count(size_t shard, size_t* out) const;
  bool page_placement(size_t layer_id, size_t* offset, size_t* bytes) const;
  bool slot_index(size_t layer_id, size_t tp_rank, size_t* out, std::string* err) const;
  const std::vector<std::string>& names() const { return names_; }
  size_t tp_size() const { return tp_size_; }

 private:
  std::map<std::string, size_t> name_to_id_;
  std::vector<std::string> names_;  // sorted; index = layer id
  size_t tp_size_ = 1;
  std::vector<uint32_t> layer_group_;
  std::vector<size_t> group_layer_count_;
  std::vector<size_t> layer_group_rank_;
  bool has_page_layout_ = false;
  PageLayout page_layout_;
};

}  // namespace pf
