#include "pf_topology.hpp"

#include <algorithm>
#include <tuple>

namespace pf {

bool build_page_layout(const std::vector<std::set<size_t>>& worker_layer_sets,
                       const std::vector<std::string>& names,
                       const std::vector<size_t>& padded_bytes, PageLayout* out,
                       std::string* err) {
  constexpr size_t kNone = static_cast<size_t>(-1);
  const size_t n = names.size();
  // Distinct registered sets become shards, ordered by their smallest layer id
  // (stable, so equal keys keep first-seen order).
  std::vector<std::set<size_t>> shards;
  for (const auto& set : worker_layer_sets) {
    if (std::find(shards.begin(), shards.end(), set) == shards.end()) shards.push_back(set);
  }
  std::stable_sort(shards.begin(), shards.end(),
                   [](const std::set<size_t>& a, const std::set<size_t>& b) {
                     size_t ka = a.empty() ? static_cast<size_t>(-1) : *a.begin();
                     size_t kb = b.empty() ? static_cast<size_t>(-1) : *b.begin();
                     return ka < kb;
                   });
  PageLayout p;
  p.layer_shard.assign(n, kNone);
  for (size_t shard_id = 0; shard_id < shards.size(); ++shard_id) {
    for (size_t layer_id : shards[shard_id]) {
      if (layer_id >= n) {
        *err = "page-first layer id " + std::to_string(layer_id) + " out of range";
        return false;
      }
      if (p.layer_shard[layer_id] != kNone) {
        *err = "page-first layer " + names[layer_id] + " claimed by shards " +
               std::to_string(p.layer_shard[layer_id]) + " and " + std::to_string(shard_id) +
               ": registered layer sets must be identical (replica) or disjoint (split)";
        return false;
      }
      p.layer_shard[layer_id] = shard_id;
    }
  }
  for (size_t layer_id = 0; layer_id < n; ++layer_id) {
    if (p.layer_shard[layer_id] == kNone) {
      *err = "page-first layer " + names[layer_id] + " has no shard owner after sealing";
      return false;
    }
  }
  p.layer_offsets.assign(n, 0);
  p.layer_bytes.assign(n, 0);
  p.shard_page_sizes.assign(shards.size(), 0);
  for (size_t layer_id = 0; layer_id < n; ++layer_id) {
    size_t shard = p.layer_shard[layer_id];
    p.layer_offsets[layer_id] = p.shard_page_sizes[shard];
    p.layer_bytes[layer_id] = padded_bytes[layer_id];
    p.shard_page_sizes[shard] += padded_bytes[layer_id];
  }
  *out = std::move(p);
  return true;
}

bool LayerTopology::seal(const std::vector<const WorkerRegistration*>& workers, size_t tp_size,
                         bool page_first, const std::string& instance_id, size_t world_size,
                         LayerTopology* out, std::string* err) {
  // 1. Same name => same stored bytes on every device.
  using Geometry = std::tuple<uint64_t, bool, uint64_t>;  // segment_bytes, split, padded_block
  std::map<std::string, Geometry> geometry;
  for (const WorkerRegistration* w : workers) {
    for (const auto& kv : w->kv_caches) {
      const KVCacheLayout& l = kv.second;
      Geometry g(l.segment_bytes(), l.is_split(), l.padded_block_bytes());
      auto it = geometry.find(kv.first);
      if (it == geometry.end()) {
        geometry.emplace(kv.first, g);
      } else if (it->second != g) {
        *err = "layer " + kv.first + " registered with inconsistent geometry: segment_bytes=" +
               std::to_string(std::get<0>(it->second)) +
               " split=" + (std::get<1>(it->second) ? "true" : "false") +
               " padded_block_bytes=" + std::to_string(std::get<2>(it->second)) +
               " vs segment_bytes=" + std::to_string(l.segment_bytes()) +
               " split=" + (l.is_split() ? "true" : "false") +
               " padded_block_bytes=" + std::to_string(l.padded_block_bytes()) + " on device " +
               std::to_string(w->device_id);
        return false;
      }
    }
  }
  LayerTopology t;
  t.tp_size_ = tp_size;
  // std::map iterates keys in byte-wise sorted order: the id space.
  for (const auto& kv : geometry) {
    t.name_to_id_[kv.first] = t.names_.size();
    t.names_.push_back(kv.first);
  }
  const size_t n = t.names_.size();

  // 2. Storage groups: consistent across devices and dense 0..N.
  std::map<std::string, uint32_t> group_by_name;
  for (const WorkerRegistration* w : workers) {
    for (const auto& kv : w->kv_caches) {
      uint32_t g = w->group_of_layer(kv.first);
      auto it = group_by_name.find(kv.first);
      if (it == group_by_name.end()) {
        group_by_name.emplace(kv.first, g);
      } else if (it->second != g) {
        *err = "layer " + kv.first + " registered in storage group " +
               std::to_string(it->second) + " on one device but group " + std::to_string(g) +
               " on device " + std::to_string(w->device_id);
        return false;
      }
    }
  }
  uint32_t max_group = 0;
  std::set<uint32_t> distinct;
  for (const auto& kv : group_by_name) {
    max_group = std::max(max_group, kv.second);
    distinct.insert(kv.second);
  }
  const size_t num_groups = static_cast<size_t>(max_group) + 1;
  if (distinct.size() != num_groups) {
    *err = "storage groups must be dense 0.." + std::to_string(num_groups) +
           ": an unregistered group would never seal its blocks";
    return false;
  }
  t.layer_group_.assign(n, 0);
  t.layer_group_rank_.assign(n, 0);
  t.group_layer_count_.assign(num_groups, 0);
  for (size_t id = 0; id < n; ++id) {
    uint32_t g = group_by_name[t.names_[id]];
    t.layer_group_[id] = g;
    t.layer_group_rank_[id] = t.group_layer_count_[g];
    t.group_layer_count_[g] += 1;
  }
  if (page_first && num_groups > 1) {
    *err = "page-first storage does not support multiple storage groups (" +
           std::to_string(num_groups) + " registered)";
    return false;
  }

  // 3. Every (layer, tp_rank) needs an owner; replicas may only agree on pp_rank.
  struct Owner {
    bool set = false;
    int device = 0;
    size_t pp_rank = 0;
  };
  std::vector<Owner> owners(n * tp_size);
  for (const WorkerRegistration* w : workers) {
    for (const auto& kv : w->kv_caches) {
      size_t grid = t.name_to_id_[kv.first] * tp_size + w->tp_rank;
      if (w->tp_rank >= tp_size) {
        *err = "tp_rank " + std::to_string(w->tp_rank) + " out of range (tp_size " +
               std::to_string(tp_size) + ")";
        return false;
      }
      Owner& o = owners[grid];
      if (!o.set) {
        o = {true, w->device_id, w->pp_rank};
      } else if (o.pp_rank != w->pp_rank) {
        *err = "layer " + kv.first + " claimed by different pipeline stages: device=" +
               std::to_string(o.device) + " pp_rank=" + std::to_string(o.pp_rank) +
               "; device=" + std::to_string(w->device_id) +
               " pp_rank=" + std::to_string(w->pp_rank) +
               " tp_rank=" + std::to_string(w->tp_rank);
        return false;
      }
    }
  }
  for (size_t i = 0; i < owners.size(); ++i) {
    if (!owners[i].set) {
      *err = "instance " + instance_id + " has incomplete KV registration: layer " +
             t.names_[i / tp_size] + " has no owner for tp_rank " + std::to_string(i % tp_size) +
             " after all " + std::to_string(world_size) + " workers registered";
      return false;
    }
  }

  // 4. Page-first: shards and per-shard offsets.
  if (page_first) {
    std::vector<std::set<size_t>> sets;
    for (const WorkerRegistration* w : workers) {
      std::set<size_t> s;
      for (const auto& kv : w->kv_caches) s.insert(t.name_to_id_[kv.first]);
      sets.push_back(std::move(s));
    }
    std::vector<size_t> padded(n);
    for (size_t id = 0; id < n; ++id) padded[id] = std::get<2>(geometry[t.names_[id]]);
    if (!build_page_layout(sets, t.names_, padded, &t.page_layout_, err)) return false;
    t.has_page_layout_ = true;
  }
  *out = std::move(t);
  return true;
}

bool LayerTopology::layer_id(const std::string& name, size_t* out, std::string* err) const {
  auto it = name_to_id_.find(name);
  if (it == name_to_id_.end()) {
    if (err) *err = "layer " + name + " is not registered";
    return false;
  }
  *out = it->second;
  return true;
}

size_t LayerTopology::total_slots() const {
  return has_page_layout_ ? page_layout_.shard_page_sizes.size() : num_layers() * tp_size_;
}

bool LayerTopology::group_total_slots(uint32_t group, size_t* out, std::string* err) const {
  if (group >= num_groups()) {
    if (err) {
      *err = "storage group " + std::to_string(group) + " out of range (" +
             std::to_string(num_groups()) + " groups)";
    }
    return false;
  }
  *out = has_page_layout_ ? page_layout_.shard_page_sizes.size()
                          : group_layer_count_[group] * tp_size_;
  return true;
}

bool LayerTopology::shard_page_size(size_t shard, size_t* out) const {
  if (!has_page_layout_ || shard >= page_layout_.shard_page_sizes.size()) return false;
  *out = page_layout_.shard_page_sizes[shard];
  return true;
}

bool LayerTopology::shard_layer_count(size_t shard, size_t* out) const {
  if (!has_page_layout_) return false;
  *out = static_cast<size_t>(
      std::count(page_layout_.layer_shard.begin(), page_layout_.layer_shard.end(), shard));
  return true;
}

bool LayerTopology::page_placement(size_t layer_id, size_t* offset, size_t* bytes) const {
  if (!has_page_layout_ || layer_id >= num_layers()) return false;
  *offset = page_layout_.layer_offsets[layer_id];
  *bytes = page_layout_.layer_bytes[layer_id];
  return true;
}

bool LayerTopology::slot_index(size_t layer_id, size_t tp_rank, size_t* out,
                               std::string* err) const {
  if (layer_id >= num_layers()) {
    if (err) {
      *err = "layer_id " + std::to_string(layer_id) + " out of range (" +
             std::to_string(num_layers()) + " layers)";
    }
    return false;
  }
  if (tp_rank >= tp_size_) {
    if (err) {
      *err = "tp_rank " + std::to_string(tp_rank) + " out of range (tp_size " +
             std::to_string(tp_size_) + ")";
    }
    return false;
  }
  *out = has_page_layout_ ? page_layout_.layer_shard[layer_id]
                          : layer_group_rank_[layer_id] * tp_size_ + tp_rank;
  return true;
}

}  // namespace pf
