// C ABI of the host-only pieces: offset allocator, pinned pool, NUMA helpers,
// layer topology.
#include <cstring>
#include <memory>

#include "pf_alloc.hpp"
#include "pf_common.hpp"
#include "pf_numa.hpp"
#include "pf_pool.hpp"
#include "pf_topology.hpp"

namespace {

struct AllocatorHandle {
  std::unique_ptr<pf::ScaledOffsetAllocator> a;
};

struct PoolHandle {
  std::unique_ptr<pf::PinnedAllocator> a;
};

int copy_string(const std::string& s, char* buf, size_t cap) {
  if (!buf || cap == 0) return pf::fail(PF_ERR_BUFFER_TOO_SMALL, "no output buffer");
  if (s.size() + 1 > cap) {
    return pf::fail(PF_ERR_BUFFER_TOO_SMALL, "need %zu bytes, have %zu", s.size() + 1, cap);
  }
  std::memcpy(buf, s.c_str(), s.size() + 1);
  return PF_OK;
}

}  // namespace

extern "C" {

// ---- allocator ------------------------------------------------------------

int pf_allocator_create(uint64_t total_bytes, uint64_t unit_size, uint32_t max_allocs,
                        pf_allocator_t* out) {
  PF_REQUIRE_PTR(out);
  pf::AllocatorError err;
  auto* a = pf::ScaledOffsetAllocator::create(total_bytes, unit_size, max_allocs, &err);
  if (!a) return pf::fail(PF_ERR_INVALID_ARGUMENT, "%s", err.to_string().c_str());
  auto* h = new AllocatorHandle();
  h->a.reset(a);
  *out = reinterpret_cast<pf_allocator_t>(h);
  return PF_OK;
}

int pf_allocator_destroy(pf_allocator_t a) {
  delete reinterpret_cast<AllocatorHandle*>(a);
  return PF_OK;
}

int pf_allocator_allocate(pf_allocator_t a, uint64_t size_bytes, pf_alloc_region* out) {
  PF_REQUIRE_PTR(a);
  PF_REQUIRE_PTR(out);
  out->offset_bytes = out->size_bytes = out->token = 0;
  pf::ScaledOffsetAllocator::Allocation al;
  pf::AllocatorError err;
  int rc = reinterpret_cast<AllocatorHandle*>(a)->a->allocate(size_bytes, &al, &err);
  if (rc < 0) return pf::fail(PF_ERR_INVALID_ARGUMENT, "%s", err.to_string().c_str());
  if (rc == 0) return PF_OK;
  out->offset_bytes = al.offset_bytes;
  out->size_bytes = al.size_bytes;
  out->token = (static_cast<uint64_t>(al.raw.metadata) << 32) | al.raw.offset;
  return PF_OK;
}

int pf_allocator_free(pf_allocator_t a, const pf_alloc_region* region) {
  PF_REQUIRE_PTR(a);
  PF_REQUIRE_PTR(region);
  if (region->size_bytes == 0) return PF_OK;
  pf::ScaledOffsetAllocator::Allocation al;
  al.offset_bytes = region->offset_bytes;
  al.size_bytes = region->size_bytes;
  al.raw.offset = static_cast<uint32_t>(region->token & 0xFFFFFFFFull);
  al.raw.metadata = static_cast<uint32_t>(region->token >> 32);
  reinterpret_cast<AllocatorHandle*>(a)->a->free(al);
  return PF_OK;
}

int pf_allocator_report(pf_allocator_t a, uint64_t* out_total_bytes, uint64_t* out_free_bytes,
                        uint64_t* out_largest_free_bytes, uint64_t* out_total_units) {
  PF_REQUIRE_PTR(a);
  auto& al = *reinterpret_cast<AllocatorHandle*>(a)->a;
  auto r = al.storage_report();
  if (out_total_bytes) *out_total_bytes = al.total_bytes();
  if (out_free_bytes) *out_free_bytes = r.total_free_bytes;
  if (out_largest_free_bytes) *out_largest_free_bytes = r.largest_free_allocation_bytes;
  if (out_total_units) *out_total_units = al.total_units();
  return PF_OK;
}

// ---- pool -------------------------------------------------------------------

uint64_t pf_pool_compute_unit_size(uint64_t pool_size, uint64_t unit_size_hint) {
  return pf::PinnedMemoryPool::compute_unit_size(pool_size, unit_size_hint);
}

int pf_pool_create(const pf_pool_config* cfg, pf_pool_t* out) {
  PF_REQUIRE_PTR(cfg);
  PF_REQUIRE_PTR(out);
  std::string err;
  int status = PF_ERR_STORAGE;
  std::unique_ptr<pf::PinnedAllocator> a;
  if (cfg->n_numa_nodes == 0) {
    a = pf::PinnedAllocator::new_global(cfg->capacity, cfg->num_shards, cfg->use_hugepages != 0,
                                        cfg->ssd_enabled != 0, cfg->unit_size_hint, &err, &status);
  } else {
    PF_REQUIRE_PTR(cfg->numa_nodes);
    std::vector<pf::NumaNode> nodes;
    for (uint32_t i = 0; i < cfg->n_numa_nodes; ++i) {
      nodes.push_back(pf::NumaNode::from_int(cfg->numa_nodes[i]));
    }
    a = pf::PinnedAllocator::new_numa(cfg->capacity, nodes, cfg->num_shards,
                                      cfg->use_hugepages != 0, cfg->ssd_enabled != 0,
                                      cfg->unit_size_hint, &err, &status);
  }
  if (!a) {
    pf::last_error() = err;
    return status == PF_OK ? PF_ERR_STORAGE : status;
  }
  auto* h = new PoolHandle();
  h->a = std::move(a);
  *out = reinterpret_cast<pf_pool_t>(h);
  return PF_OK;
}

int pf_pool_destroy(pf_pool_t p) {
  delete reinterpret_cast<PoolHandle*>(p);
  return PF_OK;
}

int pf_pool_allocate(pf_pool_t p, uint64_t size, int numa_node, pf_allocation* out) {
  PF_REQUIRE_PTR(p);
  PF_REQUIRE_PTR(out);
  out->handle = 0;
  out->host = nullptr;
  out->device = 0;
  out->size = 0;
  if (size == 0) return pf::fail(PF_ERR_INVALID_ARGUMENT, "allocation size must be non-zero");
  auto a = reinterpret_cast<PoolHandle*>(p)->a->allocate(size, pf::NumaNode::from_int(numa_node));
  if (!a) return PF_OK;  // exhausted: the caller may evict and retry
  out->host = a->as_ptr();
  out->device = reinterpret_cast<uint64_t>(a->mapped_ptr().device);
  out->size = a->size_bytes();
  out->handle = reinterpret_cast<uint64_t>(new std::shared_ptr<pf::PinnedAllocation>(std::move(a)));
  return PF_OK;
}

int pf_pool_free(pf_allocation* a) {
  PF_REQUIRE_PTR(a);
  if (a->handle == 0) return PF_OK;
  delete reinterpret_cast<std::shared_ptr<pf::PinnedAllocation>*>(a->handle);
  a->handle = 0;
  a->host = nullptr;
  a->device = 0;
  a->size = 0;
  return PF_OK;
}

int pf_pool_usage(pf_pool_t p, uint64_t* out_used, uint64_t* out_total) {
  PF_REQUIRE_PTR(p);
  PF_REQUIRE_PTR(out_used);
  PF_REQUIRE_PTR(out_total);
  reinterpret_cast<PoolHandle*>(p)->a->usage(out_used, out_total);
  return PF_OK;
}

int pf_pool_largest_free(pf_pool_t p, int numa_node, uint64_t* out_bytes) {
  PF_REQUIRE_PTR(p);
  PF_REQUIRE_PTR(out_bytes);
  *out_bytes = reinterpret_cast<PoolHandle*>(p)->a->largest_free_allocation_for_node(
      pf::NumaNode::from_int(numa_node));
  return PF_OK;
}

int pf_pool_is_numa(pf_pool_t p) { return p && reinterpret_cast<PoolHandle*>(p)->a->is_numa(); }

// ---- NUMA -------------------------------------------------------------------

int pf_numa_format_cpu_list(const uint64_t* cpus, uint64_t n, char* buf, size_t cap) {
  std::vector<size_t> v;
  for (uint64_t i = 0; i < n; ++i) v.push_back(static_cast<size_t>(cpus[i]));
  return copy_string(pf::format_cpu_list(v), buf, cap);
}

int pf_numa_parse_cpulist(const char* cpulist, uint64_t* out, uint64_t cap, uint64_t* out_n) {
  PF_REQUIRE_PTR(cpulist);
  PF_REQUIRE_PTR(out_n);
  std::vector<size_t> v;
  std::string err;
  if (!pf::parse_cpulist(cpulist, &v, &err)) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "%s", err.c_str());
  }
  *out_n = v.size();
  if (v.size() > cap) return pf::fail(PF_ERR_BUFFER_TOO_SMALL, "cpu list holds %zu ids", v.size());
  for (size_t i = 0; i < v.size(); ++i) out[i] = v[i];
  return PF_OK;
}

int pf_numa_pin_thread(int numa_node) {
  std::string err;
  if (!pf::pin_thread_to_numa_node(pf::NumaNode::from_int(numa_node), &err)) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "%s", err.c_str());
  }
  return PF_OK;
}

int pf_numa_node_count(void) {
  std::map<uint32_t, std::vector<size_t>> topo;
  std::string err;
  if (!pf::read_cpu_topology_from_sysfs(&topo, &err)) return 1;
  return static_cast<int>(topo.size());
}

int pf_numa_query_pages(const void* const* addrs, uint64_t n, int* out_nodes) {
  if (n == 0) return PF_OK;
  PF_REQUIRE_PTR(addrs);
  PF_REQUIRE_PTR(out_nodes);
  std::vector<const void*> v(addrs, addrs + n);
  std::vector<pf::NumaNode> nodes = pf::query_pages_numa(v);
  for (uint64_t i = 0; i < n; ++i) {
    out_nodes[i] = i < nodes.size() && nodes[i].is_valid() ? static_cast<int>(nodes[i].id) : -1;
  }
  return PF_OK;
}

int pf_numa_node_of_pci(const char* bdf, const char* sysfs_root) {
  return pf::numa_node_of_pci_device(bdf, sysfs_root);
}

// ---- topology ---------------------------------------------------------------

int pf_build_page_layout(const uint64_t* set_ids, const uint64_t* set_off, uint64_t n_sets,
                         uint64_t n_layers, const uint64_t* padded_bytes,
                         uint64_t* out_layer_shard, uint64_t* out_layer_offsets,
                         uint64_t* out_layer_bytes, uint64_t* out_shard_page_sizes,
                         uint64_t* out_n_shards) {
  PF_REQUIRE_PTR(set_off);
  PF_REQUIRE_PTR(out_n_shards);
  std::vector<std::set<size_t>> sets(n_sets);
  for (uint64_t w = 0; w < n_sets; ++w) {
    for (uint64_t i = set_off[w]; i < set_off[w + 1]; ++i) sets[w].insert(set_ids[i]);
  }
  std::vector<std::string> names;
  std::vector<size_t> padded;
  for (uint64_t l = 0; l < n_layers; ++l) {
    names.push_back("#" + std::to_string(l));
    padded.push_back(padded_bytes[l]);
  }
  pf::PageLayout p;
  std::string err;
  if (!pf::build_page_layout(sets, names, padded, &p, &err)) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "%s", err.c_str());
  }
  for (uint64_t l = 0; l < n_layers; ++l) {
    out_layer_shard[l] = p.layer_shard[l];
    out_layer_offsets[l] = p.layer_offsets[l];
    out_layer_bytes[l] = p.layer_bytes[l];
  }
  for (size_t s = 0; s < p.shard_page_sizes.size(); ++s) out_shard_page_sizes[s] = p.shard_page_sizes[s];
  *out_n_shards = p.shard_page_sizes.size();
  return PF_OK;
}

int pf_topology_seal(const pf_worker_layers* workers, uint32_t n_workers, uint32_t tp_size,
                     int page_first, pf_topology_t* out) {
  PF_REQUIRE_PTR(workers);
  PF_REQUIRE_PTR(out);
  if (tp_size == 0 || n_workers == 0) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "tp_size and world_size must be > 0");
  }
  std::vector<pf::WorkerRegistration> regs(n_workers);
  for (uint32_t w = 0; w < n_workers; ++w) {
    const pf_worker_layers& in = workers[w];
    regs[w].device_id = in.device_id;
    regs[w].tp_rank = in.tp_rank;
    regs[w].pp_rank = in.pp_rank;
    if (in.n_layers == 0) {
      return pf::fail(PF_ERR_INVALID_ARGUMENT, "device %d registered no KV cache layers",
                      in.device_id);
    }
    for (uint32_t i = 0; i < in.n_layers; ++i) {
      pf::KVCacheLayout l;
      std::string err;
      if (!pf::KVCacheLayout::from_c(in.layouts[i], &l, &err)) {
        return pf::fail(PF_ERR_INVALID_ARGUMENT, "layer %s: %s", in.layer_names[i], err.c_str());
      }
      if (!regs[w].kv_caches.emplace(in.layer_names[i], l).second) {
        return pf::fail(PF_ERR_INVALID_ARGUMENT, "duplicate layer name in registration batch: %s",
                        in.layer_names[i]);
      }
      if (in.group_ids) regs[w].layer_groups[in.layer_names[i]] = in.group_ids[i];
    }
  }
  std::vector<const pf::WorkerRegistration*> ptrs;
  for (auto& r : regs) ptrs.push_back(&r);
  auto topo = std::make_unique<pf::LayerTopology>();
  std::string err;
  if (!pf::LayerTopology::seal(ptrs, tp_size, page_first != 0, "instance", n_workers, topo.get(),
                               &err)) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "%s", err.c_str());
  }
  *out = reinterpret_cast<pf_topology_t>(topo.release());
  return PF_OK;
}

int pf_topology_destroy(pf_topology_t t) {
  delete reinterpret_cast<pf::LayerTopology*>(t);
  return PF_OK;
}

uint64_t pf_topology_num_layers(pf_topology_t t) {
  return t ? reinterpret_cast<pf::LayerTopology*>(t)->num_layers() : 0;
}

uint64_t pf_topology_total_slots(pf_topology_t t) {
  return t ? reinterpret_cast<pf::LayerTopology*>(t)->total_slots() : 0;
}

uint64_t pf_topology_num_groups(pf_topology_t t) {
  return t ? reinterpret_cast<pf::LayerTopology*>(t)->num_groups() : 0;
}

int pf_topology_group_of_layer(pf_topology_t t, uint64_t layer_id, uint32_t* out_group) {
  PF_REQUIRE_PTR(t);
  PF_REQUIRE_PTR(out_group);
  auto* topo = reinterpret_cast<pf::LayerTopology*>(t);
  if (layer_id >= topo->num_layers()) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "layer_id %llu out of range (%zu layers)",
                    static_cast<unsigned long long>(layer_id), topo->num_layers());
  }
  *out_group = topo->group_of_layer(layer_id);
  return PF_OK;
}

int pf_topology_group_total_slots(pf_topology_t t, uint32_t group, uint64_t* out_slots) {
  PF_REQUIRE_PTR(t);
  PF_REQUIRE_PTR(out_slots);
  size_t n = 0;
  std::string err;
  if (!reinterpret_cast<pf::LayerTopology*>(t)->group_total_slots(group, &n, &err)) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "%s", err.c_str());
  }
  *out_slots = n;
  return PF_OK;
}

int pf_topology_is_page_first(pf_topology_t t) {
  return t && reinterpret_cast<pf::LayerTopology*>(t)->is_page_first();
}

int pf_topology_layer_id(pf_topology_t t, const char* layer_name, uint64_t* out_id) {
  PF_REQUIRE_PTR(t);
  PF_REQUIRE_PTR(layer_name);
  PF_REQUIRE_PTR(out_id);
  size_t id = 0;
  std::string err;
  if (!reinterpret_cast<pf::LayerTopology*>(t)->layer_id(layer_name, &id, &err)) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "%s", err.c_str());
  }
  *out_id = id;
  return PF_OK;
}

int pf_topology_slot_index(pf_topology_t t, uint64_t layer_id, uint64_t tp_rank, uint64_t* out) {
  PF_REQUIRE_PTR(t);
  PF_REQUIRE_PTR(out);
  size_t slot = 0;
  std::string err;
  if (!reinterpret_cast<pf::LayerTopology*>(t)->slot_index(layer_id, tp_rank, &slot, &err)) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "%s", err.c_str());
  }
  *out = slot;
  return PF_OK;
}

int pf_topology_page_placement(pf_topology_t t, uint64_t layer_id, uint64_t* out_offset,
                               uint64_t* out_bytes) {
  PF_REQUIRE_PTR(t);
  size_t off = 0, bytes = 0;
  if (!reinterpret_cast<pf::LayerTopology*>(t)->page_placement(layer_id, &off, &bytes)) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "layer %llu has no page placement",
                    static_cast<unsigned long long>(layer_id));
  }
  if (out_offset) *out_offset = off;
  if (out_bytes) *out_bytes = bytes;
  return PF_OK;
}

int pf_topology_shard_page_size(pf_topology_t t, uint64_t shard, uint64_t* out) {
  PF_REQUIRE_PTR(t);
  PF_REQUIRE_PTR(out);
  size_t v = 0;
  if (!reinterpret_cast<pf::LayerTopology*>(t)->shard_page_size(shard, &v)) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "shard %llu has no page",
                    static_cast<unsigned long long>(shard));
  }
  *out = v;
  return PF_OK;
}

int pf_topology_shard_layer_count(pf_topology_t t, uint64_t shard, uint64_t* out) {
  PF_REQUIRE_PTR(t);
  PF_REQUIRE_PTR(out);
  size_t v = 0;
  if (!reinterpret_cast<pf::LayerTopology*>(t)->shard_layer_count(shard, &v)) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "topology is not page-first");
  }
  *out = v;
  return PF_OK;
}

}  // extern "C"
