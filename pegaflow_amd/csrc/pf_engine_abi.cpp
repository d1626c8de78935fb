// C ABI of the worker pool, the load-completion flag and the engine.
#include <chrono>
#include <cstring>

#include "pf_common.hpp"
#include "pf_engine.hpp"
#include "pf_sync_state.hpp"
#include "pf_worker.hpp"

namespace {

struct TaskHandle {
  std::future<pf::TaskResult> fut;
  bool settled = false;
  pf::TaskResult result;
  // Host-block storage of a task submitted through the raw worker ABI.
  std::vector<std::shared_ptr<pf::RawBlock>> blocks;
};

// A segment that points at caller-owned pinned memory (no pool allocation).
class BorrowedBlocks {
 public:
  // Rebuild LayerTransferData from the C structs.  The RawBlocks wrap the
  // caller's pointers without owning them.
  static bool build(const pf_layer_transfer* layers, uint64_t n_layers,
                    std::vector<pf::LayerTransferData>* out,
                    std::vector<std::shared_ptr<pf::RawBlock>>* keep, std::string* err);
};

}  // namespace

namespace pf {

// A pinned allocation shell over memory the pool does not own: lets a Segment
// carry caller-provided host/device addresses through the worker.
class ExternalAllocation {
 public:
  static std::shared_ptr<PinnedAllocation> wrap(uint8_t* host, uint8_t* device, uint64_t size) {
    ScaledOffsetAllocator::Allocation a;
    a.offset_bytes = 0;
    a.size_bytes = size;
    return std::make_shared<PinnedAllocation>(a, host, device, nullptr);
  }
};

}  // namespace pf

namespace {

bool BorrowedBlocks::build(const pf_layer_transfer* layers, uint64_t n_layers,
                           std::vector<pf::LayerTransferData>* out,
                           std::vector<std::shared_ptr<pf::RawBlock>>* keep, std::string* err) {
  for (uint64_t li = 0; li < n_layers; ++li) {
    const pf_layer_transfer& in = layers[li];
    pf::LayerTransferData ltd;
    ltd.layer_name = in.layer_name ? in.layer_name : ("#" + std::to_string(li));
    std::string cause;
    if (!pf::KVCacheLayout::from_c(in.layout, &ltd.layout, &cause)) {
      *err = "layer " + ltd.layer_name + ": " + cause;
      return false;
    }
    for (uint64_t bi = 0; bi < in.n_blocks; ++bi) {
      const pf_host_block& hb = in.blocks[bi];
      if (hb.num_segments == 0 || hb.num_segments > 2 || !hb.seg_host[0]) {
        *err = "layer " + ltd.layer_name + ": host block has no segment 0";
        return false;
      }
      std::vector<pf::Segment> segs;
      for (uint32_t s = 0; s < hb.num_segments; ++s) {
        // The segment must cover what the copy will touch from it.
        uint64_t size = hb.seg_size[s];
        if (size == 0) {
          size = hb.host_offset + ltd.layout.fragment_bytes() *
                                      (hb.num_segments == 1 && ltd.layout.is_split() ? 2 : 1);
        }
        auto alloc = pf::ExternalAllocation::wrap(static_cast<uint8_t*>(hb.seg_host[s]),
                                                  reinterpret_cast<uint8_t*>(hb.seg_device[s]), size);
        pf::Segment seg;
        if (!pf::Segment::create(static_cast<uint8_t*>(hb.seg_host[s]), size, alloc, &seg)) {
          *err = "layer " + ltd.layer_name + ": bad host segment";
          return false;
        }
        segs.push_back(std::move(seg));
      }
      auto raw = std::make_shared<pf::RawBlock>(std::move(segs));
      keep->push_back(raw);
      pf::TransferBlock tb;
      tb.block_idx = in.block_idx[bi];
      tb.block.raw = raw.get();
      tb.block.keep = raw;
      tb.block.offset = hb.host_offset;
      ltd.blocks.push_back(std::move(tb));
    }
    out->push_back(std::move(ltd));
  }
  return true;
}

}  // namespace

extern "C" {

// ---- LoadState --------------------------------------------------------------

int pf_load_state_create(pf_load_state_t* out) {
  PF_REQUIRE_PTR(out);
  std::string err;
  auto s = pf::LoadState::create(&err);
  if (!s) return pf::fail(PF_ERR_STORAGE, "%s", err.c_str());
  *out = reinterpret_cast<pf_load_state_t>(s.release());
  return PF_OK;
}

int pf_load_state_attach(const char* shm_name, pf_load_state_t* out) {
  PF_REQUIRE_PTR(shm_name);
  PF_REQUIRE_PTR(out);
  std::string err;
  auto s = pf::LoadState::attach(shm_name, &err);
  if (!s) return pf::fail(PF_ERR_STORAGE, "%s", err.c_str());
  *out = reinterpret_cast<pf_load_state_t>(s.release());
  return PF_OK;
}

int pf_load_state_destroy(pf_load_state_t s) {
  delete reinterpret_cast<pf::LoadState*>(s);
  return PF_OK;
}

const char* pf_load_state_name(pf_load_state_t s) {
  return s ? reinterpret_cast<pf::LoadState*>(s)->shm_name().c_str() : "";
}

int64_t pf_load_state_get(pf_load_state_t s) {
  return s ? reinterpret_cast<pf::LoadState*>(s)->get() : pf::kLoadStateError;
}

int pf_load_state_set(pf_load_state_t s, int64_t state) {
  PF_REQUIRE_PTR(s);
  auto* ls = reinterpret_cast<pf::LoadState*>(s);
  if (state == pf::kLoadStateSuccess) {
    ls->set_completed();
  } else if (state == pf::kLoadStateError) {
    ls->set_error();
  } else {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "LoadState can only be set to 1 or -1");
  }
  return PF_OK;
}

// ---- worker pool --------------------------------------------------------------

int pf_worker_pool_spawn_ex(const pf_worker_pool_config* cfg, pf_worker_pool_t* out) {
  PF_REQUIRE_PTR(cfg);
  PF_REQUIRE_PTR(out);
  if (cfg->device_id < 0) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "device_id %d must be >= 0", cfg->device_id);
  }
  if (cfg->transfer_mode != PF_MODE_DIRECT && cfg->transfer_mode != PF_MODE_KERNEL &&
      cfg->transfer_mode != PF_MODE_ZEROCOPY) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "unknown transfer mode %d", cfg->transfer_mode);
  }
  pf::WorkerPoolOptions options;
  options.use_descriptor_backends = cfg->use_descriptor_backends != 0;
  options.staging_slot_bytes = cfg->staging_slot_bytes;
  options.auto_staged_min_bytes = cfg->auto_staged_min_bytes;
  options.lazy_staging = cfg->lazy_staging != 0;
  options.side_copy_streams = cfg->side_copy_streams != 0;
  std::string err;
  int status = PF_ERR_DEVICE_INIT;
  auto pool = pf::GpuWorkerPool::spawn(cfg->device_id, pf::NumaNode::from_int(cfg->numa_node),
                                       static_cast<pf::TransferMode>(cfg->transfer_mode), options,
                                       &err, &status);
  if (!pool) {
    pf::last_error() = err;
    return status;
  }
  *out = reinterpret_cast<pf_worker_pool_t>(pool.release());
  return PF_OK;
}

int pf_worker_pool_spawn(int device_id, int numa_node, int transfer_mode,
                         int use_descriptor_backends, pf_worker_pool_t* out) {
  pf_worker_pool_config cfg;
  std::memset(&cfg, 0, sizeof(cfg));
  cfg.device_id = device_id;
  cfg.numa_node = numa_node;
  cfg.transfer_mode = transfer_mode;
  cfg.use_descriptor_backends = use_descriptor_backends != 0 ? 1u : 0u;
  return pf_worker_pool_spawn_ex(&cfg, out);
}

uint64_t pf_worker_pool_staging_bytes(pf_worker_pool_t p) {
  return p ? reinterpret_cast<pf::GpuWorkerPool*>(p)->staging_bytes() : 0;
}

uint64_t pf_worker_pool_queue_clashes(pf_worker_pool_t p) {
  return p ? reinterpret_cast<pf::GpuWorkerPool*>(p)->queue_clashes() : 0;
}

int pf_worker_stream_report(int device, uint64_t* out_streams, uint64_t* out_clashing_pairs,
                            uint64_t* out_skipped) {
  PF_REQUIRE_PTR(out_streams);
  PF_REQUIRE_PTR(out_clashing_pairs);
  PF_REQUIRE_PTR(out_skipped);
  size_t streams = 0, pairs = 0, skipped = 0;
  int st = pf::worker_stream_report(device, &streams, &pairs, &skipped);
  *out_streams = streams;
  *out_clashing_pairs = pairs;
  *out_skipped = skipped;
  return st;
}

int pf_worker_pool_destroy(pf_worker_pool_t p) {
  delete reinterpret_cast<pf::GpuWorkerPool*>(p);
  return PF_OK;
}

static void fill_task_result(const pf::TaskResult& r, pf_task_result* out) {
  std::memset(out, 0, sizeof(*out));
  out->status = r.status;
  out->done = 1;
  out->bytes = r.bytes;
  out->elapsed_ms = r.elapsed_ms;
  out->paths = r.paths;
  out->staged_groups = r.staged_groups;
  out->zero_copy_launches = r.zero_copy_launches;
  out->link_copies = r.link_copies;
  out->resolve_ms = r.resolve_ms;
  out->queue_ms = r.queue_ms;
  out->convert_ms = r.convert_ms;
  out->plan_ms = r.plan_ms;
  out->staging_alloc_ms = r.staging_alloc_ms;
  out->enqueue_ms = r.enqueue_ms;
  out->sync_ms = r.sync_ms;
  out->device_first_ms = r.device_first_ms;
  out->device_ms = r.device_ms;
}

static int submit(pf_worker_pool_t p, const pf_layer_transfer* layers, uint64_t n_layers,
                  const char* shm, bool load, pf_task_t* out_task) {
  PF_REQUIRE_PTR(p);
  PF_REQUIRE_PTR(out_task);
  if (n_layers != 0) PF_REQUIRE_PTR(layers);
  auto h = std::make_unique<TaskHandle>();
  std::vector<pf::LayerTransferData> ltds;
  std::string err;
  if (!BorrowedBlocks::build(layers, n_layers, &ltds, &h->blocks, &err)) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "%s", err.c_str());
  }
  auto* pool = reinterpret_cast<pf::GpuWorkerPool*>(p);
  if (load) {
    pf::LoadCompletion c;
    if (shm) c.load_state_shm = shm;
    h->fut = pool->submit_load(std::move(ltds), std::move(c));
  } else {
    h->fut = pool->batch_save(std::move(ltds));
  }
  *out_task = reinterpret_cast<pf_task_t>(h.release());
  return PF_OK;
}

int pf_worker_submit_load(pf_worker_pool_t p, const pf_layer_transfer* layers, uint64_t n_layers,
                          const char* load_state_shm, pf_task_t* out_task) {
  return submit(p, layers, n_layers, load_state_shm, true, out_task);
}

int pf_worker_submit_save(pf_worker_pool_t p, const pf_layer_transfer* layers, uint64_t n_layers,
                          pf_task_t* out_task) {
  return submit(p, layers, n_layers, nullptr, false, out_task);
}

int pf_task_wait(pf_task_t t, int timeout_ms, pf_task_result* out) {
  PF_REQUIRE_PTR(t);
  auto* h = reinterpret_cast<TaskHandle*>(t);
  if (!h->settled) {
    if (timeout_ms >= 0 &&
        h->fut.wait_for(std::chrono::milliseconds(timeout_ms)) != std::future_status::ready) {
      if (out) {
        std::memset(out, 0, sizeof(*out));
      }
      return PF_OK;
    }
    if (timeout_ms < 0) {
      // Short tasks settle within tens of microseconds: poll for that long
      // before parking the thread on the future (whose wake-up costs as much).
      const auto spin_until = std::chrono::steady_clock::now() + std::chrono::microseconds(100);
      while (h->fut.wait_for(std::chrono::seconds(0)) != std::future_status::ready &&
             std::chrono::steady_clock::now() < spin_until) {
      }
    }
    h->result = h->fut.get();
    h->settled = true;
  }
  if (out) fill_task_result(h->result, out);
  if (h->result.status != PF_OK) pf::last_error() = h->result.message;
  return h->result.status;
}

int pf_task_destroy(pf_task_t t) {
  auto* h = reinterpret_cast<TaskHandle*>(t);
  if (h && !h->settled && h->fut.valid()) h->fut.wait();  // buffers must outlive the copy
  delete h;
  return PF_OK;
}

// ---- engine -------------------------------------------------------------------

int pf_engine_create(const pf_engine_config* cfg, pf_engine_t* out) {
  PF_REQUIRE_PTR(cfg);
  PF_REQUIRE_PTR(out);
  pf::EngineConfig c;
  c.pool_size = cfg->pool_size;
  c.use_hugepages = cfg->use_hugepages != 0;
  c.numa_aware = cfg->numa_aware != 0;
  c.pool_shards = cfg->pool_shards ? cfg->pool_shards : 1;
  c.blockwise_alloc = cfg->blockwise_alloc != 0;
  c.ssd_enabled = cfg->ssd_enabled != 0;
  c.use_descriptor_backends = cfg->use_descriptor_backends != 0;
  c.unit_size_hint = cfg->unit_size_hint;
  if (cfg->lease_ttl_ms != 0) c.lease_ttl_ms = cfg->lease_ttl_ms;
  c.auto_staged_min_bytes = cfg->auto_staged_min_bytes;
  c.staging_slot_bytes = cfg->staging_slot_bytes;
  c.lazy_staging = cfg->lazy_staging != 0;
  c.side_copy_streams = cfg->side_copy_streams != 0;
  c.kernel_mode_zerocopy = cfg->kernel_mode_zerocopy != 0;
  std::string err;
  int status = PF_ERR_STORAGE;
  auto e = pf::Engine::create(c, &err, &status);
  if (!e) {
    pf::last_error() = err;
    return status;
  }
  *out = reinterpret_cast<pf_engine_t>(e.release());
  return PF_OK;
}

int pf_engine_destroy(pf_engine_t e) {
  delete reinterpret_cast<pf::Engine*>(e);
  return PF_OK;
}

int pf_engine_register_context_layer_batch(
    pf_engine_t e, const char* instance_id, const char* namespace_, int device_id,
    uint64_t tp_rank, uint64_t pp_rank, uint64_t tp_size, uint64_t world_size, uint64_t n_layers,
    const char* const* layer_names, const uint64_t* data_ptrs, const uint64_t* size_bytes,
    const uint64_t* num_blocks, const uint64_t* bytes_per_block, const uint64_t* kv_stride_bytes,
    const uint64_t* segments, const uint64_t* block_stride_bytes, const uint32_t* layer_group_ids,
    int transfer_mode, int page_first) {
  PF_REQUIRE_PTR(e);
  PF_REQUIRE_PTR(instance_id);
  PF_REQUIRE_PTR(namespace_);
  if (transfer_mode != PF_MODE_DIRECT && transfer_mode != PF_MODE_KERNEL &&
      transfer_mode != PF_MODE_ZEROCOPY) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "unknown transfer mode %d", transfer_mode);
  }
  std::vector<std::string> names;
  for (uint64_t i = 0; i < n_layers; ++i) names.emplace_back(layer_names[i]);
  auto vec = [n_layers](const uint64_t* p) { return std::vector<uint64_t>(p, p + n_layers); };
  std::vector<uint64_t> strides;
  std::vector<uint32_t> groups;
  if (block_stride_bytes) strides.assign(block_stride_bytes, block_stride_bytes + n_layers);
  if (layer_group_ids) groups.assign(layer_group_ids, layer_group_ids + n_layers);
  std::string err;
  int st = reinterpret_cast<pf::Engine*>(e)->register_context_layer_batch_strided(
      instance_id, namespace_, device_id, tp_rank, pp_rank, tp_size, world_size, names,
      vec(data_ptrs), vec(size_bytes), vec(num_blocks), vec(bytes_per_block), vec(kv_stride_bytes),
      vec(segments), block_stride_bytes ? &strides : nullptr, layer_group_ids ? &groups : nullptr,
      static_cast<pf::TransferMode>(transfer_mode), page_first != 0, &err);
  if (st != PF_OK) pf::last_error() = err;
  return st;
}

int pf_engine_unregister_instance(pf_engine_t e, const char* instance_id) {
  PF_REQUIRE_PTR(e);
  PF_REQUIRE_PTR(instance_id);
  std::string err;
  int st = reinterpret_cast<pf::Engine*>(e)->unregister_instance(instance_id, &err);
  if (st != PF_OK) pf::last_error() = err;
  return st;
}

int pf_engine_batch_save(pf_engine_t e, const char* instance_id, uint64_t tp_rank,
                         uint64_t pp_rank, int device_id, const pf_layer_save* saves,
                         uint64_t n_saves) {
  PF_REQUIRE_PTR(e);
  PF_REQUIRE_PTR(instance_id);
  std::vector<pf::LayerSaveView> v(n_saves);
  for (uint64_t i = 0; i < n_saves; ++i) {
    v[i].layer_name = saves[i].layer_name;
    v[i].block_ids = saves[i].block_ids;
    v[i].n_ids = saves[i].n_blocks;
    // A NULL hash list with blocks present is a length mismatch, as in the
    // reference's engine-level contract (offload.rs:328-335).
    const bool has_hashes = saves[i].block_hashes != nullptr && saves[i].block_hash_lens != nullptr;
    v[i].hashes = has_hashes ? saves[i].block_hashes : nullptr;
    v[i].hash_lens = has_hashes ? saves[i].block_hash_lens : nullptr;
    v[i].n_hashes = has_hashes ? saves[i].n_blocks : 0;
    if (saves[i].n_blocks != 0 && saves[i].block_ids == nullptr) {
      return pf::fail(PF_ERR_INVALID_ARGUMENT, "layer save %llu has blocks but no block_ids",
                      static_cast<unsigned long long>(i));
    }
  }
  std::string err;
  int st = reinterpret_cast<pf::Engine*>(e)->batch_save_kv_blocks(instance_id, tp_rank, pp_rank,
                                                                  device_id, v, &err);
  if (st != PF_OK) pf::last_error() = err;
  return st;
}

int pf_engine_last_save_profile(pf_engine_t e, pf_save_profile* out) {
  PF_REQUIRE_PTR(e);
  PF_REQUIRE_PTR(out);
  const pf::SaveProfile p = reinterpret_cast<pf::Engine*>(e)->last_save_profile();
  out->validate_ms = p.validate_ms;
  out->filter_ms = p.filter_ms;
  out->alloc_ms = p.alloc_ms;
  out->assemble_ms = p.assemble_ms;
  out->transfer_ms = p.transfer_ms;
  out->publish_ms = p.publish_ms;
  out->total_ms = p.total_ms;
  out->bytes = p.bytes;
  return PF_OK;
}

int pf_engine_last_load_profile(pf_engine_t e, pf_task_result* out) {
  PF_REQUIRE_PTR(e);
  PF_REQUIRE_PTR(out);
  pf::TaskResult r;
  if (!reinterpret_cast<pf::Engine*>(e)->last_load_profile(&r)) {
    return pf::fail(PF_ERR_STORAGE, "no load task has settled on this engine yet");
  }
  fill_task_result(r, out);
  return PF_OK;
}

uint64_t pf_engine_staging_bytes(pf_engine_t e) {
  return e ? reinterpret_cast<pf::Engine*>(e)->staging_bytes() : 0;
}

int pf_engine_query_prefix(pf_engine_t e, const char* instance_id, const uint8_t* const* hashes,
                           const uint32_t* hash_lens, uint64_t n, uint64_t* out_hits,
                           uint64_t* out_lease) {
  PF_REQUIRE_PTR(e);
  PF_REQUIRE_PTR(instance_id);
  PF_REQUIRE_PTR(out_hits);
  PF_REQUIRE_PTR(out_lease);
  std::vector<std::string_view> h;
  h.reserve(n);
  for (uint64_t i = 0; i < n; ++i) {
    h.emplace_back(reinterpret_cast<const char*>(hashes[i]), hash_lens[i]);
  }
  std::string err;
  int st = reinterpret_cast<pf::Engine*>(e)->query_prefix(instance_id, h, out_hits, out_lease, &err);
  if (st != PF_OK) pf::last_error() = err;
  return st;
}

int pf_engine_release_lease(pf_engine_t e, uint64_t lease) {
  PF_REQUIRE_PTR(e);
  return reinterpret_cast<pf::Engine*>(e)->release_query_lease(lease)
             ? PF_OK
             : pf::fail(PF_ERR_STORAGE, "query lease %llu not found",
                        static_cast<unsigned long long>(lease));
}

int pf_engine_batch_load(pf_engine_t e, const char* instance_id, uint64_t tp_rank, int device_id,
                         uint64_t n_groups, const char* const* const* group_layer_names,
                         const uint64_t* group_sizes, uint64_t lease,
                         const int64_t* const* dest_block_ids, uint64_t n_blocks,
                         const char* load_state_shm, pf_task_t* out_task) {
  PF_REQUIRE_PTR(e);
  PF_REQUIRE_PTR(instance_id);
  PF_REQUIRE_PTR(out_task);
  std::vector<std::vector<std::string>> groups(n_groups);
  pf::LoadRequest req;
  req.lease = lease;
  req.block_ids_by_group.resize(n_groups);
  for (uint64_t g = 0; g < n_groups; ++g) {
    for (uint64_t i = 0; i < group_sizes[g]; ++i) groups[g].emplace_back(group_layer_names[g][i]);
    req.block_ids_by_group[g].assign(dest_block_ids[g], dest_block_ids[g] + n_blocks);
  }
  auto h = std::make_unique<TaskHandle>();
  std::string err;
  std::string shm = load_state_shm ? load_state_shm : "";
  int st = reinterpret_cast<pf::Engine*>(e)->batch_load_kv_blocks_multi_layer(
      instance_id, tp_rank, device_id, groups, {req}, shm, &h->fut, &err);
  if (st != PF_OK) {
    pf::last_error() = err;
    // A pre-submit failure marks the caller's LoadState as failed (lib.rs:672-677).
    if (!shm.empty()) {
      std::string aerr;
      if (auto ls = pf::LoadState::attach(shm, &aerr)) ls->set_error();
    }
    return st;
  }
  *out_task = reinterpret_cast<pf_task_t>(h.release());
  return PF_OK;
}

int pf_engine_batch_load_multi(pf_engine_t e, const char* instance_id, uint64_t tp_rank,
                               int device_id, uint64_t n_groups,
                               const char* const* const* group_layer_names,
                               const uint64_t* group_sizes, const pf_load_request* loads,
                               uint64_t n_loads, const char* load_state_shm, pf_task_t* out_task) {
  PF_REQUIRE_PTR(e);
  PF_REQUIRE_PTR(instance_id);
  PF_REQUIRE_PTR(out_task);
  if (n_loads != 0) PF_REQUIRE_PTR(loads);
  std::vector<std::vector<std::string>> groups(n_groups);
  for (uint64_t g = 0; g < n_groups; ++g) {
    for (uint64_t i = 0; i < group_sizes[g]; ++i) groups[g].emplace_back(group_layer_names[g][i]);
  }
  std::vector<pf::LoadRequest> reqs(n_loads);
  for (uint64_t l = 0; l < n_loads; ++l) {
    reqs[l].lease = loads[l].lease;
    reqs[l].block_ids_by_group.resize(n_groups);
    for (uint64_t g = 0; g < n_groups; ++g) {
      if (loads[l].n_blocks != 0 && (!loads[l].dest_block_ids || !loads[l].dest_block_ids[g])) {
        return pf::fail(PF_ERR_INVALID_ARGUMENT, "load %llu has no destination list for group %llu",
                        static_cast<unsigned long long>(l), static_cast<unsigned long long>(g));
      }
      if (loads[l].n_blocks != 0) {
        reqs[l].block_ids_by_group[g].assign(loads[l].dest_block_ids[g],
                                             loads[l].dest_block_ids[g] + loads[l].n_blocks);
      }
    }
  }
  auto h = std::make_unique<TaskHandle>();
  std::string err;
  std::string shm = load_state_shm ? load_state_shm : "";
  int st = reinterpret_cast<pf::Engine*>(e)->batch_load_kv_blocks_multi_layer(
      instance_id, tp_rank, device_id, groups, reqs, shm, &h->fut, &err);
  if (st != PF_OK) {
    pf::last_error() = err;
    if (!shm.empty()) {
      std::string aerr;
      if (auto ls = pf::LoadState::attach(shm, &aerr)) ls->set_error();
    }
    return st;
  }
  *out_task = reinterpret_cast<pf_task_t>(h.release());
  return PF_OK;
}

int pf_engine_query_group_membership(pf_engine_t e, const char* instance_id, uint32_t group,
                                     const uint8_t* const* hashes, const uint32_t* hash_lens,
                                     uint64_t n, uint8_t* out_present) {
  PF_REQUIRE_PTR(e);
  PF_REQUIRE_PTR(instance_id);
  if (n != 0) {
    PF_REQUIRE_PTR(hashes);
    PF_REQUIRE_PTR(hash_lens);
    PF_REQUIRE_PTR(out_present);
  }
  std::vector<std::string_view> h;
  h.reserve(n);
  for (uint64_t i = 0; i < n; ++i) {
    h.emplace_back(reinterpret_cast<const char*>(hashes[i]), hash_lens[i]);
  }
  std::vector<uint8_t> present;
  std::string err;
  int st = reinterpret_cast<pf::Engine*>(e)->query_group_membership(instance_id, group, h, &present,
                                                                    &err);
  if (st != PF_OK) {
    pf::last_error() = err;
    return st;
  }
  for (uint64_t i = 0; i < n; ++i) out_present[i] = present[i];
  return PF_OK;
}

int pf_engine_create_group_lease(pf_engine_t e, const char* instance_id, uint32_t group,
                                 const uint8_t* const* hashes, const uint32_t* hash_lens,
                                 uint64_t n, uint64_t* out_lease) {
  PF_REQUIRE_PTR(e);
  PF_REQUIRE_PTR(instance_id);
  PF_REQUIRE_PTR(out_lease);
  if (n != 0) {
    PF_REQUIRE_PTR(hashes);
    PF_REQUIRE_PTR(hash_lens);
  }
  std::vector<std::string_view> h;
  h.reserve(n);
  for (uint64_t i = 0; i < n; ++i) {
    h.emplace_back(reinterpret_cast<const char*>(hashes[i]), hash_lens[i]);
  }
  std::string err;
  int st = reinterpret_cast<pf::Engine*>(e)->create_group_lease(instance_id, group, h, out_lease,
                                                                &err);
  if (st != PF_OK) pf::last_error() = err;
  return st;
}

int pf_engine_query_group_lease(pf_engine_t e, const char* instance_id, uint32_t group,
                                const uint8_t* const* hashes, const uint32_t* hash_lens,
                                uint64_t n, int require_all, uint8_t* out_present,
                                uint64_t* out_lease) {
  PF_REQUIRE_PTR(e);
  PF_REQUIRE_PTR(instance_id);
  PF_REQUIRE_PTR(out_lease);
  if (n != 0) {
    PF_REQUIRE_PTR(hashes);
    PF_REQUIRE_PTR(hash_lens);
    PF_REQUIRE_PTR(out_present);
  }
  std::vector<std::string_view> h;
  h.reserve(n);
  for (uint64_t i = 0; i < n; ++i) {
    h.emplace_back(reinterpret_cast<const char*>(hashes[i]), hash_lens[i]);
  }
  std::vector<uint8_t> present;
  std::string err;
  int st = reinterpret_cast<pf::Engine*>(e)->query_group_lease(instance_id, group, h,
                                                               require_all != 0, &present,
                                                               out_lease, &err);
  if (st != PF_OK) {
    pf::last_error() = err;
    return st;
  }
  for (uint64_t i = 0; i < n; ++i) out_present[i] = present[i];
  return PF_OK;
}

int pf_engine_pool_usage(pf_engine_t e, uint64_t* out_used, uint64_t* out_total) {
  PF_REQUIRE_PTR(e);
  PF_REQUIRE_PTR(out_used);
  PF_REQUIRE_PTR(out_total);
  reinterpret_cast<pf::Engine*>(e)->pool_usage(out_used, out_total);
  return PF_OK;
}

uint64_t pf_engine_cached_blocks(pf_engine_t e) {
  return e ? reinterpret_cast<pf::Engine*>(e)->cached_blocks() : 0;
}

uint64_t pf_engine_inflight_blocks(pf_engine_t e) {
  return e ? reinterpret_cast<pf::Engine*>(e)->inflight_blocks() : 0;
}

uint64_t pf_engine_gc_stale_inflight(pf_engine_t e, uint64_t max_age_ms) {
  return e ? reinterpret_cast<pf::Engine*>(e)->gc_stale_inflight(
                 std::chrono::milliseconds(max_age_ms))
           : 0;
}

uint64_t pf_engine_evict_all(pf_engine_t e) {
  return e ? reinterpret_cast<pf::Engine*>(e)->evict_all() : 0;
}

uint64_t pf_engine_sweep_expired_leases(pf_engine_t e) {
  return e ? reinterpret_cast<pf::Engine*>(e)->sweep_expired_leases() : 0;
}

uint64_t pf_engine_live_leases(pf_engine_t e) {
  return e ? reinterpret_cast<pf::Engine*>(e)->live_leases() : 0;
}

}  // extern "C"
