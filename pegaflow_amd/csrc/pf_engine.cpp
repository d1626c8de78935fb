#include "pf_engine.hpp"

#include <algorithm>
#include <chrono>
#include <cstring>
#include <set>

#include "pf_common.hpp"
#include "pf_sync_state.hpp"

namespace pf {

namespace {

constexpr uint64_t kSsdAlignment = 512;

int bad(std::string* err, int code, std::string msg) {
  if (err) *err = std::move(msg);
  return code;
}

}  // namespace

// Per-layer state of one save (offload.rs:52-66).
// One distinct (group, hash sequence) of a save call; layers that carry the
// same one share it.
struct SaveList {
  uint32_t group = 0;
  const uint8_t* const* hashes = nullptr;
  const uint32_t* lens = nullptr;
  size_t n = 0;
  std::vector<BlockKey> keys;  // group-encoded key of each position
  std::vector<uint32_t> kept;  // positions not in the store yet, ascending
  bool same_as(uint32_t g, const LayerSaveView& s) const {
    if (g != group || s.n_hashes != n) return false;
    if (s.hashes == hashes && s.hash_lens == lens) return true;
    for (size_t i = 0; i < n; ++i) {
      if (s.hash_lens[i] != lens[i]) return false;
      if (s.hashes[i] != hashes[i] && std::memcmp(s.hashes[i], hashes[i], lens[i]) != 0) {
        return false;
      }
    }
    return true;
  }
};

struct SaveLayerCtx {
  std::string layer_name;
  KVCacheLayout layout;
  size_t slot_id = 0;
  uint32_t group = 0;
  const uint64_t* block_ids = nullptr;         // the caller's list, all positions
  size_t list = 0;                             // index of its SaveList
  std::shared_ptr<std::vector<uint32_t>> ids;  // device block of each kept position
  uint64_t stride = 0;                         // host stride of one position
  // Batch image: one K (and V) allocation; blockwise: one per kept position.
  std::vector<std::shared_ptr<PinnedAllocation>> k_allocs, v_allocs;
  std::vector<RawBlock> raw_blocks;            // blockwise only: handles the task points at

  // The host image of kept position q as a block of its own (offload.rs:454-509).
  bool make_raw(size_t q, bool blockwise, RawBlock* out) const {
    const size_t a = blockwise ? q : 0;
    const uint64_t off = blockwise ? 0 : q * stride;
    Segment k;
    if (!Segment::create(k_allocs[a]->as_ptr() + off, stride, k_allocs[a], &k)) return false;
    if (v_allocs.empty()) {
      *out = RawBlock::single_segment(std::move(k));
      return true;
    }
    Segment v;
    if (!Segment::create(v_allocs[a]->as_ptr() + off, stride, v_allocs[a], &v)) return false;
    *out = RawBlock::two_segments(std::move(k), std::move(v));
    return true;
  }
};

// ---------------------------------------------------------------------------
// InstanceContext
// ---------------------------------------------------------------------------

int InstanceContext::check_accepting(int device_id, size_t tp_rank, std::string* err) {
  if (tp_rank >= tp_size_) {
    return bad(err, PF_ERR_INVALID_ARGUMENT, "tp_rank " + std::to_string(tp_rank) +
                                                 " out of range (tp_size " +
                                                 std::to_string(tp_size_) + ")");
  }
  std::lock_guard<std::mutex> lock(mu_);
  // Duplicate device first: a restarted worker must hear that its device
  // still exists, not a generic "fully registered" (instance.rs:455-470).
  if (gpus_.count(device_id)) {
    return bad(err, PF_ERR_INVALID_ARGUMENT,
               "GPU context for device " + std::to_string(device_id) + " already exists");
  }
  if (topology_) {
    return bad(err, PF_ERR_INVALID_ARGUMENT,
               "instance " + id_ + " is already fully registered (" + std::to_string(world_size_) +
                   " workers); device " + std::to_string(device_id) + " cannot join");
  }
  return PF_OK;
}

int InstanceContext::register_new_gpu(std::shared_ptr<GpuContext> ctx, std::string* err) {
  std::lock_guard<std::mutex> lock(mu_);
  const int device_id = ctx->reg.device_id;
  if (gpus_.count(device_id)) {
    return bad(err, PF_ERR_INVALID_ARGUMENT,
               "GPU context for device " + std::to_string(device_id) + " already exists");
  }
  if (topology_) {
    return bad(err, PF_ERR_INVALID_ARGUMENT,
               "instance " + id_ + " is already fully registered (" + std::to_string(world_size_) +
                   " workers); device " + std::to_string(device_id) + " cannot join");
  }
  std::shared_ptr<LayerTopology> sealed;
  if (gpus_.size() + 1 == world_size_) {
    // The registration that completes the worker set seals the topology; if
    // that fails the registration is rejected as a whole.
    std::vector<const WorkerRegistration*> workers;
    for (auto& kv : gpus_) workers.push_back(&kv.second->reg);
    workers.push_back(&ctx->reg);
    sealed = std::make_shared<LayerTopology>();
    std::string cause;
    if (!LayerTopology::seal(workers, tp_size_, page_first_, id_, world_size_, sealed.get(),
                             &cause)) {
      return bad(err, PF_ERR_INVALID_ARGUMENT, cause);
    }
  }
  gpus_[device_id] = std::move(ctx);
  if (sealed) topology_ = std::move(sealed);
  return PF_OK;
}

std::shared_ptr<LayerTopology> InstanceContext::sealed_topology(std::string* err) {
  std::lock_guard<std::mutex> lock(mu_);
  if (!topology_ && err) {
    *err = "instance " + id_ + " registration incomplete: " + std::to_string(gpus_.size()) + "/" +
           std::to_string(world_size_) + " workers registered";
  }
  return topology_;
}

std::vector<std::shared_ptr<GpuContext>> InstanceContext::gpus() {
  std::lock_guard<std::mutex> lock(mu_);
  std::vector<std::shared_ptr<GpuContext>> out;
  for (auto& kv : gpus_) out.push_back(kv.second);
  return out;
}

std::shared_ptr<GpuContext> InstanceContext::get_gpu(int device_id) {
  std::lock_guard<std::mutex> lock(mu_);
  auto it = gpus_.find(device_id);
  return it == gpus_.end() ? nullptr : it->second;
}

std::string InstanceContext::verify_topology(size_t tp_size, size_t world_size,
                                             bool page_first) const {
  if (tp_size_ == tp_size && world_size_ == world_size && page_first_ == page_first) return "";
  auto b = [](bool v) { return v ? "true" : "false"; };
  return "exists with tp=" + std::to_string(tp_size_) + ", world=" + std::to_string(world_size_) +
         ", page_first=" + b(page_first_) + "; requested tp=" + std::to_string(tp_size) +
         ", world=" + std::to_string(world_size) + ", page_first=" + b(page_first);
}

// ---------------------------------------------------------------------------
// Engine
// ---------------------------------------------------------------------------

std::unique_ptr<Engine> Engine::create(const EngineConfig& cfg, std::string* err, int* status) {
  std::unique_ptr<Engine> e(new Engine());
  e->cfg_ = cfg;
  e->numa_ = NumaTopology::detect();
  std::string perr;
  int pstatus = PF_ERR_STORAGE;
  if (cfg.numa_aware) {
    e->pool_ = PinnedAllocator::new_numa(cfg.pool_size, e->numa_.gpu_numa_nodes(), cfg.pool_shards,
                                         cfg.use_hugepages, cfg.ssd_enabled, cfg.unit_size_hint,
                                         &perr, &pstatus);
  } else {
    e->pool_ = PinnedAllocator::new_global(cfg.pool_size, cfg.pool_shards, cfg.use_hugepages,
                                           cfg.ssd_enabled, cfg.unit_size_hint, &perr, &pstatus);
  }
  if (!e->pool_) {
    if (err) *err = perr;
    if (status) *status = pstatus;
    return nullptr;
  }
  return e;
}

Engine::~Engine() {
  // Workers first (they may still touch host blocks), then blocks, then the pool.
  instances_.clear();
  leases_.clear();
  inflight_.clear();
  sealed_.clear();
  lru_reset();
}

std::shared_ptr<InstanceContext> Engine::get_instance(const std::string& id, std::string* err) {
  std::lock_guard<std::mutex> lock(mu_);
  auto it = instances_.find(id);
  if (it == instances_.end()) {
    if (err) *err = "instance " + id + " not found";  // lib.rs:92
    return nullptr;
  }
  return it->second;
}

int Engine::register_context_layer_batch_strided(
    const std::string& instance_id, const std::string& ns, int device_id, size_t tp_rank,
    size_t pp_rank, size_t tp_size, size_t world_size, const std::vector<std::string>& layer_names,
    const std::vector<uint64_t>& data_ptrs, const std::vector<uint64_t>& size_bytes,
    const std::vector<uint64_t>& num_blocks, const std::vector<uint64_t>& bytes_per_block,
    const std::vector<uint64_t>& kv_stride_bytes, const std::vector<uint64_t>& segments,
    const std::vector<uint64_t>* block_stride_bytes, const std::vector<uint32_t>* layer_group_ids,
    TransferMode mode, bool page_first, std::string* err) {
  const size_t n = layer_names.size();
  if (data_ptrs.size() != n || size_bytes.size() != n || num_blocks.size() != n ||
      bytes_per_block.size() != n || kv_stride_bytes.size() != n || segments.size() != n) {
    return bad(err, PF_ERR_INVALID_ARGUMENT,
               "registration metadata length mismatch: layer_names=" + std::to_string(n) +
                   ", data_ptrs=" + std::to_string(data_ptrs.size()) +
                   ", size_bytes=" + std::to_string(size_bytes.size()) +
                   ", num_blocks=" + std::to_string(num_blocks.size()) +
                   ", bytes_per_block=" + std::to_string(bytes_per_block.size()) +
                   ", kv_stride_bytes=" + std::to_string(kv_stride_bytes.size()) +
                   ", segments=" + std::to_string(segments.size()));
  }
  if (block_stride_bytes && block_stride_bytes->size() != n) {
    return bad(err, PF_ERR_INVALID_ARGUMENT,
               "registration metadata length mismatch: layer_names=" + std::to_string(n) +
                   ", block_stride_bytes=" + std::to_string(block_stride_bytes->size()));
  }
  if (layer_group_ids && layer_group_ids->size() != n) {
    return bad(err, PF_ERR_INVALID_ARGUMENT,
               "registration metadata length mismatch: layer_names=" + std::to_string(n) +
                   ", layer_group_ids=" + std::to_string(layer_group_ids->size()));
  }
  if (device_id < 0) {
    return bad(err, PF_ERR_INVALID_ARGUMENT,
               "device_id " + std::to_string(device_id) + " must be >= 0");
  }
  if (tp_size == 0 || world_size == 0) {
    return bad(err, PF_ERR_INVALID_ARGUMENT, "tp_size and world_size must be > 0");
  }
  auto ctx = std::make_shared<GpuContext>();
  ctx->reg.device_id = device_id;
  ctx->reg.tp_rank = tp_rank;
  ctx->reg.pp_rank = pp_rank;
  for (size_t i = 0; i < n; ++i) {
    KVCacheLayout layout;
    std::string cause;
    if (!KVCacheLayout::create(data_ptrs[i], size_bytes[i], num_blocks[i], bytes_per_block[i],
                               kv_stride_bytes[i], segments[i], &layout, &cause) ||
        (block_stride_bytes && !layout.with_block_stride((*block_stride_bytes)[i], &cause))) {
      return bad(err, PF_ERR_INVALID_ARGUMENT, "layer " + layer_names[i] + ": " + cause);
    }
    if (cfg_.ssd_enabled) layout.with_ssd_padding(kSsdAlignment);
    if (!ctx->reg.kv_caches.emplace(layer_names[i], layout).second) {
      return bad(err, PF_ERR_INVALID_ARGUMENT,
                 "duplicate layer name in registration batch: " + layer_names[i]);
    }
    if (layer_group_ids) ctx->reg.layer_groups[layer_names[i]] = (*layer_group_ids)[i];
  }
  if (ctx->reg.kv_caches.empty()) {
    return bad(err, PF_ERR_INVALID_ARGUMENT,
               "device " + std::to_string(device_id) + " registered no KV cache layers");
  }

  // get_or_create_instance (lib.rs:196-222).
  std::shared_ptr<InstanceContext> instance;
  {
    std::lock_guard<std::mutex> lock(mu_);
    auto it = instances_.find(instance_id);
    if (it != instances_.end()) {
      std::string mismatch = it->second->verify_topology(tp_size, world_size, page_first);
      if (!mismatch.empty()) {
        return bad(err, PF_ERR_INVALID_ARGUMENT, "instance " + instance_id + " " + mismatch);
      }
      instance = it->second;
    } else {
      instance = std::make_shared<InstanceContext>(instance_id, ns, ns_id_locked(ns), tp_size,
                                                   world_size, page_first);
      instances_[instance_id] = instance;
    }
  }
  ctx->preferred_numa = numa_.numa_for_gpu(device_id);
  if (pool_->is_numa() && ctx->preferred_numa.is_unknown()) {
    return bad(err, PF_ERR_INVALID_ARGUMENT,
               "NUMA-aware allocation is enabled, but GPU " + std::to_string(device_id) +
                   " NUMA affinity is unknown. Please ensure the GPU's PCI NUMA node is "
                   "detectable, or disable NUMA-aware allocation.");
  }
  int st = instance->check_accepting(device_id, tp_rank, err);
  if (st != PF_OK) return st;
  std::string werr;
  int wstatus = PF_ERR_DEVICE_INIT;
  WorkerPoolOptions options;
  options.use_descriptor_backends = cfg_.use_descriptor_backends;
  options.auto_staged_min_bytes = cfg_.auto_staged_min_bytes;
  options.lazy_staging = cfg_.lazy_staging;
  options.side_copy_streams = cfg_.side_copy_streams;
  // A staging slot is filled with the layers of a task one behind the other, so
  // it never needs to be larger than everything the context registered: a context
  // of small layers gets small slots.  Small layers that follow one another
  // share up to 32 MiB of a slot even with per-layer events: that is the floor.
  {
    uint64_t fill = 0;
    for (const auto& kv : ctx->reg.kv_caches) fill += kv.second.block_bytes() * kv.second.num_blocks();
    constexpr uint64_t kSlotFloor = 32ull << 20, kSlotDefault = 512ull << 20;
    const uint64_t cap = cfg_.staging_slot_bytes ? cfg_.staging_slot_bytes : kSlotDefault;
    fill = (std::max(fill, kSlotFloor) + 0xFFFFFull) & ~0xFFFFFull;
    options.staging_slot_bytes = std::min(cap, fill);
  }
  if (mode == TransferMode::Kernel && cfg_.kernel_mode_zerocopy) mode = TransferMode::ZeroCopy;
  ctx->worker_pool = GpuWorkerPool::spawn(device_id, ctx->preferred_numa, mode, options, &werr,
                                          &wstatus);
  if (!ctx->worker_pool) return bad(err, wstatus, werr);
  return instance->register_new_gpu(std::move(ctx), err);
}

int Engine::unregister_instance(const std::string& instance_id, std::string* err) {
  std::shared_ptr<InstanceContext> removed;
  {
    std::lock_guard<std::mutex> lock(mu_);
    auto it = instances_.find(instance_id);
    if (it == instances_.end()) {
      return bad(err, PF_ERR_INSTANCE_MISSING, "instance " + instance_id + " not found");
    }
    removed = it->second;
    instances_.erase(it);
    for (auto lit = leases_.begin(); lit != leases_.end();) {
      lit = lit->second.instance_id == instance_id ? leases_.erase(lit) : std::next(lit);
    }
  }
  removed.reset();  // joins the worker threads outside the lock
  return PF_OK;
}

uint32_t Engine::ns_id_locked(const std::string& ns) {
  auto it = ns_ids_.find(ns);
  if (it != ns_ids_.end()) return it->second;
  const uint32_t id = static_cast<uint32_t>(ns_ids_.size());
  ns_ids_.emplace(ns, id);
  return id;
}

bool Engine::seal_insert(BlockKey&& key, std::shared_ptr<SealedBlock> block) {
  auto [it, fresh] = sealed_.try_emplace(std::move(key));
  if (!fresh) return false;
  it->second.block = std::move(block);
  it->second.key = &it->first;
  lru_make_newest(&it->second);
  return true;
}

Engine::SealedEntry* Engine::find_sealed(uint32_t ns, std::string_view hash, uint32_t group) {
  SealedTable::iterator it;
  if (group == 0) {
    it = sealed_.find(BlockKeyView(ns, hash));
  } else {
    const std::string encoded = group_hash(std::string(hash), group);
    it = sealed_.find(BlockKeyView(ns, encoded));
  }
  return it == sealed_.end() ? nullptr : &it->second;
}

bool Engine::evict_one() {
  // mu_ held by the caller.  Least recently used first; blocks that are
  // leased or being loaded (someone else holds a reference) stay.
  for (SealedEntry* e = lru_.newer; e != &lru_; e = e->newer) {
    if (e->block.use_count() > 1) continue;
    lru_unlink(e);
    auto it = sealed_.find(*e->key);
    if (it != sealed_.end()) sealed_.erase(it);
    return true;
  }
  return false;
}

size_t Engine::sweep_expired_locked() {
  const auto now = std::chrono::steady_clock::now();
  size_t gone = 0;
  for (auto it = leases_.begin(); it != leases_.end();) {
    if (it->second.expires_at > now) {
      ++it;
    } else {
      it = leases_.erase(it);
      ++gone;
    }
  }
  return gone;
}

size_t Engine::sweep_expired_leases() {
  std::lock_guard<std::mutex> lock(mu_);
  return sweep_expired_locked();
}

size_t Engine::live_leases() {
  std::lock_guard<std::mutex> lock(mu_);
  return leases_.size();
}

std::shared_ptr<PinnedAllocation> Engine::allocate(uint64_t size, NumaNode numa) {
  bool swept = false;
  for (;;) {
    if (auto a = pool_->allocate(size, numa)) return a;
    std::lock_guard<std::mutex> lock(mu_);
    if (evict_one()) continue;
    // Nothing evictable is left: blocks pinned by leases whose time is up
    // (a worker that died between query and load) are given back first.
    if (swept || sweep_expired_locked() == 0) return nullptr;
    swept = true;
  }
}

size_t Engine::cached_blocks() {
  std::lock_guard<std::mutex> lock(mu_);
  return sealed_.size();
}

size_t Engine::inflight_blocks() {
  std::lock_guard<std::mutex> lock(mu_);
  return inflight_.size();
}

// write_path.rs:302-330: blocks whose remaining slots never arrived give their
// pinned memory back.
size_t Engine::gc_stale_inflight(std::chrono::milliseconds max_age) {
  std::lock_guard<std::mutex> lock(mu_);
  sweep_expired_locked();  // the same periodic caller keeps the lease table clean
  size_t cleaned = 0;
  for (auto it = inflight_.begin(); it != inflight_.end();) {
    if (it->second.age() > max_age) {
      it = inflight_.erase(it);
      ++cleaned;
    } else {
      ++it;
    }
  }
  return cleaned;
}

size_t Engine::evict_all() {
  std::lock_guard<std::mutex> lock(mu_);
  size_t n = 0;
  while (evict_one()) ++n;
  return n;
}

// offload.rs:182-282.
int Engine::alloc_page_first_targets(const LayerTopology& topo, SaveLayerCtx* ctxs, size_t n,
                                     NumaNode numa,
                                     std::vector<std::shared_ptr<PinnedAllocation>>* pages,
                                     std::vector<LayerTransferData>* out, std::string* err) {
  const size_t shard = ctxs[0].slot_id;
  size_t page_size = 0;
  topo.shard_page_size(shard, &page_size);
  const SaveLayerCtx& first = ctxs[0];
  std::set<size_t> layer_ids;
  for (size_t i = 0; i < n; ++i) {
    if (ctxs[i].layout.is_split()) {
      return bad(err, PF_ERR_INVALID_ARGUMENT,
                 "page-first save does not support split K/V (layer " + ctxs[i].layer_name + ")");
    }
    if (ctxs[i].slot_id != shard) {
      return bad(err, PF_ERR_INVALID_ARGUMENT,
                 "page-first save spans multiple shards (one writer must save one shard)");
    }
    // Same hashes (same list) and same block ids, position by position.
    if (ctxs[i].list != first.list || *ctxs[i].ids != *first.ids) {
      return bad(err, PF_ERR_INVALID_ARGUMENT,
                 "page-first save requires the same block set across all layers");
    }
    size_t id = 0;
    std::string cause;
    if (!topo.layer_id(ctxs[i].layer_name, &id, &cause)) {
      return bad(err, PF_ERR_INVALID_ARGUMENT, cause);
    }
    layer_ids.insert(id);
  }
  size_t shard_layers = 0;
  topo.shard_layer_count(shard, &shard_layers);
  if (layer_ids.size() != shard_layers) {
    return bad(err, PF_ERR_INVALID_ARGUMENT,
               "page-first save must cover all " + std::to_string(shard_layers) +
                   " layers of shard " + std::to_string(shard) + ", got " +
                   std::to_string(layer_ids.size()) +
                   " distinct (one worker must write a shard's entire page)");
  }
  if (page_size == 0) return bad(err, PF_ERR_STORAGE, "page size is zero");
  const size_t num = first.ids->size();
  auto page_ptrs = std::make_shared<std::vector<MappedPinnedPtr>>();
  auto page_ids = std::make_shared<std::vector<uint64_t>>();
  page_ptrs->reserve(num);
  page_ids->reserve(num);
  for (size_t b = 0; b < num; ++b) {
    auto page = allocate(page_size, numa);
    if (!page) return bad(err, PF_ERR_STORAGE, "pinned pool exhausted while allocating page");
    MappedPinnedPtr p;
    if (!page->mapped_ptr_for_host_range(page->as_ptr(), page_size, &p)) {
      return bad(err, PF_ERR_STORAGE, "page exceeds its pinned allocation");
    }
    page_ptrs->push_back(p);
    page_ids->push_back(page->allocation_id());
    pages->push_back(std::move(page));
  }
  for (size_t i = 0; i < n; ++i) {
    size_t id = 0, offset = 0, layer_bytes = 0;
    topo.layer_id(ctxs[i].layer_name, &id, nullptr);
    topo.page_placement(id, &offset, &layer_bytes);
    if (offset + layer_bytes > page_size) {
      return bad(err, PF_ERR_STORAGE, "page slice exceeds its pinned allocation");
    }
    LayerTransferData ltd;
    ltd.layer_name = ctxs[i].layer_name;
    ltd.layout = ctxs[i].layout;
    ltd.image.kind = HostImage::Kind::Paged;
    ltd.image.block_ids = ctxs[i].ids;
    ltd.image.pages = page_ptrs;
    ltd.image.page_allocation_ids = page_ids;
    ltd.image.offset = offset;
    ltd.image.page_len = page_size;
    out->push_back(std::move(ltd));
  }
  return PF_OK;
}

int Engine::batch_save_kv_blocks(const std::string& instance_id, size_t tp_rank, size_t pp_rank,
                                 int device_id, const std::vector<LayerSaveView>& saves,
                                 std::string* err) {
  using Clock = std::chrono::steady_clock;
  const auto t_begin = Clock::now();
  auto ms_since = [](Clock::time_point t) {
    return std::chrono::duration<double, std::milli>(Clock::now() - t).count();
  };
  SaveProfile prof;
  auto instance = get_instance(instance_id, err);
  if (!instance) return PF_ERR_INSTANCE_MISSING;
  auto topo = instance->sealed_topology(err);
  if (!topo) return PF_ERR_INVALID_ARGUMENT;
  const uint32_t ns = instance->ns_id();

  // ---- Phase 0: resolve metadata, bounds-check block ids ------------------
  auto gpu = instance->get_gpu(device_id);
  if (!gpu) {
    return bad(err, PF_ERR_WORKER_MISSING,
               "device " + std::to_string(device_id) + " not found in instance " + instance_id);  // lib.rs:93-95
  }
  if (gpu->reg.tp_rank != tp_rank || gpu->reg.pp_rank != pp_rank) {
    return bad(err, PF_ERR_INVALID_ARGUMENT,
               "device_id " + std::to_string(device_id) + " is registered for tp_rank " +
                   std::to_string(gpu->reg.tp_rank) + ", pp_rank " +
                   std::to_string(gpu->reg.pp_rank) + ", but save requested tp_rank " +
                   std::to_string(tp_rank) + ", pp_rank " + std::to_string(pp_rank));
  }
  // Layers that carry the same hash sequence for the same group (the usual
  // case: one request's blocks saved for every layer) share one SaveList, so
  // the store is consulted once per block, not once per (layer, block).
  std::vector<SaveList> lists;
  std::vector<SaveLayerCtx> ctxs;
  for (const LayerSaveView& s : saves) {
    const std::string layer_name = s.layer_name ? s.layer_name : "";
    if (s.n_ids != s.n_hashes) {
      return bad(err, PF_ERR_INVALID_ARGUMENT,
                 "block_ids length " + std::to_string(s.n_ids) + " does not match block_hashes " +
                     std::to_string(s.n_hashes) + " for layer " + layer_name);
    }
    size_t layer_id = 0;
    std::string cause;
    if (!topo->layer_id(layer_name, &layer_id, &cause)) {
      return bad(err, PF_ERR_INVALID_ARGUMENT, cause);
    }
    auto lit = gpu->reg.kv_caches.find(layer_name);
    if (lit == gpu->reg.kv_caches.end()) {
      return bad(err, PF_ERR_INVALID_ARGUMENT, "layer " + layer_name + " not registered on device");
    }
    SaveLayerCtx ctx;
    ctx.layer_name = layer_name;
    ctx.layout = lit->second;
    if (!topo->slot_index(layer_id, tp_rank, &ctx.slot_id, &cause)) {
      return bad(err, PF_ERR_INVALID_ARGUMENT, cause);
    }
    ctx.group = topo->group_of_layer(layer_id);
    const uint64_t nb = ctx.layout.num_blocks();
    for (size_t i = 0; i < s.n_ids; ++i) {
      if (s.block_ids[i] >= nb) {
        return bad(err, PF_ERR_INVALID_ARGUMENT,
                   "block_id " + std::to_string(s.block_ids[i]) + " out of range (num_blocks=" +
                       std::to_string(nb) + ") for layer " + layer_name);
      }
    }
    if (s.n_ids == 0) continue;
    ctx.block_ids = s.block_ids;
    size_t li = lists.size();
    for (size_t k = lists.size(); k-- > 0;) {
      if (lists[k].same_as(ctx.group, s)) {
        li = k;
        break;
      }
    }
    if (li == lists.size()) {
      SaveList l;
      l.group = ctx.group;
      l.hashes = s.hashes;
      l.lens = s.hash_lens;
      l.n = s.n_hashes;
      lists.push_back(std::move(l));
    }
    ctx.list = li;
    ctxs.push_back(std::move(ctx));
  }
  if (ctxs.empty()) return PF_OK;
  prof.validate_ms = ms_since(t_begin);

  // ---- Phase 1: drop hashes whose group-encoded key is already cached -----
  auto t_phase = Clock::now();
  size_t to_save = 0;
  {
    for (SaveList& l : lists) {
      l.keys.reserve(l.n);
      for (size_t i = 0; i < l.n; ++i) {
        l.keys.emplace_back(
            ns, group_hash(std::string(reinterpret_cast<const char*>(l.hashes[i]), l.lens[i]),
                           l.group));
      }
    }
    std::lock_guard<std::mutex> lock(mu_);
    for (SaveList& l : lists) {
      for (size_t i = 0; i < l.n; ++i) {
        if (sealed_.find(l.keys[i]) == sealed_.end()) l.kept.push_back(static_cast<uint32_t>(i));
      }
      to_save += l.kept.size();
    }
  }
  if (to_save == 0) return PF_OK;
  ctxs.erase(std::remove_if(ctxs.begin(), ctxs.end(),
                            [&](const SaveLayerCtx& c) { return lists[c.list].kept.empty(); }),
             ctxs.end());
  if (ctxs.empty()) return PF_OK;
  for (SaveLayerCtx& ctx : ctxs) {
    const SaveList& l = lists[ctx.list];
    auto ids = std::make_shared<std::vector<uint32_t>>();
    ids->reserve(l.kept.size());
    for (uint32_t pos : l.kept) ids->push_back(static_cast<uint32_t>(ctx.block_ids[pos]));
    ctx.ids = std::move(ids);
  }
  prof.filter_ms = ms_since(t_phase);

  // ---- Phase 2: pinned allocation + host images ----------------------------
  t_phase = Clock::now();
  const NumaNode numa = gpu->preferred_numa;
  const bool page_first = topo->is_page_first();
  std::vector<LayerTransferData> gpu_layers;
  std::vector<std::shared_ptr<PinnedAllocation>> pages;
  if (page_first) {
    int st = alloc_page_first_targets(*topo, ctxs.data(), ctxs.size(), numa, &pages, &gpu_layers,
                                      err);
    if (st != PF_OK) return st;
  } else {
    for (auto& ctx : ctxs) {
      const KVCacheLayout& layout = ctx.layout;
      const size_t num = ctx.ids->size();
      const size_t alloc_count = cfg_.blockwise_alloc ? num : 1;
      const size_t per_alloc = cfg_.blockwise_alloc ? 1 : num;
      auto alloc_pinned = [&](uint64_t stride, const char* what,
                              std::shared_ptr<PinnedAllocation>* out) -> int {
        uint64_t size = 0;
        if (__builtin_mul_overflow(stride, static_cast<uint64_t>(per_alloc), &size) || size == 0) {
          return bad(err, PF_ERR_STORAGE, std::string("allocation size overflow for ") + what);
        }
        *out = allocate(size, numa);
        if (!*out) {
          return bad(err, PF_ERR_STORAGE,
                     std::string("pinned pool exhausted while allocating ") + what);
        }
        return PF_OK;
      };
      const bool split = layout.is_split();
      ctx.stride = split ? layout.padded_segment_bytes() : layout.padded_block_bytes();
      for (size_t a = 0; a < alloc_count; ++a) {
        std::shared_ptr<PinnedAllocation> k_alloc, v_alloc;
        int st = alloc_pinned(ctx.stride, split ? "K segment buffer" : "block buffer", &k_alloc);
        if (st == PF_OK && split) st = alloc_pinned(ctx.stride, "V segment buffer", &v_alloc);
        if (st != PF_OK) return st;
        ctx.k_allocs.push_back(std::move(k_alloc));
        if (split) ctx.v_allocs.push_back(std::move(v_alloc));
      }
      LayerTransferData ltd;
      ltd.layer_name = ctx.layer_name;
      ltd.layout = layout;
      if (!cfg_.blockwise_alloc) {
        // One K buffer and one V buffer (or one block buffer): a uniform image.
        ltd.image.kind = HostImage::Kind::Uniform;
        ltd.image.block_ids = ctx.ids;
        ltd.image.stride = ctx.stride;
        const uint64_t bytes = ctx.stride * num;
        if (!ctx.k_allocs[0]->mapped_ptr_for_host_range(ctx.k_allocs[0]->as_ptr(), bytes,
                                                        &ltd.image.seg[0]) ||
            (split && !ctx.v_allocs[0]->mapped_ptr_for_host_range(ctx.v_allocs[0]->as_ptr(), bytes,
                                                                  &ltd.image.seg[1]))) {
          return bad(err, PF_ERR_STORAGE, "segment exceeds its pinned allocation");
        }
        ltd.image.seg_allocation_id[0] = ctx.k_allocs[0]->allocation_id();
        if (split) ltd.image.seg_allocation_id[1] = ctx.v_allocs[0]->allocation_id();
      } else {
        // One allocation per block and segment: per-block handles.
        ctx.raw_blocks.reserve(num);
        for (size_t q = 0; q < num; ++q) {
          RawBlock raw;
          if (!ctx.make_raw(q, cfg_.blockwise_alloc, &raw)) {
            return bad(err, PF_ERR_STORAGE, "segment exceeds its pinned allocation");
          }
          ctx.raw_blocks.push_back(std::move(raw));
        }
        ltd.blocks.reserve(num);
        for (size_t q = 0; q < num; ++q) {
          TransferBlock tb;
          tb.block_idx = (*ctx.ids)[q];
          tb.block.raw = &ctx.raw_blocks[q];
          ltd.blocks.push_back(std::move(tb));
        }
      }
      gpu_layers.push_back(std::move(ltd));
    }
  }
  prof.alloc_ms = ms_since(t_phase);

  // ---- Phase 3: one GPU copy task, one synchronisation.  While the bytes
  // move, the blocks that will enter the store are assembled on this thread;
  // nothing becomes visible before the copy has succeeded. ------------------
  t_phase = Clock::now();
  std::future<TaskResult> pending = gpu->worker_pool->batch_save(std::move(gpu_layers));

  struct Assembled {
    BlockKey* key;  // in its SaveList; moved into the store when the block is published
    InflightBlock block;
  };
  std::vector<Assembled> assembled;
  int prep_status = PF_OK;
  std::string prep_err;
  if (!page_first) {
    assembled.reserve(to_save);
    for (size_t li = 0; li < lists.size() && prep_status == PF_OK; ++li) {
      SaveList& l = lists[li];
      if (l.kept.empty()) continue;
      size_t total_slots = 0;
      std::string cause;
      if (!topo->group_total_slots(l.group, &total_slots, &cause)) {
        prep_status = PF_ERR_INVALID_ARGUMENT;
        prep_err = cause;
        break;
      }
      std::vector<SaveLayerCtx*> members;
      for (auto& ctx : ctxs) {
        if (ctx.list == li) members.push_back(&ctx);
      }
      const auto created = Clock::now();
      for (size_t q = 0; q < l.kept.size() && prep_status == PF_OK; ++q) {
        assembled.push_back(Assembled{&l.keys[l.kept[q]], InflightBlock(total_slots, created)});
        InflightBlock& block = assembled.back().block;
        for (SaveLayerCtx* ctx : members) {
          // Built in place; a slot named twice keeps its first block.
          RawBlock* slot = block.empty_slot(ctx->slot_id);
          if (slot == nullptr) continue;
          if (!ctx->make_raw(q, cfg_.blockwise_alloc, slot)) {
            prep_status = PF_ERR_STORAGE;
            prep_err = "segment exceeds its pinned allocation";
            break;
          }
          block.slot_filled();
        }
      }
    }
  }
  prof.assemble_ms = ms_since(t_phase);

  TaskResult res = pending.get();
  prof.transfer_ms = ms_since(t_phase);
  if (res.status != PF_OK) return bad(err, res.status, res.message);
  if (prep_status != PF_OK) return bad(err, prep_status, prep_err);

  // ---- Phase 4: publish -----------------------------------------------------
  t_phase = Clock::now();
  {
    std::lock_guard<std::mutex> lock(mu_);
    if (page_first) {
      const SaveList& l = lists[ctxs[0].list];
      const size_t slot_id = ctxs[0].slot_id;
      size_t page_size = 0;
      topo->shard_page_size(slot_id, &page_size);
      for (size_t b = 0; b < pages.size(); ++b) {
        Segment seg;
        Segment::create(pages[b]->as_ptr(), page_size, pages[b], &seg);
        // Page-first keys carry the raw hash (one group per shard page).
        BlockKey key(ns, std::string(reinterpret_cast<const char*>(l.hashes[l.kept[b]]),
                                     l.lens[l.kept[b]]));
        if (sealed_.find(key) != sealed_.end()) continue;
        auto it = inflight_.find(key);
        if (it == inflight_.end()) {
          it = inflight_.emplace(key, InflightBlock(topo->total_slots())).first;
        } else if (it->second.total_slots() != topo->total_slots()) {
          continue;  // another layout is filling this key: skip it (write_path.rs:147-165)
        }
        if (it->second.insert_slot(slot_id, RawBlock::single_segment(std::move(seg))) ==
            InflightBlock::Insert::Completed) {
          auto sealed_block = it->second.seal();
          inflight_.erase(it);
          seal_insert(std::move(key), std::move(sealed_block));
        }
      }
    } else {
      for (Assembled& a : assembled) {
        BlockKey& key = *a.key;
        // Usually nothing is in flight and the save carries every slot of its
        // blocks: one table operation per block.
        auto it = inflight_.empty() ? inflight_.end() : inflight_.find(key);
        if (it == inflight_.end()) {
          if (a.block.complete()) {
            seal_insert(std::move(key), a.block.seal());  // no-op when sealed meanwhile
          } else if (sealed_.find(key) == sealed_.end()) {
            inflight_.emplace(std::move(key), std::move(a.block));
          }
        } else if (sealed_.find(key) != sealed_.end()) {
          continue;
        } else if (it->second.total_slots() != a.block.total_slots()) {
          // The block in flight was begun by an instance with another slot
          // count (a namespace shared by incompatible layouts): this save's
          // part is dropped, the other one can still complete
          // (write_path.rs:147-165).
          continue;
        } else if (it->second.absorb(std::move(a.block)) == InflightBlock::Insert::Completed) {
          auto sealed_block = it->second.seal();
          inflight_.erase(it);
          seal_insert(std::move(key), std::move(sealed_block));
        }
      }
    }
  }
  prof.publish_ms = ms_since(t_phase);
  prof.total_ms = ms_since(t_begin);
  prof.bytes = res.bytes;
  {
    std::lock_guard<std::mutex> lock(mu_);
    last_save_profile_ = prof;
  }
  return PF_OK;
}

int Engine::query_group_membership(const std::string& instance_id, uint32_t group,
                                   const std::vector<std::string_view>& hashes,
                                   std::vector<uint8_t>* present, std::string* err) {
  auto instance = get_instance(instance_id, err);
  if (!instance) return PF_ERR_INSTANCE_MISSING;
  auto topo = instance->sealed_topology(err);
  if (!topo) return PF_ERR_INVALID_ARGUMENT;
  size_t slots = 0;
  std::string cause;
  if (!topo->group_total_slots(group, &slots, &cause)) return bad(err, PF_ERR_INVALID_ARGUMENT, cause);
  present->assign(hashes.size(), 0);
  std::lock_guard<std::mutex> lock(mu_);
  for (size_t i = 0; i < hashes.size(); ++i) {
    (*present)[i] = find_sealed(instance->ns_id(), hashes[i], group) != nullptr ? 1 : 0;
  }
  return PF_OK;
}

int Engine::query_group_lease(const std::string& instance_id, uint32_t group,
                              const std::vector<std::string_view>& hashes, bool require_all,
                              std::vector<uint8_t>* present, uint64_t* out_lease,
                              std::string* err) {
  auto instance = get_instance(instance_id, err);
  if (!instance) return PF_ERR_INSTANCE_MISSING;
  auto topo = instance->sealed_topology(err);
  if (!topo) return PF_ERR_INVALID_ARGUMENT;
  size_t slots = 0;
  std::string cause;
  if (!topo->group_total_slots(group, &slots, &cause)) return bad(err, PF_ERR_INVALID_ARGUMENT, cause);
  present->assign(hashes.size(), 0);
  *out_lease = 0;
  // Membership and lease under one lock: the blocks that are reported present
  // are the blocks the lease pins (service.rs:606-636 leases the handles the
  // membership query returned; nothing can evict one in between).
  std::lock_guard<std::mutex> lock(mu_);
  sweep_expired_locked();
  Lease lease;
  lease.instance_id = instance_id;
  lease.remaining_consumers = std::max<size_t>(instance->world_size(), 1);
  lease.expires_at = lease_deadline();
  for (size_t i = 0; i < hashes.size(); ++i) {
    SealedEntry* hit = find_sealed(instance->ns_id(), hashes[i], group);
    if (hit == nullptr) continue;
    (*present)[i] = 1;
    lease.blocks.push_back(hit->block);
  }
  if (lease.blocks.empty() || (require_all && lease.blocks.size() != hashes.size())) return PF_OK;
  *out_lease = next_lease_++;
  leases_[*out_lease] = std::move(lease);
  return PF_OK;
}

int Engine::create_group_lease(const std::string& instance_id, uint32_t group,
                               const std::vector<std::string_view>& hashes, uint64_t* out_lease,
                               std::string* err) {
  auto instance = get_instance(instance_id, err);
  if (!instance) return PF_ERR_INSTANCE_MISSING;
  auto topo = instance->sealed_topology(err);
  if (!topo) return PF_ERR_INVALID_ARGUMENT;
  size_t slots = 0;
  std::string cause;
  if (!topo->group_total_slots(group, &slots, &cause)) return bad(err, PF_ERR_INVALID_ARGUMENT, cause);
  if (hashes.empty()) {
    return bad(err, PF_ERR_INVALID_ARGUMENT, "query lease requires at least one block");
  }
  std::lock_guard<std::mutex> lock(mu_);
  sweep_expired_locked();
  Lease lease;
  lease.instance_id = instance_id;
  lease.remaining_consumers = std::max<size_t>(instance->world_size(), 1);
  lease.expires_at = lease_deadline();
  lease.blocks.reserve(hashes.size());
  for (size_t i = 0; i < hashes.size(); ++i) {
    SealedEntry* hit = find_sealed(instance->ns_id(), hashes[i], group);
    if (hit == nullptr) {
      return bad(err, PF_ERR_STORAGE,
                 "block " + std::to_string(i) + " of the lease is not resident in group " +
                     std::to_string(group));
    }
    lease.blocks.push_back(hit->block);
    lru_touch(hit);
  }
  *out_lease = next_lease_++;
  leases_[*out_lease] = std::move(lease);
  return PF_OK;
}

bool Engine::last_load_profile(TaskResult* out) {
  std::vector<std::shared_ptr<InstanceContext>> instances;
  {
    std::lock_guard<std::mutex> lock(mu_);
    for (auto& kv : instances_) instances.push_back(kv.second);
  }
  bool found = false;
  std::chrono::steady_clock::time_point newest;
  for (auto& instance : instances) {
    for (auto& gpu : instance->gpus()) {
      TaskResult r;
      std::chrono::steady_clock::time_point when;
      if (gpu->worker_pool && gpu->worker_pool->last_load(&r, &when) && (!found || when > newest)) {
        found = true;
        newest = when;
        *out = std::move(r);
      }
    }
  }
  return found;
}

uint64_t Engine::staging_bytes() {
  std::vector<std::shared_ptr<InstanceContext>> instances;
  {
    std::lock_guard<std::mutex> lock(mu_);
    for (auto& kv : instances_) instances.push_back(kv.second);
  }
  uint64_t total = 0;
  for (auto& instance : instances) {
    for (auto& gpu : instance->gpus()) {
      if (gpu->worker_pool) total += gpu->worker_pool->staging_bytes();
    }
  }
  return total;
}

SaveProfile Engine::last_save_profile() {
  std::lock_guard<std::mutex> lock(mu_);
  return last_save_profile_;
}

int Engine::query_prefix(const std::string& instance_id,
                         const std::vector<std::string_view>& hashes,
                         uint64_t* out_hits, uint64_t* out_lease, std::string* err) {
  auto instance = get_instance(instance_id, err);
  if (!instance) return PF_ERR_INSTANCE_MISSING;
  std::lock_guard<std::mutex> lock(mu_);
  sweep_expired_locked();
  Lease lease;
  lease.instance_id = instance_id;
  lease.remaining_consumers = std::max<size_t>(instance->world_size(), 1);
  lease.expires_at = lease_deadline();
  lease.blocks.reserve(hashes.size());
  for (std::string_view h : hashes) {
    SealedEntry* hit = find_sealed(instance->ns_id(), h, 0);
    if (hit == nullptr) break;
    lease.blocks.push_back(hit->block);
    lru_touch(hit);  // most recently used
  }
  *out_hits = lease.blocks.size();
  *out_lease = 0;
  if (!lease.blocks.empty()) {
    *out_lease = next_lease_++;
    leases_[*out_lease] = std::move(lease);
  }
  return PF_OK;
}

bool Engine::release_query_lease(uint64_t lease) {
  std::lock_guard<std::mutex> lock(mu_);
  sweep_expired_locked();
  return leases_.erase(lease) > 0;
}

int Engine::batch_load_kv_blocks_multi_layer(
    const std::string& instance_id, size_t tp_rank, int device_id,
    const std::vector<std::vector<std::string>>& layer_groups,
    const std::vector<LoadRequest>& loads, const std::string& load_state_shm,
    std::future<TaskResult>* out, std::string* err) {
  const auto t_resolve = std::chrono::steady_clock::now();
  auto instance = get_instance(instance_id, err);
  if (!instance) return PF_ERR_INSTANCE_MISSING;
  auto topo = instance->sealed_topology(err);
  if (!topo) return PF_ERR_INVALID_ARGUMENT;
  auto gpu = instance->get_gpu(device_id);
  if (!gpu) {
    return bad(err, PF_ERR_WORKER_MISSING,
               "device " + std::to_string(device_id) + " not found in instance " + instance_id);  // lib.rs:93-95
  }
  if (layer_groups.empty()) {
    return bad(err, PF_ERR_INVALID_ARGUMENT, "load requires at least one layer group");
  }
  size_t layer_count = 0;
  std::set<std::string> unique;
  for (auto& g : layer_groups) {
    layer_count += g.size();
    unique.insert(g.begin(), g.end());
  }
  if (unique.size() != layer_count) {
    return bad(err, PF_ERR_INVALID_ARGUMENT, "load layer names must be unique across groups");
  }
  // Each load group maps to exactly one storage group (lib.rs:748-770).
  std::vector<int64_t> storage_group(layer_groups.size(), -1);
  for (size_t gi = 0; gi < layer_groups.size(); ++gi) {
    for (const std::string& name : layer_groups[gi]) {
      size_t id = 0;
      std::string cause;
      if (!topo->layer_id(name, &id, &cause)) return bad(err, PF_ERR_INVALID_ARGUMENT, cause);
      int64_t g = topo->group_of_layer(id);
      if (storage_group[gi] >= 0 && storage_group[gi] != g) {
        return bad(err, PF_ERR_INVALID_ARGUMENT,
                   "load group mixes storage groups " + std::to_string(storage_group[gi]) +
                       " and " + std::to_string(g) + " (layer " + name + ")");
      }
      storage_group[gi] = g;
    }
  }
  // Consume the leases.
  std::vector<std::vector<std::pair<uint64_t, size_t>>> targets(layer_groups.size());
  std::vector<std::shared_ptr<SealedBlock>> block_cache;
  for (const LoadRequest& lr : loads) {
    std::vector<std::shared_ptr<SealedBlock>> blocks;
    {
      std::lock_guard<std::mutex> lock(mu_);
      // lease.rs:105-134.
      sweep_expired_locked();
      auto it = leases_.find(lr.lease);
      if (it == leases_.end()) {
        return bad(err, PF_ERR_STORAGE, "query lease is unknown or expired");
      }
      if (it->second.instance_id != instance_id) {
        return bad(err, PF_ERR_STORAGE,
                   "query lease belongs to instance " + it->second.instance_id + ", got " +
                       instance_id);
      }
      if (it->second.remaining_consumers > 1) {
        --it->second.remaining_consumers;
        blocks = it->second.blocks;
      } else {
        blocks = std::move(it->second.blocks);
        leases_.erase(it);
      }
    }
    if (lr.block_ids_by_group.size() != layer_groups.size()) {
      return bad(err, PF_ERR_INVALID_ARGUMENT,
                 "load group count " + std::to_string(lr.block_ids_by_group.size()) +
                     " does not match layer group count " + std::to_string(layer_groups.size()));
    }
    const size_t start = block_cache.size();
    for (size_t gi = 0; gi < layer_groups.size(); ++gi) {
      const auto& ids = lr.block_ids_by_group[gi];
      if (blocks.size() != ids.size()) {
        return bad(err, PF_ERR_INVALID_ARGUMENT,
                   "query lease block count " + std::to_string(blocks.size()) +
                       " does not match destination block count " + std::to_string(ids.size()) +
                       " for group " + std::to_string(gi));
      }
      if (storage_group[gi] >= 0) {
        size_t expected = 0;
        std::string cause;
        if (!topo->group_total_slots(static_cast<uint32_t>(storage_group[gi]), &expected, &cause)) {
          return bad(err, PF_ERR_INVALID_ARGUMENT, cause);
        }
        for (size_t si = 0; si < ids.size(); ++si) {
          if (ids[si] >= 0 && blocks[si]->num_slots() != expected) {
            return bad(err, PF_ERR_INVALID_ARGUMENT,
                       "stored block has " + std::to_string(blocks[si]->num_slots()) +
                           " slots but storage group " + std::to_string(storage_group[gi]) +
                           " of instance " + instance_id + " expects " + std::to_string(expected) +
                           ": namespace is shared by incompatible KV layouts");
          }
        }
      }
      for (size_t si = 0; si < ids.size(); ++si) {
        if (ids[si] >= 0) targets[gi].emplace_back(static_cast<uint64_t>(ids[si]), start + si);
      }
    }
    block_cache.insert(block_cache.end(), std::make_move_iterator(blocks.begin()),
                       std::make_move_iterator(blocks.end()));
  }
  // One LayerTransferData per layer.
  struct PageList {
    std::shared_ptr<std::vector<MappedPinnedPtr>> pages;
    std::shared_ptr<std::vector<uint64_t>> alloc_ids;
    std::shared_ptr<std::vector<uint32_t>> ids;
    uint64_t page_len = 0;
  };
  std::map<std::pair<size_t, size_t>, PageList> page_lists;
  const bool page_first = topo->is_page_first();
  std::vector<LayerTransferData> layers;
  for (size_t gi = 0; gi < layer_groups.size(); ++gi) {
    for (const std::string& name : layer_groups[gi]) {
      size_t layer_id = 0;
      topo->layer_id(name, &layer_id, nullptr);
      auto lit = gpu->reg.kv_caches.find(name);
      if (lit == gpu->reg.kv_caches.end()) {
        return bad(err, PF_ERR_INVALID_ARGUMENT,
                   "layer " + name + " not registered on device " + std::to_string(device_id));
      }
      size_t slot_id = 0;
      std::string cause;
      if (!topo->slot_index(layer_id, tp_rank, &slot_id, &cause)) {
        return bad(err, PF_ERR_INVALID_ARGUMENT, cause);
      }
      size_t host_offset = 0, unused = 0;
      if (!topo->page_placement(layer_id, &host_offset, &unused)) host_offset = 0;
      LayerTransferData ltd;
      ltd.layer_name = name;
      ltd.layout = lit->second;
      if (page_first && !targets[gi].empty()) {
        // Every layer of a shard reads the same pages at its own offset: one
        // shared page list per (group, slot) instead of per-block handles.
        PageList& pl = page_lists[{gi, slot_id}];
        if (!pl.pages) {
          auto pages = std::make_shared<std::vector<MappedPinnedPtr>>();
          auto alloc_ids = std::make_shared<std::vector<uint64_t>>();
          auto ids = std::make_shared<std::vector<uint32_t>>();
          uint64_t page_len = UINT64_MAX;
          for (auto& t : targets[gi]) {
            const RawBlock* raw = block_cache[t.second]->get_slot(slot_id);
            MappedPinnedPtr p;
            if (!raw || !raw->segment_mapped_ptr(0, &p)) {
              return bad(err, PF_ERR_INVALID_ARGUMENT,
                         "stored block is missing slot " + std::to_string(slot_id) +
                             " for layer " + name);
            }
            pages->push_back(p);
            alloc_ids->push_back(raw->segment_allocation_id(0));
            ids->push_back(static_cast<uint32_t>(t.first));
            page_len = std::min(page_len, raw->segment_size(0));
          }
          pl.pages = std::move(pages);
          pl.alloc_ids = std::move(alloc_ids);
          pl.ids = std::move(ids);
          pl.page_len = page_len;
        }
        ltd.image.kind = HostImage::Kind::Paged;
        ltd.image.block_ids = pl.ids;
        ltd.image.pages = pl.pages;
        ltd.image.page_allocation_ids = pl.alloc_ids;
        ltd.image.offset = host_offset;
        ltd.image.page_len = pl.page_len;
        layers.push_back(std::move(ltd));
        continue;
      }
      ltd.blocks.reserve(targets[gi].size());
      for (auto& t : targets[gi]) {
        const auto& sealed = block_cache[t.second];
        const RawBlock* raw = sealed->get_slot(slot_id);
        if (!raw) {
          return bad(err, PF_ERR_INVALID_ARGUMENT,
                     "stored block is missing slot " + std::to_string(slot_id) + " for layer " +
                         name);
        }
        TransferBlock tb;
        tb.block_idx = t.first;
        tb.block.raw = raw;
        tb.block.offset = host_offset;
        ltd.blocks.push_back(std::move(tb));
      }
      if (!ltd.blocks.empty()) layers.push_back(std::move(ltd));
    }
  }
  // The leased blocks stay alive through the first layer of the task.
  if (!layers.empty()) {
    layers.front().keep.reserve(block_cache.size());
    for (auto& b : block_cache) layers.front().keep.push_back(std::move(b));
  }
  if (layers.empty()) {
    // Nothing to load: complete at once (lib.rs:885-890).
    std::promise<TaskResult> p;
    p.set_value(TaskResult());
    *out = p.get_future();
    if (!load_state_shm.empty()) {
      std::string aerr;
      if (auto ls = LoadState::attach(load_state_shm, &aerr)) ls->set_completed();
    }
    return PF_OK;
  }
  LoadCompletion completion;
  completion.load_state_shm = load_state_shm;
  completion.resolve_ms = std::chrono::duration<double, std::milli>(
                              std::chrono::steady_clock::now() - t_resolve).count();
  *out = gpu->worker_pool->submit_load(std::move(layers), std::move(completion));
  return PF_OK;
}

}  // namespace pf
