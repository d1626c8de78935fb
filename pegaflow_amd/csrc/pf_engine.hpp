// Save / load by block ID over the transfer path: registration, host image
// construction, submission to the per-GPU workers, and the minimal block
// store the cycle needs.  Follows the parts of PegaEngine that sit on the
// path (pegaflow-core/src/lib.rs:228-440,654-898, offload.rs:182-659,
// instance.rs:293-478,680-860 of the reference).  The cache policy behind
// the reference's StorageEngine (TinyLFU/LRU, SSD, RDMA, prefetch) is not
// reproduced: blocks are kept until evicted oldest-first under pool pressure.
#pragma once

#include <chrono>
#include <cstdint>
#include <future>
#include <list>
#include <map>
#include <unordered_map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "pf_block.hpp"
#include "pf_pool.hpp"
#include "pf_topology.hpp"
#include "pf_worker.hpp"

namespace pf {

struct EngineConfig {
  uint64_t pool_size = 0;
  bool use_hugepages = false;
  bool numa_aware = false;        // one pool per NUMA node that has a GPU
  uint32_t pool_shards = 1;
  bool blockwise_alloc = false;   // one pinned allocation per block instead of per layer
  bool ssd_enabled = false;       // pad host strides to 512 B; regular (CPU-readable) backing
  bool use_descriptor_backends = false;  // workers use per-fragment descriptors + backends
  uint64_t unit_size_hint = 0;
  // lease.rs:11: a lease that nobody consumes stops pinning its blocks after this long.
  uint64_t lease_ttl_ms = 600000;
  // PF_PATH_AUTO threshold of the workers' transfer engines; 0 = the engine's default.
  uint64_t auto_staged_min_bytes = 0;
  // Upper bound of one staging slot of a worker (0 = 512 MiB).  A context's
  // pool holds 2 workers x 2 slots of min(this, what its layers can fill).
  uint64_t staging_slot_bytes = 0;
  // Workers allocate their staging on the first staged task, not at registration.
  bool lazy_staging = false;
  bool side_copy_streams = false;
  // Registrations that ask for TransferMode::Kernel get zero-copy workers (the
  // reference's meaning of that mode: one copy kernel over mapped host memory,
  // gpu_worker.rs:264-276) instead of the per-task choice.
  bool kernel_mode_zerocopy = false;
};

// block.rs:20-25, as a view of the caller's arrays (valid for the call).
struct LayerSaveView {
  const char* layer_name = nullptr;
  const uint64_t* block_ids = nullptr;
  size_t n_ids = 0;
  const uint8_t* const* hashes = nullptr;
  const uint32_t* hash_lens = nullptr;
  size_t n_hashes = 0;
};

// Where the time of the last successful save went (offload.rs:560-574 records
// the same phases as metrics).  assemble_ms runs inside transfer_ms.
struct SaveProfile {
  double validate_ms = 0, filter_ms = 0, alloc_ms = 0, assemble_ms = 0, transfer_ms = 0,
         publish_ms = 0, total_ms = 0;
  uint64_t bytes = 0;
};

// One lease's destinations: per load group, one entry per leased block; -1 = skip.
struct LoadRequest {
  uint64_t lease = 0;
  std::vector<std::vector<int64_t>> block_ids_by_group;
};

// instance.rs:293-378.
struct GpuContext {
  WorkerRegistration reg;
  NumaNode preferred_numa;
  std::unique_ptr<GpuWorkerPool> worker_pool;
};

// instance.rs:380-478,680-860.
class InstanceContext {
 public:
  InstanceContext(std::string id, std::string ns, uint32_t ns_id, size_t tp_size,
                  size_t world_size, bool page_first)
      : id_(std::move(id)), ns_(std::move(ns)), ns_id_(ns_id), tp_size_(tp_size),
        world_size_(world_size), page_first_(page_first) {}
  int register_new_gpu(std::shared_ptr<GpuContext> ctx, std::string* err);
  // Fails while workers are still registering.
  std::shared_ptr<LayerTopology> sealed_topology(std::string* err);
  std::shared_ptr<GpuContext> get_gpu(int device_id);
  std::vector<std::shared_ptr<GpuContext>> gpus();
  std::string verify_topology(size_t tp_size, size_t world_size, bool page_first) const;
  const std::string& id() const { return id_; }
  const std::string& ns() const { return ns_; }
  // The engine's number for the namespace: what block keys carry.
  uint32_t ns_id() const { return ns_id_; }
  size_t tp_size() const { return tp_size_; }
  size_t world_size() const { return world_size_; }
  // Validation that must precede the (expensive) GPU context construction.
  int check_accepting(int device_id, size_t tp_rank, std::string* err);

 private:
  std::string id_, ns_;
  uint32_t ns_id_;
  size_t tp_size_, world_size_;
  bool page_first_;
  std::mutex mu_;
  std::map<int, std::shared_ptr<GpuContext>> gpus_;
  std::shared_ptr<LayerTopology> topology_;
};

class Engine {
 public:
  static std::unique_ptr<Engine> create(const EngineConfig& cfg, std::string* err, int* status);
  ~Engine();

  // lib.rs:302-440.
  int register_context_layer_batch_strided(
      const std::string& instance_id, const std::string& ns, int device_id, size_t tp_rank,
      size_t pp_rank, size_t tp_size, size_t world_size, const std::vector<std::string>& layer_names,
      const std::vector<uint64_t>& data_ptrs, const std::vector<uint64_t>& size_bytes,
      const std::vector<uint64_t>& num_blocks, const std::vector<uint64_t>& bytes_per_block,
      const std::vector<uint64_t>& kv_stride_bytes, const std::vector<uint64_t>& segments,
      const std::vector<uint64_t>* block_stride_bytes, const std::vector<uint32_t>* layer_group_ids,
      TransferMode mode, bool page_first, std::string* err);
  // lib.rs:443-457.
  int unregister_instance(const std::string& instance_id, std::string* err);
  // offload.rs:293-659.  Returns once the bytes are in host memory and the
  // blocks are queryable.
  int batch_save_kv_blocks(const std::string& instance_id, size_t tp_rank, size_t pp_rank,
                           int device_id, const std::vector<LayerSaveView>& saves, std::string* err);
  SaveProfile last_save_profile();
  // The load task that settled last on any of the engine's worker pools (what
  // the reference logs per load, gpu_worker.rs:458-474, plus its phases); false
  // when none has.
  bool last_load_profile(TaskResult* out);
  // Device memory the worker pools of all registered contexts hold for staging.
  uint64_t staging_bytes();
  // Longest cached prefix of `hashes` (group 0 keys) + a lease over those
  // blocks (lib.rs:506-546,614-629).
  int query_prefix(const std::string& instance_id, const std::vector<std::string_view>& hashes,
                   uint64_t* out_hits, uint64_t* out_lease, std::string* err);
  // lib.rs:593-611: per-position membership of `hashes` in one storage group
  // (no prefix rule, no lease).  An unknown group is an error.
  int query_group_membership(const std::string& instance_id, uint32_t group,
                             const std::vector<std::string_view>& hashes,
                             std::vector<uint8_t>* present,
                             std::string* err);
  // lib.rs:614-628 over hashes instead of block handles: a lease that pins the
  // sealed blocks of exactly these hashes in `group`.  Fails when one of them
  // is not resident (it may have been evicted since the membership query).
  int create_group_lease(const std::string& instance_id, uint32_t group,
                         const std::vector<std::string_view>& hashes, uint64_t* out_lease,
                         std::string* err);
  // The two above in one step, under one lock (service.rs:606-636): which of
  // `hashes` are sealed in `group`, and a lease over exactly those blocks in
  // that order (*out_lease = 0 when none is, or when `require_all` and one is
  // missing).
  int query_group_lease(const std::string& instance_id, uint32_t group,
                        const std::vector<std::string_view>& hashes, bool require_all,
                        std::vector<uint8_t>* present, uint64_t* out_lease, std::string* err);
  bool release_query_lease(uint64_t lease);
  // The periodic sweep of the reference's lease manager (lease.rs:66-80), for
  // the embedder's timer: drops expired leases, returns how many.
  size_t sweep_expired_leases();
  size_t live_leases();
  // lib.rs:654-898.  On success *out is fulfilled when the load settles (at
  // once when nothing is to be loaded).
  int batch_load_kv_blocks_multi_layer(const std::string& instance_id, size_t tp_rank,
                                       int device_id,
                                       const std::vector<std::vector<std::string>>& layer_groups,
                                       const std::vector<LoadRequest>& loads,
                                       const std::string& load_state_shm,
                                       std::future<TaskResult>* out, std::string* err);
  void pool_usage(uint64_t* used, uint64_t* total) { pool_->usage(used, total); }
  size_t cached_blocks();
  // Blocks that have some but not all of their slots.
  size_t inflight_blocks();
  // Drop the incomplete blocks older than `max_age`; returns how many.
  size_t gc_stale_inflight(std::chrono::milliseconds max_age);
  // Test hook / pressure valve: drop every sealed block that is not leased.
  size_t evict_all();

 private:
  Engine() { lru_reset(); }
  std::shared_ptr<InstanceContext> get_instance(const std::string& id, std::string* err);
  // storage/mod.rs:294-330: allocate, evicting oldest sealed blocks on pressure.
  std::shared_ptr<PinnedAllocation> allocate(uint64_t size, NumaNode numa);
  bool evict_one();
  int alloc_page_first_targets(const LayerTopology& topo, struct SaveLayerCtx* ctxs, size_t n,
                               NumaNode numa, std::vector<std::shared_ptr<PinnedAllocation>>* pages,
                               std::vector<LayerTransferData>* out, std::string* err);

  EngineConfig cfg_;
  std::unique_ptr<PinnedAllocator> pool_;
  NumaTopology numa_;
  std::mutex mu_;  // instances, store, leases
  std::map<std::string, std::shared_ptr<InstanceContext>> instances_;
  std::map<std::string, uint32_t> ns_ids_;  // namespace name -> the number in block keys
  uint32_t ns_id_locked(const std::string& ns);
  std::unordered_map<BlockKey, InflightBlock, BlockKeyHash, BlockKeyEqual> inflight_;
  // The read cache: sealed blocks in least-recently-used order (a prefix query
  // makes its hits the most recently used), storage/mod.rs:482-554 and
  // storage/read_cache.rs of the reference without its admission policy.  The
  // order is a ring threaded through the table's own entries (their addresses
  // do not change while they are in the table), so making a block the most
  // recently used touches no allocator.
  struct SealedEntry {
    std::shared_ptr<SealedBlock> block;
    const BlockKey* key = nullptr;  // the table's copy of the key
    SealedEntry* older = nullptr;
    SealedEntry* newer = nullptr;
  };
  using SealedTable = std::unordered_map<BlockKey, SealedEntry, BlockKeyHash, BlockKeyEqual>;
  SealedTable sealed_;
  // Ring head: lru_.newer is the least recently used entry, lru_.older the most.
  SealedEntry lru_;
  void lru_reset() { lru_.older = lru_.newer = &lru_; }
  static void lru_unlink(SealedEntry* e) {
    e->older->newer = e->newer;
    e->newer->older = e->older;
  }
  void lru_make_newest(SealedEntry* e) {
    e->older = lru_.older;
    e->newer = &lru_;
    lru_.older->newer = e;
    lru_.older = e;
  }
  void lru_touch(SealedEntry* e) {
    lru_unlink(e);
    lru_make_newest(e);
  }
  // The sealed entry of (namespace, group-encoded hash), or null; mu_ held.
  SealedEntry* find_sealed(uint32_t ns, std::string_view hash, uint32_t group);
  // Enters a block under `key` unless the key is sealed already; mu_ held.
  bool seal_insert(BlockKey&& key, std::shared_ptr<SealedBlock> block);
  // lease.rs:40-134: a lease serves one load per worker of the instance's
  // world size, then disappears.
  struct Lease {
    std::string instance_id;
    std::vector<std::shared_ptr<SealedBlock>> blocks;
    size_t remaining_consumers = 1;
    std::chrono::steady_clock::time_point expires_at;  // lease.rs:47
  };
  std::map<uint64_t, Lease> leases_;
  uint64_t next_lease_ = 1;
  // lease.rs:91-118,174-181: drop the leases whose time is up; runs (mu_ held)
  // whenever a lease is created, consumed or released, before an allocation
  // gives up, and from sweep_expired_leases().  Returns how many went.
  size_t sweep_expired_locked();
  std::chrono::steady_clock::time_point lease_deadline() const {
    return std::chrono::steady_clock::now() + std::chrono::milliseconds(cfg_.lease_ttl_ms);
  }
  SaveProfile last_save_profile_;
};

}  // namespace pf
