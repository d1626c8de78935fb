// Per-GPU worker pair: one load thread and one save thread, each with its own
// stream and transfer engine, processing tasks serially with one
// synchronisation per task.  Follows pegaflow-core/src/gpu_worker.rs:15-523 of
// the reference.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <deque>
#include <functional>
#include <future>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "pf_block.hpp"
#include "pf_layout.hpp"
#include "pf_numa.hpp"
#include "pf_transfer.hpp"

namespace pf {

// gpu_worker.rs:61-94: the host image of one block in a transfer.  `raw`
// points at a block owned by the task (save) or at a slot of a cached sealed
// block kept alive by `keep` (load); `offset` is the page-first byte offset.
struct HostBlock {
  const RawBlock* raw = nullptr;
  std::shared_ptr<const void> keep;
  uint64_t offset = 0;
};

// gpu_worker.rs:96-101.
struct TransferBlock {
  uint64_t block_idx = 0;
  HostBlock block;
};

// The host side of a whole layer when it is regular, so that a task of
// hundreds of thousands of fragments needs no per-block handle.  It describes
// exactly the blocks a list of TransferBlocks over the same memory would:
//   Uniform: list position i at seg[s] + i * stride (the batch image of a
//            save: one K buffer and one V buffer, or one block buffer);
//   Paged:   list position i at pages[i] + offset, V right behind K (one page
//            or one allocation per block).
struct HostImage {
  enum class Kind { None, Uniform, Paged };
  Kind kind = Kind::None;
  std::shared_ptr<const std::vector<uint32_t>> block_ids;  // device block of each position
  MappedPinnedPtr seg[2];
  uint64_t seg_allocation_id[2] = {0, 0};
  uint64_t stride = 0;
  std::shared_ptr<const std::vector<MappedPinnedPtr>> pages;
  std::shared_ptr<const std::vector<uint64_t>> page_allocation_ids;
  uint64_t offset = 0;
  uint64_t page_len = 0;
  std::vector<std::shared_ptr<const void>> keep;  // what owns the memory
  size_t size() const { return block_ids ? block_ids->size() : 0; }
};

// gpu_worker.rs:54-59.  Either `blocks` (one handle per block) or `image`.
struct LayerTransferData {
  std::string layer_name;
  KVCacheLayout layout;
  std::vector<TransferBlock> blocks;
  HostImage image;
  // Owners of the host memory for the whole layer (or task), for callers that
  // would otherwise repeat one owner in every block's `keep`.
  std::vector<std::shared_ptr<const void>> keep;
};

// Result of a task: status code (PF_OK or an error class) and message, then
// what the reference's workers log per task (bytes, duration;
// gpu_worker.rs:458-474,505-520) and where the time went, phase by phase (the
// fields of pf_task_result).
struct TaskResult {
  int status = 0;
  std::string message;
  uint64_t bytes = 0;
  double elapsed_ms = 0;
  uint32_t paths = 0;  // PF_TASK_PATH_* bits
  uint32_t staged_groups = 0, zero_copy_launches = 0, link_copies = 0;
  double resolve_ms = 0;  // filled by the engine for loads
  double queue_ms = 0, convert_ms = 0, plan_ms = 0, staging_alloc_ms = 0, enqueue_ms = 0,
         sync_ms = 0, device_first_ms = 0, device_ms = 0;
};

// What a pool's workers are given besides device, NUMA node and mode.
struct WorkerPoolOptions {
  bool use_descriptor_backends = false;
  // A task whose dense layers add up to this much is staged (0 = 8 MiB).
  uint64_t auto_staged_min_bytes = 0;
  // Size of one staging slot; each worker of a staging pool holds two
  // (0 = the transfer engine's default, 512 MiB).
  uint64_t staging_slot_bytes = 0;
  // false: both workers allocate their slots when the pool is spawned, so no
  // task pays for it; true: a worker allocates on its first staged task.
  bool lazy_staging = false;
  bool side_copy_streams = false;  // link copies on a second stream per worker instead of in order
};

// gpu_worker.rs:29-52: how a finished load reports back.  Shm = a LoadState
// object the submitter polls; the future is always fulfilled as well.
struct LoadCompletion {
  std::string load_state_shm;  // empty = none
  // What the submitter spent turning leases into host blocks; travels with the
  // task so that its result tells the whole load.
  double resolve_ms = 0;
};

class Xfer;

class GpuWorkerPool {
 public:
  // gpu_worker.rs:131-201.  `use_descriptor_backends` makes the workers build
  // one descriptor per fragment and submit them to the reference-compatible
  // backend of `mode`; otherwise they use the block-ID engine, with `mode`
  // choosing the link path (Direct = staged when possible, Kernel = zero-copy).
  static std::unique_ptr<GpuWorkerPool> spawn(int device_id, NumaNode numa_node, TransferMode mode,
                                              const WorkerPoolOptions& options, std::string* err,
                                              int* status);
  ~GpuWorkerPool();
  // gpu_worker.rs:204-212: fire and forget; the future (and the LoadState, if
  // named) is signalled when the task settles.
  std::future<TaskResult> submit_load(std::vector<LayerTransferData> layers,
                                      LoadCompletion completion);
  // gpu_worker.rs:216-243.
  std::future<TaskResult> batch_save(std::vector<LayerTransferData> layers);
  int device_id() const { return device_id_; }
  // Pairs among {this pool's two streams, the idle worker streams of the other
  // pools on the device that were probed} whose kernels did NOT run side by
  // side when the pool was spawned: 0 = every worker stream probed has a
  // hardware queue of its own.
  size_t queue_clashes() const { return queue_clashes_; }
  // Device memory the two workers hold for staging right now.
  uint64_t staging_bytes() const { return staging_bytes_.load(); }
  // The last load task this pool settled (status != 0 included) and when, on
  // the steady clock; false when it has settled none.
  bool last_load(TaskResult* out, std::chrono::steady_clock::time_point* when);

 private:
  struct Task {
    std::vector<LayerTransferData> layers;
    LoadCompletion completion;
    std::promise<TaskResult> reply;
    std::chrono::steady_clock::time_point submitted;
  };
  struct Worker {
    std::thread thread;
    std::mutex mu;
    std::condition_variable cv;
    std::deque<std::unique_ptr<Task>> queue;
    bool stop = false;
    hipStream_t stream = nullptr;  // set by the worker before it reports ready
    hipStream_t side = nullptr;    // link copies, with WorkerPoolOptions::side_copy_streams
  };
  // One large copy in each direction, in flight together, before the first task.
  void prime_copy_overlap();
  // Make sure the two workers' streams execute kernels concurrently.
  void separate_worker_queues();
  GpuWorkerPool() = default;
  void run(Worker* w, bool is_load, NumaNode numa, std::promise<TaskResult>* ready);
  std::future<TaskResult> push(Worker* w, std::unique_ptr<Task> t);

  int device_id_ = 0;
  TransferMode mode_ = TransferMode::Direct;
  WorkerPoolOptions options_;
  std::atomic<uint64_t> staging_bytes_{0};
  std::mutex last_load_mu_;
  bool has_last_load_ = false;
  TaskResult last_load_;
  std::chrono::steady_clock::time_point last_load_when_;
  Worker load_;
  Worker save_;
  size_t queue_clashes_ = 0;
  // Buffers of prime_copy_overlap, kept until the pool goes: freeing device or
  // pinned memory synchronises the whole device, and a pool is spawned while
  // other instances transfer.
  void* prime_host_ = nullptr;
  void* prime_dev_ = nullptr;
};

// Worker streams of the live pools on `device` and how many pairs of them share
// a hardware queue right now (kernels of the two do not overlap).  Streams that
// are busy are left out of the probe and counted in *out_skipped.
int worker_stream_report(int device, size_t* out_streams, size_t* out_clashing_pairs,
                         size_t* out_skipped);

// gpu_worker.rs:353-423 over the C++ types (the C-ABI form is pf_build_copy_descs).
// Layers [begin, end) only when end > begin; the whole task otherwise.
bool build_copy_descs(const std::vector<LayerTransferData>& layers, std::vector<CopyDesc>* out,
                      uint64_t* total_bytes, std::string* err, size_t begin = 0, size_t end = 0);

}  // namespace pf
