// Per-GPU worker pair: one load thread and one save thread, each with its own
// stream and transfer engine, processing tasks serially with one
// synchronisation per task.  Follows pegaflow-core/src/gpu_worker.rs:15-523 of
// the reference.
#pragma once

#include <hip/hip_runtime.h>

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

// gpu_worker.rs:54-59.
struct LayerTransferData {
  std::string layer_name;
  KVCacheLayout layout;
  std::vector<TransferBlock> blocks;
};

// Result of a task: status code (PF_OK or an error class) and message.
struct TaskResult {
  int status = 0;
  std::string message;
  uint64_t bytes = 0;
  double elapsed_ms = 0;
};

// gpu_worker.rs:29-52: how a finished load reports back.  Shm = a LoadState
// object the submitter polls; the future is always fulfilled as well.
struct LoadCompletion {
  std::string load_state_shm;  // empty = none
};

class Xfer;

class GpuWorkerPool {
 public:
  // gpu_worker.rs:131-201.  `use_descriptor_backends` makes the workers build
  // one descriptor per fragment and submit them to the reference-compatible
  // backend of `mode`; otherwise they use the block-ID engine, with `mode`
  // choosing the link path (Direct = staged when possible, Kernel = zero-copy).
  static std::unique_ptr<GpuWorkerPool> spawn(int device_id, NumaNode numa_node, TransferMode mode,
                                              bool use_descriptor_backends, std::string* err,
                                              int* status);
  ~GpuWorkerPool();
  // gpu_worker.rs:204-212: fire and forget; the future (and the LoadState, if
  // named) is signalled when the task settles.
  std::future<TaskResult> submit_load(std::vector<LayerTransferData> layers,
                                      LoadCompletion completion);
  // gpu_worker.rs:216-243.
  std::future<TaskResult> batch_save(std::vector<LayerTransferData> layers);
  int device_id() const { return device_id_; }

 private:
  struct Task {
    std::vector<LayerTransferData> layers;
    LoadCompletion completion;
    std::promise<TaskResult> reply;
  };
  struct Worker {
    std::thread thread;
    std::mutex mu;
    std::condition_variable cv;
    std::deque<std::unique_ptr<Task>> queue;
    bool stop = false;
  };
  GpuWorkerPool() = default;
  void run(Worker* w, bool is_load, NumaNode numa, std::promise<TaskResult>* ready);
  std::future<TaskResult> push(Worker* w, std::unique_ptr<Task> t);

  int device_id_ = 0;
  TransferMode mode_ = TransferMode::Direct;
  bool use_descriptors_ = false;
  Worker load_;
  Worker save_;
};

// gpu_worker.rs:353-423 over the C++ types (the C-ABI form is pf_build_copy_descs).
bool build_copy_descs(const std::vector<LayerTransferData>& layers, std::vector<CopyDesc>* out,
                      uint64_t* total_bytes, std::string* err);

}  // namespace pf
