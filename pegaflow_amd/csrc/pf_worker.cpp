#include "pf_worker.hpp"

#include <chrono>
#include <cstring>

#include "pf_common.hpp"
#include "pf_sync_state.hpp"
#include "pf_xfer.hpp"

namespace pf {

bool build_copy_descs(const std::vector<LayerTransferData>& layers, std::vector<CopyDesc>* out,
                      uint64_t* total_bytes, std::string* err) {
  out->clear();
  uint64_t total = 0;
  for (size_t li = 0; li < layers.size(); ++li) {
    const LayerTransferData& layer = layers[li];
    for (const TransferBlock& tb : layer.blocks) {
      BlockCopies bc;
      std::string cause;
      if (!layer.layout.block_copies(tb.block_idx, &bc, &cause)) {
        *err = "layer " + layer.layer_name + ": " + cause;
        return false;
      }
      const RawBlock* raw = tb.block.raw;
      MappedPinnedPtr k;
      if (!raw || !raw->segment_mapped_ptr(0, &k)) {
        *err = "layer " + layer.layer_name + ": host block has no segment 0";
        return false;
      }
      k = k.add(tb.block.offset);
      if (bc.n == 2) {
        MappedPinnedPtr v;
        uint64_t v_alloc;
        if (raw->segment_mapped_ptr(1, &v)) {
          v = v.add(tb.block.offset);
          v_alloc = raw->segment_allocation_id(1);
        } else {
          v = k.add(bc.k.bytes);  // single-segment host block: V follows K
          v_alloc = raw->segment_allocation_id(0);
        }
        out->push_back({bc.k.addr, k.host, reinterpret_cast<uint64_t>(k.device), bc.k.bytes, li,
                        raw->segment_allocation_id(0)});
        out->push_back({bc.v.addr, v.host, reinterpret_cast<uint64_t>(v.device), bc.v.bytes, li,
                        v_alloc});
        total += bc.k.bytes + bc.v.bytes;
      } else {
        out->push_back({bc.k.addr, k.host, reinterpret_cast<uint64_t>(k.device), bc.k.bytes, li,
                        raw->segment_allocation_id(0)});
        total += bc.k.bytes;
      }
    }
  }
  if (total_bytes) *total_bytes = total;
  return true;
}

namespace {

// Storage for one task's block-ID form.
struct BlockForm {
  std::vector<pf_layer_blocks> layers;
  std::vector<std::vector<uint32_t>> ids;
  std::vector<std::vector<uint64_t>> page_host;
  std::vector<std::vector<uint64_t>> page_dev;
  uint64_t total_bytes = 0;
};

// Express the task through block ids: per layer either a uniform-stride host
// image or a per-block base table.  Returns false when some layer fits
// neither form (e.g. K and V of each block in unrelated allocations); the
// caller then falls back to per-fragment descriptors.  Errors are reported
// through *err with *failed = true.
bool to_block_form(const std::vector<LayerTransferData>& layers, BlockForm* out, bool* failed,
                   std::string* err) {
  *failed = false;
  const size_t n_layers = layers.size();
  out->layers.resize(n_layers);
  out->ids.resize(n_layers);
  out->page_host.resize(n_layers);
  out->page_dev.resize(n_layers);
  for (size_t li = 0; li < n_layers; ++li) {
    const LayerTransferData& layer = layers[li];
    pf_layer_blocks& lb = out->layers[li];
    std::memset(&lb, 0, sizeof(lb));
    lb.layer_name = layer.layer_name.c_str();
    lb.layout = layer.layout.c();
    const size_t n = layer.blocks.size();
    lb.n_blocks = n;
    if (n == 0) continue;
    const bool split = layer.layout.is_split();
    const uint64_t frag = layer.layout.fragment_bytes();
    std::vector<uint32_t>& ids = out->ids[li];
    ids.resize(n);
    std::vector<MappedPinnedPtr> k(n), v(n);
    for (size_t i = 0; i < n; ++i) {
      const TransferBlock& tb = layer.blocks[i];
      if (tb.block_idx >= layer.layout.num_blocks()) {
        *err = "layer " + layer.layer_name + ": block " + std::to_string(tb.block_idx) +
               " out of range (" + std::to_string(layer.layout.num_blocks()) + " blocks)";
        *failed = true;
        return false;
      }
      ids[i] = static_cast<uint32_t>(tb.block_idx);
      const RawBlock* raw = tb.block.raw;
      if (!raw || !raw->segment_mapped_ptr(0, &k[i])) {
        *err = "layer " + layer.layer_name + ": host block has no segment 0";
        *failed = true;
        return false;
      }
      k[i] = k[i].add(tb.block.offset);
      if (split) {
        if (raw->segment_mapped_ptr(1, &v[i])) {
          v[i] = v[i].add(tb.block.offset);
        } else {
          v[i] = k[i].add(frag);
        }
      }
    }
    lb.block_ids = ids.data();
    out->total_bytes += frag * (split ? 2 : 1) * n;

    // Uniform stride?
    bool uniform = true;
    uint64_t stride = frag;
    if (n > 1) {
      if (k[1].host < k[0].host) {
        uniform = false;
      } else {
        stride = static_cast<uint64_t>(k[1].host - k[0].host);
        if (stride < frag) uniform = false;
      }
    }
    for (size_t i = 1; uniform && i < n; ++i) {
      uniform = k[i].host == k[0].host + i * stride && k[i].device == k[0].device + i * stride;
      if (uniform && split) {
        uniform = v[i].host == v[0].host + i * stride && v[i].device == v[0].device + i * stride;
      }
    }
    if (uniform) {
      lb.host[0] = k[0].host;
      lb.host_device[0] = reinterpret_cast<uint64_t>(k[0].device);
      lb.host_len[0] = (n - 1) * stride + frag;
      if (split) {
        lb.host[1] = v[0].host;
        lb.host_device[1] = reinterpret_cast<uint64_t>(v[0].device);
        lb.host_len[1] = (n - 1) * stride + frag;
      }
      lb.host_stride = stride;
      continue;
    }
    // Per-block bases: needs V right behind K when split.
    bool table_ok = true;
    for (size_t i = 0; table_ok && split && i < n; ++i) {
      table_ok = v[i].host == k[i].host + frag && v[i].device == k[i].device + frag;
    }
    if (!table_ok) return false;
    std::vector<uint64_t>& ph = out->page_host[li];
    std::vector<uint64_t>& pd = out->page_dev[li];
    ph.resize(n);
    pd.resize(n);
    for (size_t i = 0; i < n; ++i) {
      ph[i] = reinterpret_cast<uint64_t>(k[i].host);
      pd[i] = reinterpret_cast<uint64_t>(k[i].device);
    }
    lb.page_host = ph.data();
    lb.page_host_device = pd.data();
    lb.page_offset = 0;
    lb.page_len = frag * (split ? 2 : 1);
  }
  return true;
}

}  // namespace

std::unique_ptr<GpuWorkerPool> GpuWorkerPool::spawn(int device_id, NumaNode numa_node,
                                                    TransferMode mode,
                                                    bool use_descriptor_backends, std::string* err,
                                                    int* status) {
  std::unique_ptr<GpuWorkerPool> pool(new GpuWorkerPool());
  pool->device_id_ = device_id;
  pool->mode_ = mode;
  pool->use_descriptors_ = use_descriptor_backends;
  std::promise<TaskResult> load_ready, save_ready;
  auto lf = load_ready.get_future();
  auto sf = save_ready.get_future();
  GpuWorkerPool* p = pool.get();
  pool->load_.thread = std::thread([p, numa_node, &load_ready] { p->run(&p->load_, true, numa_node, &load_ready); });
  pool->save_.thread = std::thread([p, numa_node, &save_ready] { p->run(&p->save_, false, numa_node, &save_ready); });
  // Initialisation errors surface synchronously (gpu_worker.rs:189-190,250-260).
  TaskResult lr = lf.get();
  TaskResult sr = sf.get();
  if (lr.status != PF_OK || sr.status != PF_OK) {
    const TaskResult& bad = lr.status != PF_OK ? lr : sr;
    if (err) *err = bad.message;
    if (status) *status = bad.status;
    return nullptr;  // destructor joins the threads
  }
  return pool;
}

GpuWorkerPool::~GpuWorkerPool() {
  for (Worker* w : {&load_, &save_}) {
    {
      std::lock_guard<std::mutex> lock(w->mu);
      w->stop = true;
    }
    w->cv.notify_all();
    if (w->thread.joinable()) w->thread.join();
  }
}

std::future<TaskResult> GpuWorkerPool::push(Worker* w, std::unique_ptr<Task> t) {
  auto fut = t->reply.get_future();
  {
    std::lock_guard<std::mutex> lock(w->mu);
    if (w->stop) {
      TaskResult r;
      r.status = PF_ERR_STORAGE;
      r.message = "worker channel closed for device " + std::to_string(device_id_);
      t->reply.set_value(r);
      return fut;
    }
    w->queue.push_back(std::move(t));
  }
  w->cv.notify_one();
  return fut;
}

std::future<TaskResult> GpuWorkerPool::submit_load(std::vector<LayerTransferData> layers,
                                                   LoadCompletion completion) {
  auto t = std::make_unique<Task>();
  t->layers = std::move(layers);
  t->completion = std::move(completion);
  return push(&load_, std::move(t));
}

std::future<TaskResult> GpuWorkerPool::batch_save(std::vector<LayerTransferData> layers) {
  auto t = std::make_unique<Task>();
  t->layers = std::move(layers);
  return push(&save_, std::move(t));
}

void GpuWorkerPool::run(Worker* w, bool is_load, NumaNode numa, std::promise<TaskResult>* ready) {
  // Pin before any allocation (gpu_worker.rs:147-152); failure is not fatal.
  if (numa.is_valid()) {
    std::string e;
    (void)pin_thread_to_numa_node(numa, &e);
  }
  // init_worker, gpu_worker.rs:278-298.
  TaskResult init;
  hipStream_t stream = nullptr;
  hipEvent_t done = nullptr;
  std::unique_ptr<TransferBackend> backend;
  std::unique_ptr<Xfer> xfer;
  hipError_t e = hipSetDevice(device_id_);
  if (e == hipSuccess) e = hipStreamCreateWithFlags(&stream, hipStreamNonBlocking);
  if (e == hipSuccess) e = hipEventCreateWithFlags(&done, hipEventDisableTiming);
  if (e != hipSuccess) {
    fail_hip(e, "worker init");
    init.status = PF_ERR_DEVICE_INIT;
    init.message = "Failed to initialise GPU worker on device " + std::to_string(device_id_) +
                   ": " + last_error();
  } else {
    backend = build_backend(mode_);
    if (!use_descriptors_) {
      xfer = Xfer::create(nullptr);
      if (!xfer) {
        init.status = PF_ERR_DEVICE_INIT;
        init.message = "transfer engine init failed: " + last_error();
      }
    }
  }
  ready->set_value(init);
  if (init.status != PF_OK) {
    if (done) (void)hipEventDestroy(done);
    if (stream) (void)hipStreamDestroy(stream);
    return;
  }
  const int path = mode_ == TransferMode::Kernel ? PF_PATH_ZEROCOPY : PF_PATH_AUTO;

  for (;;) {
    std::unique_ptr<Task> task;
    {
      std::unique_lock<std::mutex> lock(w->mu);
      w->cv.wait(lock, [w] { return w->stop || !w->queue.empty(); });
      if (w->queue.empty()) break;  // stop requested and drained
      task = std::move(w->queue.front());
      w->queue.pop_front();
    }
    // process_load_task / process_save_task, gpu_worker.rs:428-523.
    const auto t0 = std::chrono::steady_clock::now();
    TaskResult res;
    std::string err;
    int st = PF_OK;
    bool done_fast = false;
    if (xfer) {
      BlockForm form;
      bool failed = false;
      if (to_block_form(task->layers, &form, &failed, &err)) {
        st = is_load ? xfer->load(form.layers.data(), form.layers.size(), path, stream)
                     : xfer->save(form.layers.data(), form.layers.size(), path, stream);
        if (st != PF_OK) err = last_error();
        res.bytes = form.total_bytes;
        done_fast = true;
      } else if (failed) {
        st = PF_ERR_STORAGE;
        done_fast = true;
      }
    }
    if (!done_fast) {
      std::vector<CopyDesc> copies;
      uint64_t total = 0;
      if (!build_copy_descs(task->layers, &copies, &total, &err)) {
        st = PF_ERR_STORAGE;
      } else {
        st = is_load ? backend->h2d(copies.data(), copies.size(), stream)
                     : backend->d2h(copies.data(), copies.size(), stream);
        if (st != PF_OK) err = last_error();
        res.bytes = total;
      }
    }
    if (st == PF_OK) {
      // One synchronisation for all layers.
      hipError_t he = hipEventRecord(done, stream);
      if (he == hipSuccess) he = hipEventSynchronize(done);
      if (he != hipSuccess) {
        st = fail_hip(he, "Failed to synchronize");
        err = last_error();
      }
    } else {
      // Something may already be enqueued: drain it before the buffers go away.
      (void)hipStreamSynchronize(stream);
      (void)hipGetLastError();
    }
    res.status = st;
    res.message = err;
    res.elapsed_ms =
        std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    if (is_load && !task->completion.load_state_shm.empty()) {
      std::string aerr;
      auto ls = LoadState::attach(task->completion.load_state_shm, &aerr);
      if (ls) {
        if (st == PF_OK) ls->set_completed(); else ls->set_error();
      } else {
        fprintf(stderr, "Failed to attach to LoadState shm=%s: %s\n",
                task->completion.load_state_shm.c_str(), aerr.c_str());
      }
    }
    // The host blocks travel back with the layers (gpu_worker.rs:333-341):
    // release them before replying so the caller observes settled ownership.
    task->layers.clear();
    task->reply.set_value(res);
  }
  xfer.reset();
  backend.reset();
  (void)hipEventDestroy(done);
  (void)hipStreamDestroy(stream);
}

}  // namespace pf
