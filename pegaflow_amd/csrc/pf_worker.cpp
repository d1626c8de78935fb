#include "pf_worker.hpp"

#include <chrono>
#include <cstring>

#include "pf_common.hpp"
#include "pf_kernels.hpp"
#include "pf_sync_state.hpp"
#include "pf_xfer.hpp"

namespace pf {

namespace {
// The workers move KV beside a running model: a task whose dense layers add up
// to this much is staged whatever the size of its layers (see run()).
constexpr uint64_t kWorkerStagedCallBytes = 8ull << 20;
}  // namespace

bool build_copy_descs(const std::vector<LayerTransferData>& layers, std::vector<CopyDesc>* out,
                      uint64_t* total_bytes, std::string* err, size_t begin, size_t end) {
  out->clear();
  uint64_t total = 0;
  if (end <= begin) {
    begin = 0;
    end = layers.size();
  }
  for (size_t li = begin; li < end && li < layers.size(); ++li) {
    const LayerTransferData& layer = layers[li];
    if (layer.image.kind != HostImage::Kind::None) {
      // The same descriptors per-block handles over this image would give.
      const HostImage& im = layer.image;
      const size_t n = im.size();
      const bool paged = im.kind == HostImage::Kind::Paged;
      if (paged && (!im.pages || im.pages->size() != n || !im.page_allocation_ids ||
                    im.page_allocation_ids->size() != n)) {
        *err = "layer " + layer.layer_name + ": host image has a page list of the wrong length";
        return false;
      }
      for (size_t i = 0; i < n; ++i) {
        BlockCopies bc;
        std::string cause;
        if (!layer.layout.block_copies((*im.block_ids)[i], &bc, &cause)) {
          *err = "layer " + layer.layer_name + ": " + cause;
          return false;
        }
        MappedPinnedPtr k, v;
        uint64_t k_alloc, v_alloc;
        if (paged) {
          k = (*im.pages)[i].add(im.offset);
          v = k.add(bc.k.bytes);
          k_alloc = v_alloc = (*im.page_allocation_ids)[i];
        } else {
          k = im.seg[0].add(i * im.stride);
          k_alloc = im.seg_allocation_id[0];
          if (bc.n == 2 && im.seg[1].host != nullptr) {
            v = im.seg[1].add(i * im.stride);
            v_alloc = im.seg_allocation_id[1];
          } else {
            v = k.add(bc.k.bytes);
            v_alloc = k_alloc;
          }
        }
        out->push_back({bc.k.addr, k.host, reinterpret_cast<uint64_t>(k.device), bc.k.bytes, li,
                        k_alloc});
        total += bc.k.bytes;
        if (bc.n == 2) {
          out->push_back({bc.v.addr, v.host, reinterpret_cast<uint64_t>(v.device), bc.v.bytes, li,
                          v_alloc});
          total += bc.v.bytes;
        }
      }
      continue;
    }
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
  // Page tables of host images, one per distinct page list, so that the
  // layers of a page-first task pass the very same table.
  std::vector<const void*> image_pages;
  std::vector<std::vector<uint64_t>> image_page_host;
  std::vector<std::vector<uint64_t>> image_page_dev;
  std::vector<int> layer_table;  // per layer: index into image_pages, or -1
  uint64_t total_bytes = 0;
};

// Express the task through block ids: per layer either a uniform-stride host
// image or a per-block base table.  Returns false when some layer fits
// neither form (e.g. K and V of each block in unrelated allocations); the
// caller then falls back to per-fragment descriptors.  Errors are reported
// through *err with *failed = true.
bool to_block_form(const std::vector<LayerTransferData>& all_layers, size_t begin, size_t end,
                   BlockForm* out, bool* failed, std::string* err) {
  *failed = false;
  const size_t n_layers = end - begin;
  out->layers.resize(n_layers);
  out->ids.resize(n_layers);
  out->page_host.resize(n_layers);
  out->page_dev.resize(n_layers);
  out->layer_table.assign(n_layers, -1);
  for (size_t li = 0; li < n_layers; ++li) {
    const LayerTransferData& layer = all_layers[begin + li];
    pf_layer_blocks& lb = out->layers[li];
    std::memset(&lb, 0, sizeof(lb));
    lb.layer_name = layer.layer_name.c_str();
    lb.layout = layer.layout.c();
    const bool split = layer.layout.is_split();
    const uint64_t frag = layer.layout.fragment_bytes();
    if (layer.image.kind != HostImage::Kind::None) {
      const HostImage& im = layer.image;
      const size_t n_im = im.size();
      lb.n_blocks = n_im;
      if (n_im == 0) continue;
      // Block ids are range-checked by the transfer engine's own planning.
      lb.block_ids = im.block_ids->data();
      out->total_bytes += frag * (split ? 2 : 1) * n_im;
      if (im.kind == HostImage::Kind::Uniform) {
        const int n_seg = split ? 2 : 1;
        for (int sgi = 0; sgi < n_seg; ++sgi) {
          const MappedPinnedPtr base = (sgi == 1 && im.seg[1].host == nullptr)
                                           ? im.seg[0].add(frag) : im.seg[sgi];
          lb.host[sgi] = base.host;
          lb.host_device[sgi] = reinterpret_cast<uint64_t>(base.device);
          lb.host_len[sgi] = (n_im - 1) * im.stride + frag;
        }
        lb.host_stride = im.stride;
        continue;
      }
      if (!im.pages || im.pages->size() != n_im) {
        *err = "layer " + layer.layer_name + ": host image has a page list of the wrong length";
        *failed = true;
        return false;
      }
      size_t ti = 0;
      while (ti < out->image_pages.size() && out->image_pages[ti] != im.pages.get()) ++ti;
      if (ti == out->image_pages.size()) {
        out->image_pages.push_back(im.pages.get());
        out->image_page_host.emplace_back(n_im);
        out->image_page_dev.emplace_back(n_im);
        for (size_t i = 0; i < n_im; ++i) {
          out->image_page_host[ti][i] = reinterpret_cast<uint64_t>((*im.pages)[i].host);
          out->image_page_dev[ti][i] = reinterpret_cast<uint64_t>((*im.pages)[i].device);
        }
      }
      // (the vectors are filled once and never resized afterwards; the outer
      // vectors may grow, so the pointers are taken after the loop below)
      lb.page_offset = im.offset;
      lb.page_len = im.page_len;
      out->layer_table[li] = static_cast<int>(ti);
      continue;
    }
    const size_t n = layer.blocks.size();
    lb.n_blocks = n;
    if (n == 0) continue;
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
  for (size_t li = 0; li < n_layers; ++li) {
    const int ti = out->layer_table[li];
    if (ti < 0) continue;
    out->layers[li].page_host = out->image_page_host[ti].data();
    out->layers[li].page_host_device = out->image_page_dev[ti].data();
  }
  return true;
}

}  // namespace

std::unique_ptr<GpuWorkerPool> GpuWorkerPool::spawn(int device_id, NumaNode numa_node,
                                                    TransferMode mode,
                                                    const WorkerPoolOptions& options,
                                                    std::string* err, int* status) {
  std::unique_ptr<GpuWorkerPool> pool(new GpuWorkerPool());
  pool->device_id_ = device_id;
  pool->mode_ = mode;
  pool->options_ = options;
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
  pool->separate_worker_queues();
  pool->prime_copy_overlap();
  // One line per pool: an operator who asked for `kernel` (the connector's
  // default for MLA models, common.py:577-594) should see that the workers here
  // choose the path per task in both of the reference's modes.
  const char* mode_name = mode == TransferMode::Direct ? "direct"
                          : mode == TransferMode::Kernel ? "kernel" : "zerocopy";
  if (options.use_descriptor_backends) {
    log_line(LogLevel::Info,
             "worker pool on device %d: transfer mode '%s' -> per-fragment descriptors through the "
             "%s backend", device_id, mode_name, mode == TransferMode::Direct ? "direct" : "kernel");
  } else if (mode == TransferMode::ZeroCopy) {
    log_line(LogLevel::Info,
             "worker pool on device %d: transfer mode 'zerocopy' -> block-ID kernel over mapped "
             "host memory for every task, no staging memory", device_id);
  } else {
    const uint64_t call_min = options.auto_staged_min_bytes ? options.auto_staged_min_bytes
                                                             : kWorkerStagedCallBytes;
    log_line(LogLevel::Info,
             "worker pool on device %d: transfer mode '%s' -> block-ID engine, path chosen per "
             "task (staged through device memory from %llu bytes of dense layers per task, "
             "zero-copy kernel below); staging memory held: %llu MiB%s",
             device_id, mode_name, static_cast<unsigned long long>(call_min),
             static_cast<unsigned long long>(pool->staging_bytes() >> 20),
             options.lazy_staging ? " (allocated on the first staged task)" : "");
  }
  return pool;
}

bool GpuWorkerPool::last_load(TaskResult* out, std::chrono::steady_clock::time_point* when) {
  std::lock_guard<std::mutex> lock(last_load_mu_);
  if (!has_last_load_) return false;
  *out = last_load_;
  *when = last_load_when_;
  return true;
}

// Worker streams must not share a hardware queue: a zero-copy save and a
// zero-copy load are one long kernel each, and on one queue the second simply
// waits for the first (seen with rocprofv3 --kernel-trace: the save worker of
// one instance and the load worker of another both on queue 3, the load
// starting the moment the save ended, 57 GB/s for the pair instead of 94).
// The runtime decides which queue a stream gets and offers no way to ask, so
// a new pool checks whether kernels of its streams overlap with each other
// and with the idle worker streams of the other pools on the device, and
// replaces a stream that does not by a fresh one, a few times at most, keeping
// the candidate with the fewest clashes.  Rejected streams are destroyed at
// the end (destroying one at once could hand its queue to the very next
// stream).  No task has been accepted yet.
namespace {
// Work on the pool's device from a thread that may have another one current
// (spawn runs on the registering thread): the previous device comes back.
class DeviceScope {
 public:
  explicit DeviceScope(int device) {
    if (hipGetDevice(&previous_) != hipSuccess) previous_ = -1;
    ok_ = hipSetDevice(device) == hipSuccess;
  }
  ~DeviceScope() {
    if (previous_ >= 0) (void)hipSetDevice(previous_);
    (void)hipGetLastError();
  }
  bool ok() const { return ok_; }

 private:
  int previous_ = -1;
  bool ok_ = false;
};

std::mutex g_worker_streams_mu;
std::vector<std::pair<int, hipStream_t>> g_worker_streams;  // (device, stream) of live pools
// The same for the copy streams of pools with side_copy_streams, and which
// direction each serves: a clash between copy streams of one direction costs
// nothing (they share the link anyway), one across directions costs the overlap
// of a save with a load.
struct SideStream {
  int device;
  hipStream_t stream;
  bool is_load;
};
std::vector<SideStream> g_side_streams;

// Do kernels of `candidate` (idle by construction) and `other` run side by side?
// `other` belongs to a live pool and may receive a task at any moment: a probe
// that finds it busy, or that reports a clash once but not twice, says nothing.
bool clash_with(hipStream_t candidate, hipStream_t other) {
  for (int attempt = 0; attempt < 2; ++attempt) {
    if (hipStreamQuery(other) != hipSuccess) {
      (void)hipGetLastError();
      return false;  // busy: the posting kernel would queue behind its work
    }
    bool concurrent = true;
    // The waiting kernel goes on the candidate.
    if (streams_run_concurrently(candidate, other, &concurrent) != PF_OK) return false;
    if (concurrent) return false;
  }
  return true;
}

size_t clashes(hipStream_t candidate, const std::vector<hipStream_t>& others) {
  size_t n = 0;
  for (hipStream_t other : others) n += clash_with(candidate, other) ? 1 : 0;
  return n;
}
}  // namespace

int worker_stream_report(int device, size_t* out_streams, size_t* out_clashing_pairs,
                         size_t* out_skipped) {
  DeviceScope scope(device);
  if (!scope.ok()) return fail(PF_ERR_DEVICE_INIT, "cannot select device %d", device);
  std::lock_guard<std::mutex> registry(g_worker_streams_mu);
  std::vector<hipStream_t> idle;
  size_t skipped = 0, total = 0;
  for (const auto& entry : g_worker_streams) {
    if (entry.first != device) continue;
    ++total;
    if (hipStreamQuery(entry.second) == hipSuccess) {
      idle.push_back(entry.second);
    } else {
      ++skipped;
    }
  }
  (void)hipGetLastError();
  size_t pairs = 0;
  for (size_t i = 0; i < idle.size(); ++i) {
    for (size_t j = i + 1; j < idle.size(); ++j) pairs += clash_with(idle[i], idle[j]) ? 1 : 0;
  }
  *out_streams = total;
  *out_clashing_pairs = pairs;
  *out_skipped = skipped;
  return PF_OK;
}

void GpuWorkerPool::separate_worker_queues() {
  DeviceScope device(device_id_);
  if (!device.ok()) return;
  std::lock_guard<std::mutex> registry(g_worker_streams_mu);
  std::vector<hipStream_t> others;
  for (auto it = g_worker_streams.rbegin(); it != g_worker_streams.rend() && others.size() < 6;
       ++it) {
    // A stream that is busy would make the probe wait for its work: skip it.
    if (it->first == device_id_ && hipStreamQuery(it->second) == hipSuccess) {
      others.push_back(it->second);
    }
  }
  (void)hipGetLastError();
  std::vector<hipStream_t> rejected;
  for (Worker* w : {&save_, &load_}) {
    hipStream_t best = w->stream;
    size_t best_clashes = clashes(best, others);
    for (int attempt = 0; attempt < 6 && best_clashes != 0; ++attempt) {
      hipStream_t fresh = nullptr;
      if (hipStreamCreateWithFlags(&fresh, hipStreamNonBlocking) != hipSuccess) break;
      const size_t c = clashes(fresh, others);
      if (c < best_clashes) {
        rejected.push_back(best);
        best = fresh;
        best_clashes = c;
      } else {
        rejected.push_back(fresh);
      }
    }
    {
      std::lock_guard<std::mutex> lock(w->mu);
      w->stream = best;
    }
    queue_clashes_ += best_clashes;
    others.push_back(best);
  }
  // The copy streams of a pool with side_copy_streams: each on a queue that
  // none of the pool's other streams uses, nor a worker or copy stream of
  // another pool that serves the opposite direction (kernels and copies of one
  // direction may queue behind one another across pools; they share the link).
  if (options_.side_copy_streams) {
    for (Worker* w : {&save_, &load_}) {
      if (w->side == nullptr) continue;
      const bool is_load = w == &load_;
      std::vector<hipStream_t> avoid = {save_.stream, load_.stream};
      if (is_load && save_.side != nullptr) avoid.push_back(save_.side);
      for (const SideStream& other : g_side_streams) {
        if (other.device == device_id_ && other.is_load != is_load && avoid.size() < 8 &&
            hipStreamQuery(other.stream) == hipSuccess) {
          avoid.push_back(other.stream);
        }
      }
      // Worker streams are registered in pairs, save then load.
      for (size_t i = 0; i < g_worker_streams.size(); ++i) {
        const bool other_is_load = (i & 1) != 0;
        if (g_worker_streams[i].first == device_id_ && other_is_load != is_load &&
            avoid.size() < 8 && hipStreamQuery(g_worker_streams[i].second) == hipSuccess) {
          avoid.push_back(g_worker_streams[i].second);
        }
      }
      (void)hipGetLastError();
      hipStream_t best = w->side;
      size_t best_clashes = clashes(best, avoid);
      for (int attempt = 0; attempt < 8 && best_clashes != 0; ++attempt) {
        hipStream_t fresh = nullptr;
        if (hipStreamCreateWithFlags(&fresh, hipStreamNonBlocking) != hipSuccess) break;
        const size_t c = clashes(fresh, avoid);
        if (c < best_clashes) {
          rejected.push_back(best);
          best = fresh;
          best_clashes = c;
        } else {
          rejected.push_back(fresh);
        }
      }
      {
        std::lock_guard<std::mutex> lock(w->mu);
        w->side = best;
      }
      queue_clashes_ += best_clashes;
    }
  }
  for (hipStream_t s : rejected) (void)hipStreamDestroy(s);
  (void)hipGetLastError();
  g_worker_streams.emplace_back(device_id_, save_.stream);
  g_worker_streams.emplace_back(device_id_, load_.stream);
  if (save_.side) g_side_streams.push_back({device_id_, save_.side, false});
  if (load_.side) g_side_streams.push_back({device_id_, load_.side, true});
}

// Measured on MI355X with this runtime: whether the link copies of the save
// stream and of the load stream overlap is settled by their first large copies.
// When the load stream's first host -> device copy is issued while a device ->
// host copy of the save stream is in flight, the two directions overlap from
// then on (a save and a load together: 88-107 GB/s); when that first copy runs
// with nothing else in flight, every later pair is serialised (55 GB/s), and
// so is a pool whose load stream was warmed up alone.  So the pool issues,
// once, a few 32 MiB copies on the save stream and, while they run, the same
// on the load stream.  Failure here only loses the overlap.
void GpuWorkerPool::prime_copy_overlap() {
  DeviceScope device(device_id_);
  if (!device.ok()) return;
  const size_t chunk = 32u << 20;
  if (hipHostMalloc(&prime_host_, 2 * chunk, hipHostMallocMapped) == hipSuccess &&
      hipMalloc(&prime_dev_, 2 * chunk) == hipSuccess) {
    std::memset(prime_host_, 0, 2 * chunk);
    uint8_t* h = static_cast<uint8_t*>(prime_host_);
    uint8_t* d = static_cast<uint8_t*>(prime_dev_);
    // On the streams that will carry the copies.
    hipStream_t save_copies = save_.side ? save_.side : save_.stream;
    hipStream_t load_copies = load_.side ? load_.side : load_.stream;
    for (int i = 0; i < 6; ++i) {
      (void)hipMemcpyAsync(h, d, chunk, hipMemcpyDeviceToHost, save_copies);
    }
    for (int i = 0; i < 3; ++i) {
      (void)hipMemcpyAsync(d + chunk, h + chunk, chunk, hipMemcpyHostToDevice, load_copies);
    }
    (void)hipStreamSynchronize(save_copies);
    (void)hipStreamSynchronize(load_copies);
  }
  (void)hipGetLastError();
}

GpuWorkerPool::~GpuWorkerPool() {
  {
    // Out of the registry before the workers destroy their streams.
    std::lock_guard<std::mutex> registry(g_worker_streams_mu);
    for (auto it = g_worker_streams.begin(); it != g_worker_streams.end();) {
      const bool mine = it->second == save_.stream || it->second == load_.stream;
      it = mine ? g_worker_streams.erase(it) : it + 1;
    }
    for (auto it = g_side_streams.begin(); it != g_side_streams.end();) {
      const bool mine = it->stream == save_.side || it->stream == load_.side;
      it = mine ? g_side_streams.erase(it) : it + 1;
    }
  }
  for (Worker* w : {&load_, &save_}) {
    {
      std::lock_guard<std::mutex> lock(w->mu);
      w->stop = true;
    }
    w->cv.notify_all();
    if (w->thread.joinable()) w->thread.join();
  }
  if (prime_dev_ || prime_host_) {
    DeviceScope device(device_id_);
    if (prime_dev_) (void)hipFree(prime_dev_);
    if (prime_host_) (void)hipHostFree(prime_host_);
    (void)hipGetLastError();
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
    t->submitted = std::chrono::steady_clock::now();
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
  hipStream_t side = nullptr;
  hipError_t e = hipSetDevice(device_id_);
  if (e == hipSuccess) e = hipStreamCreateWithFlags(&stream, hipStreamNonBlocking);
  if (e == hipSuccess && options_.side_copy_streams && !options_.use_descriptor_backends &&
      mode_ != TransferMode::ZeroCopy) {
    e = hipStreamCreateWithFlags(&side, hipStreamNonBlocking);
  }
  if (e == hipSuccess) e = hipEventCreateWithFlags(&done, hipEventDisableTiming);
  if (e != hipSuccess) {
    fail_hip(e, "worker init");
    init.status = PF_ERR_DEVICE_INIT;
    init.message = "Failed to initialise GPU worker on device " + std::to_string(device_id_) +
                   ": " + last_error();
  } else {
    backend = build_backend(mode_);
    if (!options_.use_descriptor_backends) {
      // The pool always has a second engine (load next to save), so each
      // worker keeps to one stream: with a side stream per engine the link
      // copies of the two directions were seen on one hardware queue (a
      // process gets 4 by default) and a save and a load together shared
      // 56 GB/s.  One stream per worker costs 1.4 % when one direction is
      // active alone (see also prime_copy_overlap).
      pf_xfer_config cfg;
      std::memset(&cfg, 0, sizeof(cfg));
      // With side_copy_streams the pool gives each worker a second stream for
      // the link copies, placed and primed like the worker streams (see
      // separate_worker_queues, prime_copy_overlap).
      cfg.copy_stream = side != nullptr ? 1 : 2;
      // The workers move KV beside a running model, so they also stage tasks
      // of small layers once the task is long enough for the resident
      // zero-copy kernel to matter to the kernels beside it.  A stream of
      // 2048^3 bf16 GEMMs beside an unbroken loop of saves and loads through
      // these workers, 32 layers per call, keeps 0.94-0.96 of its rate when
      // the layers are staged and 0.21 (4 MiB layers), 0.36 (1 MiB), 0.58
      // (256 KiB), 0.84 (64 KiB) beside the resident kernel; staging costs
      // such a call 50-70 us, the length of a 3-4 MiB transfer.
      cfg.auto_staged_min_call_bytes = options_.auto_staged_min_bytes != 0
                                           ? options_.auto_staged_min_bytes
                                           : kWorkerStagedCallBytes;
      cfg.staging_slot_bytes = options_.staging_slot_bytes;
      xfer = Xfer::create(&cfg);
      // Everything a worker needs exists before its first task (init_worker,
      // gpu_worker.rs:278-298): the staging slots too, unless the pool was
      // asked to leave them to the first staged task.  A zero-copy pool never
      // stages.
      int xst = xfer ? xfer->enable_profile() : PF_ERR_DEVICE_INIT;
      if (xst == PF_OK && mode_ != TransferMode::ZeroCopy && !options_.lazy_staging) {
        xst = xfer->reserve_staging();
        if (xst != PF_OK && xfer->staging_out_of_memory()) {
          // Not fatal: every task can cross the link with the zero-copy kernel,
          // and each staged task tries the allocation again (Xfer::run).
          log_line(LogLevel::Info,
                   "worker pool on device %d: no device memory for the %s worker's staging slots "
                   "(%s); its tasks take the zero-copy path until the slots can be allocated",
                   device_id_, is_load ? "load" : "save", last_error().c_str());
          (void)hipGetLastError();
          xst = PF_OK;
        }
      }
      if (xst != PF_OK) {
        init.status = PF_ERR_DEVICE_INIT;
        init.message = "transfer engine init failed: " + last_error();
        xfer.reset();
      } else {
        staging_bytes_ += xfer->staging_bytes();
      }
    }
  }
  w->stream = stream;
  w->side = side;
  ready->set_value(init);
  if (init.status != PF_OK) {
    if (done) (void)hipEventDestroy(done);
    if (side) (void)hipStreamDestroy(side);
    if (stream) (void)hipStreamDestroy(stream);
    return;
  }
  // Direct and kernel mode alike let the engine choose per call: large dense
  // transfers are staged (their link crossing needs no compute unit, so model
  // kernels beside them keep their rate), small and scattered ones go zero-copy.
  const int path = mode_ == TransferMode::ZeroCopy ? PF_PATH_ZEROCOPY : PF_PATH_AUTO;

  for (;;) {
    std::unique_ptr<Task> task;
    {
      std::unique_lock<std::mutex> lock(w->mu);
      w->cv.wait(lock, [w] { return w->stop || !w->queue.empty(); });
      if (w->queue.empty()) break;  // stop requested and drained
      task = std::move(w->queue.front());
      w->queue.pop_front();
      stream = w->stream;  // the pool may have replaced it before the first task
      side = w->side;
    }
    if (xfer && side != nullptr) xfer->set_side_stream(side);
    // process_load_task / process_save_task, gpu_worker.rs:428-523.
    const auto t0 = std::chrono::steady_clock::now();
    TaskResult res;
    res.queue_ms = std::chrono::duration<double, std::milli>(t0 - task->submitted).count();
    res.resolve_ms = task->completion.resolve_ms;
    std::string err;
    int st = PF_OK;
    const uint64_t staging_before = xfer ? xfer->staging_bytes() : 0;
    if (xfer) xfer->reset_profile();
    auto since = [](std::chrono::steady_clock::time_point t) {
      return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t).count();
    };
    // A task whose layers come as per-block handles is converted in two
    // parts: a few layers first, so that the device starts on them while the
    // (much larger) rest is still being converted.  Everything is only
    // enqueued; there is still one synchronisation.  Tasks described by host
    // images need no conversion work and go in one call, which also keeps the
    // layers of page-first pages together for whole-page staging.  Zero-copy
    // tasks go in one call as well: a two-layer zero-copy launch that starts
    // next to a zero-copy save of another worker crawled (124 ms instead of
    // 11 ms, the save beside it at a quarter of its rate; a save and a load
    // together 68 GB/s), while single launches share the link at 91-92 GB/s;
    // alone, the one call costs 0.5-2 % of a load.
    const size_t n_layers = task->layers.size();
    bool per_block = false;
    size_t handles = 0;
    for (const auto& l : task->layers) {
      per_block |= !l.blocks.empty();
      handles += l.blocks.size();
    }
    size_t first_part = n_layers ? n_layers : 1;
    // (Descriptor backends build one descriptor per fragment whatever the form.)
    // A task of few handles converts in microseconds: splitting it would only
    // cost the second call's launches.
    constexpr size_t kSplitFromHandles = 32768;
    if ((!xfer || (per_block && path != PF_PATH_ZEROCOPY && handles >= kSplitFromHandles)) &&
        n_layers >= 16) {
      first_part = n_layers / 16 < 2 ? 2 : n_layers / 16;
    }
    for (size_t begin = 0; begin < n_layers && st == PF_OK;) {
      // Block-ID form: the rest goes in one call (a call boundary drains the
      // engine's copy pipeline).  Descriptor form: every part is that small;
      // its copies are in order on one stream, so boundaries cost nothing.
      const size_t end = (begin == 0 || !xfer)
                             ? (begin + first_part < n_layers ? begin + first_part : n_layers)
                             : n_layers;
      bool done_fast = false;
      if (xfer) {
        BlockForm form;
        bool failed = false;
        const auto t_convert = std::chrono::steady_clock::now();
        const bool converted = to_block_form(task->layers, begin, end, &form, &failed, &err);
        res.convert_ms += since(t_convert);
        if (converted) {
          st = is_load ? xfer->load(form.layers.data(), form.layers.size(), path, stream)
                       : xfer->save(form.layers.data(), form.layers.size(), path, stream);
          if (st != PF_OK) err = last_error();
          res.bytes += form.total_bytes;
          done_fast = true;
        } else if (failed) {
          st = PF_ERR_STORAGE;
          done_fast = true;
        }
      }
      if (!done_fast) {
        std::vector<CopyDesc> copies;
        uint64_t total = 0;
        const auto t_convert = std::chrono::steady_clock::now();
        const bool built = build_copy_descs(task->layers, &copies, &total, &err, begin, end);
        res.convert_ms += since(t_convert);
        if (!built) {
          st = PF_ERR_STORAGE;
        } else {
          const auto t_enqueue = std::chrono::steady_clock::now();
          st = is_load ? backend->h2d(copies.data(), copies.size(), stream)
                       : backend->d2h(copies.data(), copies.size(), stream);
          res.enqueue_ms += since(t_enqueue);
          if (st != PF_OK) err = last_error();
          res.bytes += total;
          res.paths |= PF_TASK_PATH_DESCRIPTORS;
        }
      }
      begin = end;
    }
    const auto t_sync = std::chrono::steady_clock::now();
    if (st == PF_OK) {
      // One synchronisation for all layers.
      hipError_t he = hipEventRecord(done, stream);
      if (he == hipSuccess) {
        // A blocking wait costs its wake-up (10-15 us measured here, a fifth of
        // a 2 MiB task): poll for the length of a short task first.
        const auto spin_until = std::chrono::steady_clock::now() + std::chrono::microseconds(150);
        he = hipErrorNotReady;
        while (std::chrono::steady_clock::now() < spin_until) {
          he = hipEventQuery(done);
          if (he != hipErrorNotReady) break;
        }
        if (he == hipErrorNotReady) {
          (void)hipGetLastError();
          he = hipEventSynchronize(done);
        }
      }
      if (he != hipSuccess) {
        st = fail_hip(he, "Failed to synchronize");
        err = last_error();
      }
    } else {
      // Something may already be enqueued: drain it before the buffers go away.
      (void)hipStreamSynchronize(stream);
      (void)hipGetLastError();
    }
    res.sync_ms = since(t_sync);
    if (xfer) {
      const XferProfile prof = xfer->read_profile();
      res.plan_ms = prof.plan_ms;
      res.staging_alloc_ms = prof.staging_alloc_ms;
      res.enqueue_ms += prof.enqueue_ms;
      res.staged_groups = prof.staged_groups;
      res.zero_copy_launches = prof.zero_copy_launches;
      res.link_copies = prof.link_copies;
      res.device_first_ms = prof.device_first_ms;
      res.device_ms = prof.device_ms;
      if (prof.staged_groups != 0) res.paths |= PF_TASK_PATH_STAGED;
      if (prof.zero_copy_launches != 0) res.paths |= PF_TASK_PATH_ZEROCOPY;
      const uint64_t staging_now = xfer->staging_bytes();
      if (staging_now != staging_before) staging_bytes_ += staging_now - staging_before;
    }
    res.status = st;
    res.message = err;
    res.elapsed_ms = since(t0);
    if (log_level() == LogLevel::Debug) {
      // gpu_worker.rs:465-474,511-520.
      log_line(LogLevel::Debug,
               "device %d %s task: %llu bytes in %.3f ms (%.2f GB/s), paths=%u staged_groups=%u "
               "zero_copy_launches=%u, queue %.3f convert %.3f plan %.3f staging_alloc %.3f "
               "enqueue %.3f sync %.3f ms, device first %.3f total %.3f ms%s%s",
               device_id_, is_load ? "load" : "save", static_cast<unsigned long long>(res.bytes),
               res.elapsed_ms, res.elapsed_ms > 0 ? res.bytes / res.elapsed_ms / 1e6 : 0.0,
               res.paths, res.staged_groups, res.zero_copy_launches, res.queue_ms, res.convert_ms,
               res.plan_ms, res.staging_alloc_ms, res.enqueue_ms, res.sync_ms,
               res.device_first_ms, res.device_ms, st == PF_OK ? "" : ": ", err.c_str());
    }
    if (is_load) {
      std::lock_guard<std::mutex> lock(last_load_mu_);
      has_last_load_ = true;
      last_load_ = res;
      last_load_when_ = std::chrono::steady_clock::now();
    }
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
  {
    std::lock_guard<std::mutex> lock(w->mu);
    stream = w->stream;
    side = w->side;
  }
  if (side) {
    (void)hipStreamSynchronize(side);
    (void)hipStreamDestroy(side);
  }
  (void)hipStreamDestroy(stream);
}

}  // namespace pf
