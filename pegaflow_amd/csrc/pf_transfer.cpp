#include "pf_transfer.hpp"

#include <algorithm>
#include <cstring>

#include "pf_common.hpp"

namespace pf {

// ---------------------------------------------------------------------------
// merge
// ---------------------------------------------------------------------------

std::vector<MergedRange> merge(const CopyDesc* copies, uint64_t n) {
  std::vector<MergedRange> out;
  out.reserve(n);
  uint64_t run_first = 0;  // index of the descriptor that opened the current run
  for (uint64_t i = 0; i < n; ++i) {
    const CopyDesc& c = copies[i];
    if (!out.empty()) {
      MergedRange& run = out.back();
      const CopyDesc& first = copies[run_first];
      const bool same_allocations = first.device_allocation == c.device_allocation &&
                                    first.host_allocation == c.host_allocation;
      const bool device_contiguous = run.device + run.size == c.device;
      const bool host_contiguous = static_cast<uint8_t*>(run.host) + run.size == c.host;
      if (same_allocations && device_contiguous && host_contiguous) {
        run.size += c.size;
        continue;
      }
    }
    run_first = i;
    out.push_back({c.device, c.host, c.size});
  }
  return out;
}

// ---------------------------------------------------------------------------
// build_copy_descs
// ---------------------------------------------------------------------------

bool build_copy_descs(const pf_layer_transfer* layers, uint64_t n_layers,
                      std::vector<CopyDesc>* out, uint64_t* total_bytes, std::string* err) {
  out->clear();
  uint64_t total = 0;
  for (uint64_t li = 0; li < n_layers; ++li) {
    const pf_layer_transfer& layer = layers[li];
    const std::string name = layer.layer_name ? layer.layer_name : "";
    KVCacheLayout layout;
    std::string cause;
    if (!KVCacheLayout::from_c(layer.layout, &layout, &cause)) {
      *err = "layer " + name + ": " + cause;
      return false;
    }
    if (layer.n_blocks != 0 && (!layer.block_idx || !layer.blocks)) {
      *err = "layer " + name + ": block list is null";
      return false;
    }
    for (uint64_t bi = 0; bi < layer.n_blocks; ++bi) {
      const pf_host_block& hb = layer.blocks[bi];
      BlockCopies bc;
      if (!layout.block_copies(layer.block_idx[bi], &bc, &cause)) {
        *err = "layer " + name + ": " + cause;
        return false;
      }
      if (hb.num_segments == 0 || hb.num_segments > 2 || !hb.seg_host[0]) {
        *err = "layer " + name + ": host block has no segment 0";
        return false;
      }
      uint8_t* k_host = static_cast<uint8_t*>(hb.seg_host[0]) + hb.host_offset;
      uint64_t k_dev = hb.seg_device[0] + hb.host_offset;
      if (bc.n == 2) {
        // A single-segment host block holds K then V back to back
        // (gpu_worker.rs:373-379).
        const bool has_v = hb.num_segments >= 2 && hb.seg_host[1];
        uint8_t* v_host = has_v ? static_cast<uint8_t*>(hb.seg_host[1]) + hb.host_offset
                                : k_host + bc.k.bytes;
        uint64_t v_dev = has_v ? hb.seg_device[1] + hb.host_offset : k_dev + bc.k.bytes;
        uint64_t v_alloc = has_v ? hb.seg_alloc[1] : hb.seg_alloc[0];
        out->push_back({bc.k.addr, k_host, k_dev, bc.k.bytes, li, hb.seg_alloc[0]});
        out->push_back({bc.v.addr, v_host, v_dev, bc.v.bytes, li, v_alloc});
        total += bc.k.bytes + bc.v.bytes;
      } else {
        out->push_back({bc.k.addr, k_host, k_dev, bc.k.bytes, li, hb.seg_alloc[0]});
        total += bc.k.bytes;
      }
    }
  }
  if (total_bytes) *total_bytes = total;
  return true;
}

// ---------------------------------------------------------------------------
// SlabPool
// ---------------------------------------------------------------------------

SlabPool::~SlabPool() {
  for (auto& s : slabs_) {
    if (s->in_flight && s->done) (void)hipEventSynchronize(s->done);
    if (s->done) (void)hipEventDestroy(s->done);
    if (s->host) (void)hipHostFree(s->host);
    if (s->dev) (void)hipFree(s->dev);
  }
  (void)hipGetLastError();
}

int SlabPool::acquire(uint64_t bytes, Slab** out) {
  for (auto& s : slabs_) {
    if (s->cap < bytes) continue;
    if (s->in_flight) {
      hipError_t q = hipEventQuery(s->done);
      if (q == hipErrorNotReady) {
        (void)hipGetLastError();
        continue;
      }
      if (q != hipSuccess) return fail_hip(q, "hipEventQuery(slab)");
      s->in_flight = false;
    }
    *out = s.get();
    return PF_OK;
  }
  uint64_t cap = 64 * 1024;
  while (cap < bytes) cap <<= 1;
  std::unique_ptr<Slab> s(new Slab());
  PF_HIP(hipHostMalloc(&s->host, cap, hipHostMallocMapped | hipHostMallocPortable));
  hipError_t e = hipMalloc(&s->dev, cap);
  if (e == hipSuccess) e = hipEventCreateWithFlags(&s->done, hipEventDisableTiming);
  if (e != hipSuccess) {
    (void)hipHostFree(s->host);
    if (s->dev) (void)hipFree(s->dev);
    return fail_hip(e, "slab allocation");
  }
  s->cap = cap;
  *out = s.get();
  slabs_.push_back(std::move(s));
  return PF_OK;
}

int SlabPool::release_after(Slab* slab, hipStream_t s) {
  PF_HIP(hipEventRecord(slab->done, s));
  slab->in_flight = true;
  return PF_OK;
}

// ---------------------------------------------------------------------------
// MemcpyBackend
// ---------------------------------------------------------------------------

int MemcpyBackend::h2d(const CopyDesc* copies, uint64_t n, hipStream_t s) {
  for (const MergedRange& m : merge(copies, n)) {
    hipError_t e =
        hipMemcpyHtoDAsync(reinterpret_cast<hipDeviceptr_t>(m.device), m.host, m.size, s);
    if (e != hipSuccess) return fail_hip(e, "hipMemcpyHtoDAsync");
  }
  return PF_OK;
}

int MemcpyBackend::d2h(const CopyDesc* copies, uint64_t n, hipStream_t s) {
  for (const MergedRange& m : merge(copies, n)) {
    hipError_t e =
        hipMemcpyDtoHAsync(m.host, reinterpret_cast<hipDeviceptr_t>(m.device), m.size, s);
    if (e != hipSuccess) return fail_hip(e, "hipMemcpyDtoHAsync");
  }
  return PF_OK;
}

// ---------------------------------------------------------------------------
// KernelBackend
// ---------------------------------------------------------------------------

int KernelBackend::submit(const CopyDesc* copies, uint64_t n, bool host_is_src, hipStream_t s) {
  if (n == 0) return PF_OK;  // kernel.rs:85-87
  if (n > 0x7FFFFFFFull) {
    return fail(PF_ERR_INVALID_ARGUMENT, "descriptor batch of %llu exceeds the kernel limit",
                static_cast<unsigned long long>(n));
  }
  const uint64_t bytes = n * 3 * sizeof(uint64_t);
  SlabPool::Slab* slab = nullptr;
  int st = slabs_.acquire(bytes, &slab);
  if (st != PF_OK) return st;
  uint64_t* table = static_cast<uint64_t*>(slab->host);
  uint64_t max_size = 0;
  for (uint64_t i = 0; i < n; ++i) {
    const CopyDesc& c = copies[i];
    table[3 * i + 0] = host_is_src ? c.device : c.host_device;
    table[3 * i + 1] = host_is_src ? c.host_device : c.device;
    table[3 * i + 2] = c.size;
    max_size = std::max<uint64_t>(max_size, c.size);
  }
  PF_HIP(hipMemcpyAsync(slab->dev, slab->host, bytes, hipMemcpyHostToDevice, s));
  st = launch_desc_copy(static_cast<const uint64_t*>(slab->dev), n, max_size, s);
  if (st != PF_OK) return st;
  return slabs_.release_after(slab, s);
}

std::unique_ptr<TransferBackend> build_backend(TransferMode mode) {
  if (mode == TransferMode::Kernel) return std::unique_ptr<TransferBackend>(new KernelBackend());
  return std::unique_ptr<TransferBackend>(new MemcpyBackend());
}

}  // namespace pf

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------

extern "C" {

int pf_merge_copies(const pf_copy_desc* copies, uint64_t n, pf_merged_range* out,
                    uint64_t* out_n) {
  PF_REQUIRE_PTR(out_n);
  if (n != 0) {
    PF_REQUIRE_PTR(copies);
    PF_REQUIRE_PTR(out);
  }
  auto merged = pf::merge(copies, n);
  for (size_t i = 0; i < merged.size(); ++i) out[i] = merged[i];
  *out_n = merged.size();
  return PF_OK;
}

int pf_backend_create(int mode, pf_backend_t* out) {
  PF_REQUIRE_PTR(out);
  if (mode != PF_MODE_DIRECT && mode != PF_MODE_KERNEL) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "unknown transfer mode %d", mode);
  }
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) {
    int code = pf::fail_hip(e, "hipGetDevice");
    (void)code;
    return pf::fail(PF_ERR_DEVICE_INIT, "backend init failed: %s", pf::last_error().c_str());
  }
  *out = reinterpret_cast<pf_backend_t>(
      pf::build_backend(static_cast<pf::TransferMode>(mode)).release());
  return PF_OK;
}

int pf_backend_destroy(pf_backend_t b) {
  delete reinterpret_cast<pf::TransferBackend*>(b);
  return PF_OK;
}

const char* pf_backend_name(pf_backend_t b) {
  return b ? reinterpret_cast<pf::TransferBackend*>(b)->name() : "";
}

int pf_backend_h2d(pf_backend_t b, const pf_copy_desc* copies, uint64_t n, pf_stream_t s) {
  PF_REQUIRE_PTR(b);
  if (n != 0) PF_REQUIRE_PTR(copies);
  return reinterpret_cast<pf::TransferBackend*>(b)->h2d(copies, n, pf::native(s));
}

int pf_backend_d2h(pf_backend_t b, const pf_copy_desc* copies, uint64_t n, pf_stream_t s) {
  PF_REQUIRE_PTR(b);
  if (n != 0) PF_REQUIRE_PTR(copies);
  return reinterpret_cast<pf::TransferBackend*>(b)->d2h(copies, n, pf::native(s));
}

int pf_transfer_mode_from_name(const char* name, int* out_mode) {
  PF_REQUIRE_PTR(name);
  PF_REQUIRE_PTR(out_mode);
  std::string s(name);
  size_t a = s.find_first_not_of(" \t\r\n");
  size_t b = s.find_last_not_of(" \t\r\n");
  s = a == std::string::npos ? "" : s.substr(a, b - a + 1);
  std::transform(s.begin(), s.end(), s.begin(), [](unsigned char c) { return std::tolower(c); });
  if (s == "direct") {
    *out_mode = PF_MODE_DIRECT;
    return PF_OK;
  }
  if (s == "kernel") {
    *out_mode = PF_MODE_KERNEL;
    return PF_OK;
  }
  return pf::fail(PF_ERR_INVALID_ARGUMENT,
                  "Unsupported pegaflow.transfer_backend '%s'; expected one of: direct, kernel",
                  name);
}

int pf_build_copy_descs(const pf_layer_transfer* layers, uint64_t n_layers, pf_copy_desc* out,
                        uint64_t cap, uint64_t* out_n, uint64_t* out_total_bytes) {
  PF_REQUIRE_PTR(out_n);
  if (n_layers != 0) PF_REQUIRE_PTR(layers);
  std::vector<pf::CopyDesc> descs;
  uint64_t total = 0;
  std::string err;
  if (!pf::build_copy_descs(layers, n_layers, &descs, &total, &err)) {
    return pf::fail(PF_ERR_STORAGE, "%s", err.c_str());
  }
  *out_n = descs.size();
  if (out_total_bytes) *out_total_bytes = total;
  if (descs.size() > cap) {
    return pf::fail(PF_ERR_BUFFER_TOO_SMALL, "descriptor buffer holds %llu entries, need %llu",
                    static_cast<unsigned long long>(cap),
                    static_cast<unsigned long long>(descs.size()));
  }
  if (!descs.empty()) {
    PF_REQUIRE_PTR(out);
    std::memcpy(out, descs.data(), descs.size() * sizeof(pf::CopyDesc));
  }
  return PF_OK;
}

}  // extern "C"
