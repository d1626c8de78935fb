// Device memory handed over by another process: the export a worker makes of
// its KV cache tensors and the server-side registry that opens them.
//
// Stands in for the reference's CudaIPCWrapper (python/pegaflow/ipc_wrapper.py:
// 102-160: IPC handle of the tensor's storage + size + offset + GPU UUID) and
// CudaTensorRegistry (pegaflow-server/src/registry.rs:45-203: per context key,
// open every layer's handle once, hand `data_ptr` / `size_bytes` to the engine,
// keep the mapping alive until the context is dropped).  The reference goes
// through pickled torch objects; here the record is a plain struct and the
// mapping is a hipIpcOpenMemHandle kept by the registry.
#include <cstring>
#include <map>
#include <mutex>
#include <set>
#include <string>
#include <vector>

#include "pf_common.hpp"

namespace pf {

namespace {

using HandleKey = std::string;  // the 64 handle bytes

HandleKey key_of(const pf_ipc_tensor& t) {
  return std::string(reinterpret_cast<const char*>(t.handle), sizeof(t.handle));
}

int device_of_uuid(const uint8_t uuid[16], int* out) {
  int count = 0;
  PF_HIP(hipGetDeviceCount(&count));
  for (int d = 0; d < count; ++d) {
    hipUUID u;
    if (hipDeviceGetUuid(&u, d) != hipSuccess) {
      (void)hipGetLastError();
      continue;
    }
    if (std::memcmp(u.bytes, uuid, 16) == 0) {
      *out = d;
      return PF_OK;
    }
  }
  // ipc_wrapper.py:93-97
  return fail(PF_ERR_INVALID_ARGUMENT,
              "Device UUID not found in the discovered devices. Please make sure the process can "
              "see all the GPU devices.");
}

}  // namespace

// One opened allocation of another process; layers that live in the same
// allocation share it (a handle can be opened once per process).
struct OpenedAllocation {
  void* base = nullptr;
  uint64_t size = 0;
  int device = 0;
  size_t users = 0;
};

class TensorRegistry {
 public:
  ~TensorRegistry() { clear(); }

  int register_layers(const std::string& context_key, int device_id, uint64_t n,
                      const char* const* layer_names, const pf_ipc_tensor* tensors,
                      uint64_t* out_ptrs, uint64_t* out_sizes) {
    std::lock_guard<std::mutex> lock(mu_);
    if (contexts_.count(context_key)) {
      return fail(PF_ERR_INVALID_ARGUMENT, "context %s is already registered",
                  context_key.c_str());
    }
    std::set<std::string> seen;
    for (uint64_t i = 0; i < n; ++i) {
      if (!seen.insert(layer_names[i]).second) {
        return fail(PF_ERR_INVALID_ARGUMENT, "layer %s appears more than once in context %s",
                    layer_names[i], context_key.c_str());
      }
    }
    Context ctx;
    ctx.device_id = device_id;
    int status = PF_OK;
    int previous = 0;
    PF_HIP(hipGetDevice(&previous));
    for (uint64_t i = 0; i < n && status == PF_OK; ++i) {
      const pf_ipc_tensor& t = tensors[i];
      int device = -1;
      status = device_of_uuid(t.device_uuid, &device);
      if (status != PF_OK) break;
      if (device != device_id) {
        status = fail(PF_ERR_INVALID_ARGUMENT, "context %s is pinned to device %d but got %d",
                      context_key.c_str(), device_id, device);
        break;
      }
      if (t.size_bytes == 0 || t.offset > t.alloc_size || t.size_bytes > t.alloc_size - t.offset) {
        status = fail(PF_ERR_INVALID_ARGUMENT,
                      "layer %s: tensor [%llu, +%llu) does not fit its allocation of %llu bytes",
                      layer_names[i], static_cast<unsigned long long>(t.offset),
                      static_cast<unsigned long long>(t.size_bytes),
                      static_cast<unsigned long long>(t.alloc_size));
        break;
      }
      const HandleKey key = key_of(t);
      auto it = opened_.find(key);
      if (it == opened_.end()) {
        hipError_t e = hipSetDevice(device);
        hipIpcMemHandle_t handle;
        static_assert(sizeof(handle) == sizeof(t.handle), "handle size");
        std::memcpy(&handle, t.handle, sizeof(handle));
        void* base = nullptr;
        if (e == hipSuccess) e = hipIpcOpenMemHandle(&base, handle, hipIpcMemLazyEnablePeerAccess);
        if (e != hipSuccess) {
          fail_hip(e, "hipIpcOpenMemHandle");
          status = fail(PF_ERR_STORAGE, "register tensor failed: layer %s: %s", layer_names[i],
                        last_error().c_str());
          break;
        }
        OpenedAllocation a;
        a.base = base;
        a.size = t.alloc_size;
        a.device = device;
        it = opened_.emplace(key, a).first;
      }
      ++it->second.users;
      ctx.layers.push_back({layer_names[i], key});
      out_ptrs[i] = reinterpret_cast<uint64_t>(it->second.base) + t.offset;
      out_sizes[i] = t.size_bytes;
    }
    (void)hipSetDevice(previous);
    if (status != PF_OK) {
      const std::string message = last_error();
      release(ctx);
      last_error() = message;
      return status;
    }
    contexts_.emplace(context_key, std::move(ctx));
    return PF_OK;
  }

  // registry.rs:108-171: returns how many tensors were released.
  size_t drop_context(const std::string& context_key) {
    std::lock_guard<std::mutex> lock(mu_);
    auto it = contexts_.find(context_key);
    if (it == contexts_.end()) return 0;
    const size_t n = release(it->second);
    contexts_.erase(it);
    return n;
  }

  size_t drop_instance(const std::string& instance_id) {
    std::lock_guard<std::mutex> lock(mu_);
    const std::string prefix = instance_id + ":";
    size_t n = 0;
    for (auto it = contexts_.begin(); it != contexts_.end();) {
      if (it->first.compare(0, prefix.size(), prefix) == 0) {
        n += release(it->second);
        it = contexts_.erase(it);
      } else {
        ++it;
      }
    }
    return n;
  }

  size_t clear() {
    std::lock_guard<std::mutex> lock(mu_);
    size_t n = 0;
    for (auto& kv : contexts_) n += release(kv.second);
    contexts_.clear();
    return n;
  }

  size_t context_count() {
    std::lock_guard<std::mutex> lock(mu_);
    return contexts_.size();
  }

 private:
  struct Layer {
    std::string name;
    HandleKey allocation;
  };
  struct Context {
    int device_id = 0;
    std::vector<Layer> layers;
  };

  // mu_ held.  Closes an allocation when its last layer goes.
  size_t release(Context& ctx) {
    size_t n = 0;
    for (const Layer& l : ctx.layers) {
      auto it = opened_.find(l.allocation);
      if (it == opened_.end()) continue;
      ++n;
      if (--it->second.users == 0) {
        int previous = 0;
        (void)hipGetDevice(&previous);
        (void)hipSetDevice(it->second.device);
        (void)hipIpcCloseMemHandle(it->second.base);
        (void)hipSetDevice(previous);
        (void)hipGetLastError();
        opened_.erase(it);
      }
    }
    ctx.layers.clear();
    return n;
  }

  std::mutex mu_;
  std::map<std::string, Context> contexts_;
  std::map<HandleKey, OpenedAllocation> opened_;
};

}  // namespace pf

extern "C" {

int pf_device_uuid(int device, uint8_t out_uuid[16]) {
  PF_REQUIRE_PTR(out_uuid);
  hipUUID u;
  PF_HIP(hipDeviceGetUuid(&u, device));
  std::memcpy(out_uuid, u.bytes, 16);
  return PF_OK;
}

int pf_device_from_uuid(const uint8_t uuid[16], int* out_device) {
  PF_REQUIRE_PTR(uuid);
  PF_REQUIRE_PTR(out_device);
  return pf::device_of_uuid(uuid, out_device);
}

int pf_ipc_export(uint64_t dev_ptr, uint64_t size_bytes, pf_ipc_tensor* out) {
  PF_REQUIRE_PTR(out);
  if (dev_ptr == 0 || size_bytes == 0) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "pf_ipc_export needs a device pointer and a size");
  }
  std::memset(out, 0, sizeof(*out));
  hipPointerAttribute_t attr;
  PF_HIP(hipPointerGetAttributes(&attr, reinterpret_cast<void*>(dev_ptr)));
  if (attr.type != hipMemoryTypeDevice) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "pf_ipc_export: %#llx is not device memory",
                    static_cast<unsigned long long>(dev_ptr));
  }
  hipDeviceptr_t base = nullptr;
  size_t alloc_size = 0;
  PF_HIP(hipMemGetAddressRange(&base, &alloc_size, reinterpret_cast<hipDeviceptr_t>(dev_ptr)));
  const uint64_t offset = dev_ptr - reinterpret_cast<uint64_t>(base);
  if (size_bytes > alloc_size - offset) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT,
                    "pf_ipc_export: %llu bytes at offset %llu exceed the allocation of %llu bytes",
                    static_cast<unsigned long long>(size_bytes),
                    static_cast<unsigned long long>(offset),
                    static_cast<unsigned long long>(alloc_size));
  }
  hipIpcMemHandle_t handle;
  PF_HIP(hipIpcGetMemHandle(&handle, base));
  static_assert(sizeof(handle) == sizeof(out->handle), "handle size");
  std::memcpy(out->handle, &handle, sizeof(handle));
  out->alloc_size = alloc_size;
  out->offset = offset;
  out->size_bytes = size_bytes;
  hipUUID u;
  PF_HIP(hipDeviceGetUuid(&u, attr.device));
  std::memcpy(out->device_uuid, u.bytes, 16);
  return PF_OK;
}

int pf_registry_create(pf_tensor_registry_t* out) {
  PF_REQUIRE_PTR(out);
  *out = reinterpret_cast<pf_tensor_registry_t>(new pf::TensorRegistry());
  return PF_OK;
}

int pf_registry_destroy(pf_tensor_registry_t r) {
  delete reinterpret_cast<pf::TensorRegistry*>(r);
  return PF_OK;
}

int pf_registry_register_layers(pf_tensor_registry_t r, const char* context_key, int device_id,
                                uint64_t n_layers, const char* const* layer_names,
                                const pf_ipc_tensor* tensors, uint64_t* out_data_ptrs,
                                uint64_t* out_size_bytes) {
  PF_REQUIRE_PTR(r);
  PF_REQUIRE_PTR(context_key);
  if (n_layers != 0) {
    PF_REQUIRE_PTR(layer_names);
    PF_REQUIRE_PTR(tensors);
    PF_REQUIRE_PTR(out_data_ptrs);
    PF_REQUIRE_PTR(out_size_bytes);
  }
  if (device_id < 0) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "device_id %d must be >= 0", device_id);
  }
  return reinterpret_cast<pf::TensorRegistry*>(r)->register_layers(
      context_key, device_id, n_layers, layer_names, tensors, out_data_ptrs, out_size_bytes);
}

uint64_t pf_registry_drop_context(pf_tensor_registry_t r, const char* context_key) {
  return r && context_key ? reinterpret_cast<pf::TensorRegistry*>(r)->drop_context(context_key) : 0;
}

uint64_t pf_registry_drop_instance(pf_tensor_registry_t r, const char* instance_id) {
  return r && instance_id ? reinterpret_cast<pf::TensorRegistry*>(r)->drop_instance(instance_id) : 0;
}

uint64_t pf_registry_clear(pf_tensor_registry_t r) {
  return r ? reinterpret_cast<pf::TensorRegistry*>(r)->clear() : 0;
}

uint64_t pf_registry_context_count(pf_tensor_registry_t r) {
  return r ? reinterpret_cast<pf::TensorRegistry*>(r)->context_count() : 0;
}

int pf_server_register_context_batch(
    pf_engine_t e, pf_tensor_registry_t r, const char* instance_id, const char* namespace_,
    int device_id, uint64_t tp_rank, uint64_t pp_rank, uint64_t tp_size, uint64_t world_size,
    uint64_t n_layers, const char* const* layer_names, const pf_ipc_tensor* tensors,
    const uint64_t* num_blocks, const uint64_t* bytes_per_block, const uint64_t* kv_stride_bytes,
    const uint64_t* segments, const uint32_t* layer_group_ids, int transfer_mode, int page_first) {
  PF_REQUIRE_PTR(e);
  PF_REQUIRE_PTR(r);
  PF_REQUIRE_PTR(instance_id);
  // service.rs:127-148
  if (device_id < 0) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "device_id %d must be >= 0", device_id);
  }
  if (tp_size == 0) return pf::fail(PF_ERR_INVALID_ARGUMENT, "tp_size must be > 0");
  if (world_size == 0) return pf::fail(PF_ERR_INVALID_ARGUMENT, "world_size must be > 0");
  if (tp_rank >= tp_size) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "tp_rank %llu out of range (tp_size %llu)",
                    static_cast<unsigned long long>(tp_rank),
                    static_cast<unsigned long long>(tp_size));
  }
  if (n_layers == 0) {
    // service.rs:239-251
    return pf::fail(PF_ERR_INVALID_ARGUMENT,
                    "all layer arrays must have the same non-zero length (got layer_names=0)");
  }
  // service.rs:74-76
  const std::string context_key = std::string(instance_id) + ":tp" + std::to_string(tp_rank) +
                                  ":pp" + std::to_string(pp_rank) + ":dev" +
                                  std::to_string(device_id);
  std::vector<uint64_t> ptrs(n_layers), sizes(n_layers);
  int st = pf_registry_register_layers(r, context_key.c_str(), device_id, n_layers, layer_names,
                                       tensors, ptrs.data(), sizes.data());
  if (st != PF_OK) return st;
  st = pf_engine_register_context_layer_batch(
      e, instance_id, namespace_, device_id, tp_rank, pp_rank, tp_size, world_size, n_layers,
      layer_names, ptrs.data(), sizes.data(), num_blocks, bytes_per_block, kv_stride_bytes,
      segments, nullptr, layer_group_ids, transfer_mode, page_first);
  if (st != PF_OK) {
    // service.rs:326-336: a registration the engine refuses leaves no mapping behind.
    const std::string message = pf::last_error();
    (void)pf_registry_drop_context(r, context_key.c_str());
    pf::last_error() = message;
  }
  return st;
}

}  // extern "C"
