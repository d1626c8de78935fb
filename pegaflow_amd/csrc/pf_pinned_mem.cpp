#include "pf_pinned_mem.hpp"

#include <sys/mman.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cstring>
#include <fstream>
#include <mutex>
#include <sstream>
#include <thread>
#include <vector>

#include "pf_common.hpp"

namespace pf {

uint64_t parse_huge_page_size(const std::string& meminfo) {
  std::istringstream in(meminfo);
  std::string line;
  while (std::getline(in, line)) {
    if (line.rfind("Hugepagesize:", 0) != 0) continue;
    std::istringstream fields(line);
    std::string key, value, unit, extra;
    fields >> key >> value >> unit;
    if (fields >> extra) return 0;
    if (unit != "kB" || value.empty()) return 0;
    uint64_t kb = 0;
    for (char c : value) {
      if (c < '0' || c > '9') return 0;
      kb = kb * 10 + static_cast<uint64_t>(c - '0');
    }
    return kb * 1024;
  }
  return 0;
}

uint64_t huge_page_size() {
  static std::once_flag once;
  static uint64_t cached = 0;
  std::call_once(once, [] {
    std::ifstream f("/proc/meminfo");
    std::stringstream ss;
    ss << f.rdbuf();
    cached = parse_huge_page_size(ss.str());
  });
  return cached;
}

uint64_t touch_threads(uint64_t size) {
  constexpr uint64_t kMinBytesPerThread = 1ull << 30;
  uint64_t by_size = std::max<uint64_t>((size + kMinBytesPerThread - 1) / kMinBytesPerThread, 1);
  uint64_t by_cpu = std::thread::hardware_concurrency();
  if (by_cpu == 0) by_cpu = 8;
  return std::min(by_size, by_cpu);
}

static uint64_t os_page_size() {
  long v = sysconf(_SC_PAGESIZE);
  return v > 0 ? static_cast<uint64_t>(v) : 4096;
}

void parallel_pre_touch(uint8_t* ptr, uint64_t size, NumaNode node) {
  if (size == 0) return;
  const uint64_t page = os_page_size();
  const uint64_t threads = touch_threads(size);
  const uint64_t chunk = (size + threads - 1) / threads;
  std::vector<std::thread> pool;
  for (uint64_t i = 0; i < threads; ++i) {
    uint64_t off = i * chunk;
    if (off >= size) break;
    uint64_t len = std::min(chunk, size - off);
    pool.emplace_back([=] {
      if (node.is_valid()) {
        std::string err;
        (void)pin_thread_to_numa_node(node, &err);
      }
      volatile uint8_t* p = ptr + off;
      for (uint64_t o = 0; o < len; o += page) p[o] = 0;
      p[len - 1] = 0;
    });
  }
  for (auto& t : pool) t.join();
}

static bool mapped_device_pointer(void* host, uint8_t** out, std::string* err, int* status) {
  void* dev = nullptr;
  hipError_t e = hipHostGetDevicePointer(&dev, host, 0);
  if (e != hipSuccess) {
    *status = fail_hip(e, "hipHostGetDevicePointer");
    *err = last_error();
    return false;
  }
  *out = static_cast<uint8_t*>(dev);
  return true;
}

std::unique_ptr<PinnedMemory> PinnedMemory::allocate(uint64_t size, AllocStrategy strategy,
                                                     NumaNode node, std::string* err,
                                                     int* status) {
  std::string local_err;
  int local_status = PF_OK;
  if (!err) err = &local_err;
  if (!status) status = &local_status;
  if (size == 0) {
    *err = "size must be greater than zero";
    *status = PF_ERR_INVALID_ARGUMENT;
    return nullptr;
  }
  std::unique_ptr<PinnedMemory> mem(new PinnedMemory());
  mem->strategy_ = strategy;

  if (strategy == AllocStrategy::HipHostAlloc) {
    void* p = nullptr;
    // Placement follows the calling thread's affinity; callers that want a
    // node wrap the call in run_on_numa (pinned_mem.rs:17-19).
    unsigned flags = hipHostMallocMapped | hipHostMallocPortable;
    if (node.is_valid()) flags |= hipHostMallocNumaUser;
    hipError_t e = hipHostMalloc(&p, size, flags);
    if (e != hipSuccess) {
      *status = fail_hip(e, "hipHostMalloc");
      *err = last_error();
      return nullptr;
    }
    mem->ptr_ = static_cast<uint8_t*>(p);
    mem->size_ = size;
    if (!mapped_device_pointer(p, &mem->device_ptr_, err, status)) {
      (void)hipHostFree(p);
      mem->ptr_ = nullptr;
      return nullptr;
    }
    return mem;
  }

  uint64_t aligned = size;
  int flags = MAP_PRIVATE | MAP_ANONYMOUS;
  if (strategy == AllocStrategy::HugePages) {
    uint64_t hp = huge_page_size();
    if (hp == 0) {
      *err = "cannot determine huge page size: Hugepagesize not found in /proc/meminfo";
      *status = PF_ERR_STORAGE;
      return nullptr;
    }
    aligned = (size + hp - 1) & ~(hp - 1);
    flags |= MAP_HUGETLB;
  }
  void* p = mmap(nullptr, aligned, PROT_READ | PROT_WRITE, flags, -1, 0);
  if (p == MAP_FAILED) {
    *err = std::string("mmap failed: ") + strerror(errno);
    *status = PF_ERR_STORAGE;
    return nullptr;
  }
  parallel_pre_touch(static_cast<uint8_t*>(p), aligned, node);
  hipError_t e = hipHostRegister(p, aligned, hipHostRegisterMapped);
  if (e != hipSuccess) {
    *status = fail_hip(e, "hipHostRegister");
    *err = last_error();
    munmap(p, aligned);
    return nullptr;
  }
  mem->ptr_ = static_cast<uint8_t*>(p);
  mem->size_ = aligned;
  if (!mapped_device_pointer(p, &mem->device_ptr_, err, status)) {
    (void)hipHostUnregister(p);
    munmap(p, aligned);
    mem->ptr_ = nullptr;
    return nullptr;
  }
  return mem;
}

PinnedMemory::~PinnedMemory() {
  if (!ptr_) return;
  if (strategy_ == AllocStrategy::HipHostAlloc) {
    hipError_t e = hipHostFree(ptr_);
    if (e != hipSuccess && e != hipErrorDeinitialized) {
      fprintf(stderr, "Warning: hipHostFree failed: %s\n", hipGetErrorName(e));
      (void)hipGetLastError();
    }
  } else {
    hipError_t e = hipHostUnregister(ptr_);
    if (e != hipSuccess && e != hipErrorDeinitialized) {
      fprintf(stderr, "Warning: hipHostUnregister failed: %s\n", hipGetErrorName(e));
      (void)hipGetLastError();
    }
    if (munmap(ptr_, size_) != 0) {
      fprintf(stderr, "Warning: munmap failed: %s\n", strerror(errno));
    }
  }
}

}  // namespace pf

extern "C" {

int pf_host_alloc(uint64_t size, int strategy, int numa_node, pf_host_mem* out) {
  PF_REQUIRE_PTR(out);
  if (strategy < 0 || strategy > 2) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "unknown host allocation strategy %d", strategy);
  }
  std::string err;
  int status = PF_OK;
  std::unique_ptr<pf::PinnedMemory> mem;
  pf::NumaNode node = pf::NumaNode::from_int(numa_node);
  auto strat = static_cast<pf::AllocStrategy>(strategy);
  if (node.is_valid() && strat == pf::AllocStrategy::HipHostAlloc) {
    // First-touch placement: allocate from a thread pinned to the node.
    int device = 0;
    (void)hipGetDevice(&device);
    std::string numa_err;
    bool ran = pf::run_on_numa(node, [&] {
      (void)hipSetDevice(device);
      mem = pf::PinnedMemory::allocate(size, strat, node, &err, &status);
    }, &numa_err);
    if (!ran) return pf::fail(PF_ERR_STORAGE, "%s", numa_err.c_str());
  } else {
    mem = pf::PinnedMemory::allocate(size, strat, node, &err, &status);
  }
  if (!mem) {
    pf::last_error() = err;
    return status;
  }
  out->host = mem->as_ptr();
  out->device = reinterpret_cast<uint64_t>(mem->device_ptr());
  out->size = mem->size();
  out->strategy = strategy;
  out->numa_node = numa_node;
  // Ownership of the region moves to the caller's struct; pf_host_free ends it.
  mem->disown();
  return PF_OK;
}

int pf_host_free(pf_host_mem* mem) {
  PF_REQUIRE_PTR(mem);
  if (!mem->host) return PF_OK;
  if (mem->strategy == PF_HOST_HIP_ALLOC) {
    PF_HIP(hipHostFree(mem->host));
  } else {
    hipError_t e = hipHostUnregister(mem->host);
    munmap(mem->host, mem->size);
    if (e != hipSuccess) return pf::fail_hip(e, "hipHostUnregister");
  }
  mem->host = nullptr;
  mem->device = 0;
  mem->size = 0;
  return PF_OK;
}

uint64_t pf_touch_threads(uint64_t size) { return pf::touch_threads(size); }

uint64_t pf_huge_page_size(void) { return pf::huge_page_size(); }

}  // extern "C"
