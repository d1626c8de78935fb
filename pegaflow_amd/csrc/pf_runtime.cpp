// Device, stream, event and raw device-memory entry points of the C ABI.
// These are thin: they exist so that a host-side binding needs no HIP headers.
#include <cstdlib>
#include <cstring>
#include <fstream>

#include "pf_common.hpp"
#include "pf_kernels.hpp"
#include "pf_numa.hpp"

namespace pf {

std::string& last_error() {
  thread_local std::string msg;
  return msg;
}

int fail(int code, const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  last_error() = buf;
  return code;
}

int fail_hip(hipError_t e, const char* what) {
  char buf[1024];
  snprintf(buf, sizeof(buf), "%s failed: %s (%s)", what, hipGetErrorName(e),
           hipGetErrorString(e));
  last_error() = buf;
  // Clear HIP's sticky per-thread error so it is not reported again by an
  // unrelated later call.
  (void)hipGetLastError();
  return static_cast<int>(e);
}

LogLevel log_level() {
  static const LogLevel level = [] {
    const char* v = std::getenv("PEGAHIP_LOG");
    if (v == nullptr) return LogLevel::Info;
    if (std::strcmp(v, "off") == 0 || std::strcmp(v, "0") == 0) return LogLevel::Off;
    if (std::strcmp(v, "debug") == 0) return LogLevel::Debug;
    return LogLevel::Info;
  }();
  return level;
}

void log_line(LogLevel level, const char* fmt, ...) {
  if (static_cast<int>(level) > static_cast<int>(log_level())) return;
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  fprintf(stderr, "pegahip: %s\n", buf);
}

}  // namespace pf

extern "C" {

const char* pf_last_error(void) { return pf::last_error().c_str(); }

const char* pf_version(void) { return "pegahip 0.1.0 (gfx950)"; }

int pf_device_count(int* out_count) {
  PF_REQUIRE_PTR(out_count);
  *out_count = 0;
  PF_HIP(hipGetDeviceCount(out_count));
  return PF_OK;
}

int pf_set_device(int device) {
  if (device < 0) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "device_id %d must be >= 0", device);
  }
  PF_HIP(hipSetDevice(device));
  return PF_OK;
}

int pf_get_device(int* out_device) {
  PF_REQUIRE_PTR(out_device);
  PF_HIP(hipGetDevice(out_device));
  return PF_OK;
}

int pf_device_synchronize(void) {
  PF_HIP(hipDeviceSynchronize());
  return PF_OK;
}

int pf_device_numa_node(int device, int* out_node) {
  PF_REQUIRE_PTR(out_node);
  *out_node = -1;
  char bdf[64] = {0};
  PF_HIP(hipDeviceGetPCIBusId(bdf, sizeof(bdf), device));
  *out_node = pf::numa_node_of_pci_device(bdf);
  return PF_OK;
}

int pf_device_name(int device, char* buf, size_t cap) {
  PF_REQUIRE_PTR(buf);
  hipDeviceProp_t prop;
  PF_HIP(hipGetDeviceProperties(&prop, device));
  snprintf(buf, cap, "%s (%s)", prop.name, prop.gcnArchName);
  return PF_OK;
}

int pf_stream_create(pf_stream_t* out) {
  PF_REQUIRE_PTR(out);
  hipStream_t s = nullptr;
  PF_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  auto* w = new pf::Stream();
  w->s = s;
  w->owned = true;
  *out = reinterpret_cast<pf_stream_t>(w);
  return PF_OK;
}

int pf_stream_wrap(void* hip_stream, pf_stream_t* out) {
  PF_REQUIRE_PTR(out);
  auto* w = new pf::Stream();
  w->s = reinterpret_cast<hipStream_t>(hip_stream);
  w->owned = false;
  *out = reinterpret_cast<pf_stream_t>(w);
  return PF_OK;
}

int pf_stream_destroy(pf_stream_t s) {
  if (!s) return PF_OK;
  auto* w = reinterpret_cast<pf::Stream*>(s);
  hipError_t e = hipSuccess;
  if (w->owned) e = hipStreamDestroy(w->s);
  delete w;
  if (e != hipSuccess) return pf::fail_hip(e, "hipStreamDestroy");
  return PF_OK;
}

int pf_streams_run_concurrently(pf_stream_t a, pf_stream_t b, int* out) {
  PF_REQUIRE_PTR(out);
  bool concurrent = false;
  const int st = pf::streams_run_concurrently(pf::native(a), pf::native(b), &concurrent);
  *out = concurrent ? 1 : 0;
  return st;
}

int pf_stream_synchronize(pf_stream_t s) {
  PF_HIP(hipStreamSynchronize(pf::native(s)));
  return PF_OK;
}

int pf_stream_wait_event(pf_stream_t s, pf_event_t e) {
  PF_REQUIRE_PTR(e);
  PF_HIP(hipStreamWaitEvent(pf::native(s), pf::native(e), 0));
  return PF_OK;
}

void* pf_stream_native(pf_stream_t s) { return pf::native(s); }

int pf_event_create(int enable_timing, pf_event_t* out) {
  PF_REQUIRE_PTR(out);
  hipEvent_t e = nullptr;
  PF_HIP(hipEventCreateWithFlags(&e, enable_timing ? hipEventDefault : hipEventDisableTiming));
  auto* w = new pf::Event();
  w->e = e;
  *out = reinterpret_cast<pf_event_t>(w);
  return PF_OK;
}

int pf_event_destroy(pf_event_t e) {
  if (!e) return PF_OK;
  auto* w = reinterpret_cast<pf::Event*>(e);
  hipError_t st = hipEventDestroy(w->e);
  delete w;
  if (st != hipSuccess) return pf::fail_hip(st, "hipEventDestroy");
  return PF_OK;
}

int pf_event_record(pf_event_t e, pf_stream_t s) {
  PF_REQUIRE_PTR(e);
  PF_HIP(hipEventRecord(pf::native(e), pf::native(s)));
  return PF_OK;
}

int pf_event_synchronize(pf_event_t e) {
  PF_REQUIRE_PTR(e);
  PF_HIP(hipEventSynchronize(pf::native(e)));
  return PF_OK;
}

int pf_event_query(pf_event_t e, int* out_done) {
  PF_REQUIRE_PTR(e);
  PF_REQUIRE_PTR(out_done);
  hipError_t st = hipEventQuery(pf::native(e));
  if (st == hipSuccess) {
    *out_done = 1;
    return PF_OK;
  }
  if (st == hipErrorNotReady) {
    (void)hipGetLastError();
    *out_done = 0;
    return PF_OK;
  }
  return pf::fail_hip(st, "hipEventQuery");
}

int pf_event_elapsed_ms(pf_event_t start, pf_event_t stop, float* out_ms) {
  PF_REQUIRE_PTR(start);
  PF_REQUIRE_PTR(stop);
  PF_REQUIRE_PTR(out_ms);
  PF_HIP(hipEventElapsedTime(out_ms, pf::native(start), pf::native(stop)));
  return PF_OK;
}

int pf_dev_malloc(uint64_t size, uint64_t* out_ptr) {
  PF_REQUIRE_PTR(out_ptr);
  if (size == 0) return pf::fail(PF_ERR_INVALID_ARGUMENT, "size must be greater than zero");
  void* p = nullptr;
  PF_HIP(hipMalloc(&p, size));
  *out_ptr = reinterpret_cast<uint64_t>(p);
  return PF_OK;
}

int pf_dev_free(uint64_t ptr) {
  if (ptr == 0) return PF_OK;
  PF_HIP(hipFree(reinterpret_cast<void*>(ptr)));
  return PF_OK;
}

int pf_dev_memset(uint64_t ptr, int value, uint64_t size) {
  PF_HIP(hipMemset(reinterpret_cast<void*>(ptr), value, size));
  PF_HIP(hipDeviceSynchronize());
  return PF_OK;
}

int pf_dev_copy_from_host(uint64_t dst, const void* src, uint64_t size) {
  PF_REQUIRE_PTR(src);
  PF_HIP(hipMemcpy(reinterpret_cast<void*>(dst), src, size, hipMemcpyHostToDevice));
  return PF_OK;
}

int pf_dev_copy_to_host(void* dst, uint64_t src, uint64_t size) {
  PF_REQUIRE_PTR(dst);
  PF_HIP(hipMemcpy(dst, reinterpret_cast<const void*>(src), size, hipMemcpyDeviceToHost));
  return PF_OK;
}

int pf_memcpy_h2d_async(uint64_t dst, const void* src, uint64_t size, pf_stream_t s) {
  PF_REQUIRE_PTR(src);
  PF_HIP(hipMemcpyHtoDAsync(reinterpret_cast<hipDeviceptr_t>(dst), const_cast<void*>(src), size,
                            pf::native(s)));
  return PF_OK;
}

int pf_memcpy_d2h_async(void* dst, uint64_t src, uint64_t size, pf_stream_t s) {
  PF_REQUIRE_PTR(dst);
  PF_HIP(hipMemcpyDtoHAsync(dst, reinterpret_cast<hipDeviceptr_t>(src), size, pf::native(s)));
  return PF_OK;
}

}  // extern "C"
