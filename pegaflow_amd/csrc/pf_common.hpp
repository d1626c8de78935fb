// Shared internals of libpegahip: status codes, the thread-local error
// message, and HIP call checking.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "../../include/pegahip.h"

namespace pf {

// Last error message of the calling thread, read through pf_last_error().
std::string& last_error();

// Store a printf-formatted message and return `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Store "<what> failed: <hip error name> (<hip error string>)" and return the
// hipError_t as a positive status.
int fail_hip(hipError_t e, const char* what);

// Diagnostics on stderr, one line per call, prefixed "pegahip:".  The level comes
// from the environment variable PEGAHIP_LOG when the library is first used:
// "off", "info" (the default: one line per worker pool that is spawned) or
// "debug" (also one line per task, as the reference's workers log at debug
// level, gpu_worker.rs:465-474,511-520).
enum class LogLevel { Off = 0, Info = 1, Debug = 2 };
LogLevel log_level();
void log_line(LogLevel level, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

struct Stream {
  hipStream_t s = nullptr;
  bool owned = false;
};

struct Event {
  hipEvent_t e = nullptr;
};

inline hipStream_t native(pf_stream_t s) {
  return s ? reinterpret_cast<Stream*>(s)->s : nullptr;
}
inline hipEvent_t native(pf_event_t e) {
  return e ? reinterpret_cast<Event*>(e)->e : nullptr;
}

}  // namespace pf

#define PF_HIP(call)                                  \
  do {                                                \
    hipError_t pf_hip_status_ = (call);               \
    if (pf_hip_status_ != hipSuccess) {               \
      return ::pf::fail_hip(pf_hip_status_, #call);   \
    }                                                 \
  } while (0)

#define PF_REQUIRE_PTR(p)                                                    \
  do {                                                                       \
    if ((p) == nullptr) {                                                    \
      return ::pf::fail(PF_ERR_INVALID_ARGUMENT, "%s: %s must not be null",  \
                        __func__, #p);                                       \
    }                                                                        \
  } while (0)
