// Shared host-side helpers for the C-ABI entry points: error reporting and launch checks.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "redrafter_hip.h"

namespace rd {

// Thread-local message returned by rd_last_error().
char* error_buffer();
int fail(int code, const char* fmt, ...);

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// Checks the launch that was just enqueued; does not synchronise.
inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(RD_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
  return RD_OK;
}

// Optional per-kernel timing with HIP events on the launch stream (off by default; see
// rd_timing_enable).  Wrap one launch:  { rd::ScopedTiming t("kernel_name", stream); launch; }
struct ScopedTiming {
  ScopedTiming(const char* name, hipStream_t stream);
  ~ScopedTiming();
  ScopedTiming(const ScopedTiming&) = delete;
  ScopedTiming& operator=(const ScopedTiming&) = delete;

 private:
  hipStream_t stream_;
  int slot_;
};

// For launches made with hipExtLaunchKernelGGL, which stamps the two events with the kernel's own
// begin and end (no dispatch latency in between, unlike events recorded around a launch): hands
// out a pair from the timing pool, or two nulls when this kernel is not being timed.
void timing_events(const char* name, hipEvent_t* start, hipEvent_t* stop);

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

}  // namespace rd

#define RD_REQUIRE(cond, code, ...)                 \
  do {                                              \
    if (!(cond)) return rd::fail(code, __VA_ARGS__); \
  } while (0)
