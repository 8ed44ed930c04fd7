// Yardstick for the library's event timing: what timing a kernel costs (an empty kernel timed the
// same way).
#include <hip/hip_ext.h>

#include "rd_common.h"

namespace {
__global__ void null_kernel() {}

}  // namespace

extern "C" int rd_timing_null_kernel_us(int launches, void* stream, float* avg_us) {
  RD_REQUIRE(launches > 0 && launches <= 4096 && avg_us, RD_EINVAL, "rd_timing_null_kernel_us: bad arguments");
  hipStream_t s = rd::as_stream(stream);
  hipEvent_t t0, t1;
  RD_REQUIRE(hipEventCreate(&t0) == hipSuccess && hipEventCreate(&t1) == hipSuccess, RD_ELAUNCH,
             "rd_timing_null_kernel_us: hipEventCreate failed");
  double total = 0.0;
  int n = 0;
  for (int i = 0; i < launches; ++i) {
    hipExtLaunchKernelGGL(null_kernel, dim3(1), dim3(64), 0, s, t0, t1, 0);
    if (hipEventSynchronize(t1) != hipSuccess) break;
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, t0, t1) != hipSuccess) break;
    if (i > 0) { total += ms; ++n; }  // the first launch loads the code object
  }
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  RD_REQUIRE(n > 0 || launches == 1, RD_ELAUNCH, "rd_timing_null_kernel_us: timing failed");
  *avg_us = n ? (float)(total / n * 1e3) : 0.f;
  return RD_OK;
}
