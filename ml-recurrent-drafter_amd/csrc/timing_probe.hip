// Yardsticks for the measurements: what the event timing of a kernel costs (an empty kernel timed
// the same way), and what the memory system delivers to the verification attention's access
// pattern when nothing but the loads is done.
#include <hip/hip_ext.h>

#include "rd_common.h"

namespace {
__global__ void null_kernel() {}

// One 512-thread workgroup per (batch row, head) streams its K slab and its V slab in tiles of 64
// rows of 256 bytes, as attn_mfma_kernel does (threads 0-255 the K tile, 256-511 the V tile, four
// 16-byte loads per thread and tile, DEPTH tiles ahead in registers), stores each tile to LDS,
// meets at a barrier and reads it back: the loads, the staging and the barrier of the attention's
// tile loop without its arithmetic.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
constexpr int kStreamThreads = 512, kStreamTile = 64 * 256;
constexpr int kStreamLds = 90 * 1024;  // one workgroup per compute unit, as the attention kernel has

template <int DEPTH>
__global__ __launch_bounds__(kStreamThreads) void stream_tiles_kernel(const char* __restrict__ k, const char* __restrict__ v,
                                                                      int64_t slab_bytes, int tiles,
                                                                      unsigned* __restrict__ sink) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int tid = threadIdx.x, role = tid >> 8, lt = tid & 255;
  const char* base = (role ? v : k) + (int64_t)blockIdx.x * slab_bytes + (lt >> 4) * 256 + (lt & 15) * 16;
  u32x4 r[DEPTH][4];
#pragma unroll
  for (int j = 0; j < DEPTH; ++j) {
    const int t = j < tiles ? j : tiles - 1;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[j][i] = *reinterpret_cast<const u32x4*>(base + (int64_t)t * kStreamTile + i * 16 * 256);
  }
  u32x4 acc = {0, 0, 0, 0};
  for (int t0 = 0; t0 < tiles; t0 += DEPTH) {
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) {
      const int t = t0 + j;
      char* buf = lds + ((t & 1) * 2 + role) * kStreamTile + (lt >> 4) * 256 + (lt & 15) * 16;
#pragma unroll
      for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(buf + i * 16 * 256) = r[j][i];
      int nt = t + DEPTH;
      nt = nt < tiles ? nt : tiles - 1;  // (clamped, not skipped: the same loads on every path)
#pragma unroll
      for (int i = 0; i < 4; ++i) r[j][i] = *reinterpret_cast<const u32x4*>(base + (int64_t)nt * kStreamTile + i * 16 * 256);
      __syncthreads();
      const char* rd = lds + (t & 1) * 2 * kStreamTile + tid * 64;
#pragma unroll
      for (int i = 0; i < 4; ++i) acc ^= *reinterpret_cast<const u32x4*>(rd + 16 * i);
    }
  }
  sink[(int64_t)blockIdx.x * kStreamThreads + tid] = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
}
}  // namespace

extern "C" int rd_stream_tiles_probe(const void* k, const void* v, int64_t slab_bytes, int slabs, int tiles,
                                     int depth, void* sink, void* stream) {
  RD_REQUIRE(k && v && sink && slabs > 0 && slabs <= 65535 && tiles > 0, RD_EINVAL,
             "rd_stream_tiles_probe: bad arguments (slabs %d tiles %d)", slabs, tiles);
  RD_REQUIRE(slab_bytes >= (int64_t)tiles * kStreamTile && slab_bytes % 16 == 0 &&
                 ((uintptr_t)k & 15) == 0 && ((uintptr_t)v & 15) == 0, RD_EINVAL,
             "rd_stream_tiles_probe: a slab of %lld bytes does not hold %d tiles of %d bytes, or is not 16-byte aligned",
             (long long)slab_bytes, tiles, kStreamTile);
  RD_REQUIRE(depth == 1 || depth == 2 || depth == 4, RD_ELIMIT, "rd_stream_tiles_probe: depth %d (1, 2 or 4)", depth);
  hipStream_t s = rd::as_stream(stream);
#define RD_STREAM(D)                                                                                   \
  do {                                                                                                 \
    static bool once = false;                                                                          \
    if (!once) {                                                                                       \
      RD_REQUIRE(hipFuncSetAttribute(reinterpret_cast<const void*>(stream_tiles_kernel<D>),            \
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kStreamLds) == hipSuccess, \
                 RD_ELAUNCH, "rd_stream_tiles_probe: cannot reserve %d bytes of LDS", kStreamLds);      \
      once = true;                                                                                     \
    }                                                                                                  \
    rd::ScopedTiming rd_t("stream_tiles_kernel", s);                                                   \
    hipLaunchKernelGGL(stream_tiles_kernel<D>, dim3(slabs), dim3(kStreamThreads), kStreamLds, s,       \
                       reinterpret_cast<const char*>(k), reinterpret_cast<const char*>(v), slab_bytes, tiles, \
                       reinterpret_cast<unsigned*>(sink));                                             \
  } while (0)
  if (depth == 1) RD_STREAM(1); else if (depth == 2) RD_STREAM(2); else RD_STREAM(4);
#undef RD_STREAM
  return rd::check_launch("rd_stream_tiles_probe");
}

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
