// Bench-only yardstick (not part of libredrafter_hip.so or its C ABI; kernel_bench.py loads the
// shared object built from this file): what the memory system delivers to the verification
// attention's access pattern when nothing but the loads is done.
#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {
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

// `slabs` workgroups of 512 threads each stream `tiles` tiles of 64 rows x 256 bytes from their
// slab of k and of v (slab i begins at i * slab_bytes), `depth` (1, 2 or 4) tiles ahead in
// registers, through LDS and a barrier per tile -- the loads, staging and barrier of the
// attention's tile loop without its arithmetic.  sink: slabs * 512 uint32, written so that the
// loads cannot be dropped.  The kernel is launched `reps` times; *avg_us receives the mean of the
// kernels' own begin-to-end times (HIP events stamped by the launch), when avg_us is not null.
// Returns 0, -1 for bad arguments, -2 for an unsupported depth, -3 for a HIP error.
extern "C" __attribute__((visibility("default"))) int bench_stream_tiles(
    const void* k, const void* v, int64_t slab_bytes, int slabs, int tiles, int depth, void* sink, int reps,
    void* stream, float* avg_us) {
  if (!k || !v || !sink || slabs <= 0 || slabs > 65535 || tiles <= 0 || reps <= 0) return -1;
  if (slab_bytes < (int64_t)tiles * kStreamTile || slab_bytes % 16 != 0 || ((uintptr_t)k & 15) || ((uintptr_t)v & 15)) return -1;
  if (depth != 1 && depth != 2 && depth != 4) return -2;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  hipEvent_t t0 = nullptr, t1 = nullptr;
  if (avg_us && (hipEventCreate(&t0) != hipSuccess || hipEventCreate(&t1) != hipSuccess)) return -3;
  double total_ms = 0.0;
  int rc = 0;
  for (int i = 0; i < reps && rc == 0; ++i) {
#define RD_STREAM(DEPTH)                                                                                    \
    do {                                                                                                      \
      static bool once = false;                                                                               \
      if (!once) {                                                                                            \
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(stream_tiles_kernel<DEPTH>),                    \
                                hipFuncAttributeMaxDynamicSharedMemorySize, kStreamLds) != hipSuccess) { rc = -3; break; } \
        once = true;                                                                                          \
      }                                                                                                       \
      hipExtLaunchKernelGGL(stream_tiles_kernel<DEPTH>, dim3(slabs), dim3(kStreamThreads), kStreamLds, s, t0, t1, 0, \
                            reinterpret_cast<const char*>(k), reinterpret_cast<const char*>(v), slab_bytes, tiles, \
                            reinterpret_cast<unsigned*>(sink));                                               \
    } while (0)
    if (depth == 1) RD_STREAM(1); else if (depth == 2) RD_STREAM(2); else RD_STREAM(4);
#undef RD_STREAM
    if (rc == 0 && hipGetLastError() != hipSuccess) rc = -3;
    if (rc == 0 && avg_us) {
      float ms = 0.f;
      if (hipEventSynchronize(t1) != hipSuccess || hipEventElapsedTime(&ms, t0, t1) != hipSuccess) rc = -3;
      total_ms += ms;
    }
  }
  if (t0) (void)hipEventDestroy(t0);
  if (t1) (void)hipEventDestroy(t1);
  if (rc == 0 && avg_us) *avg_us = (float)(total_ms / reps * 1e3);
  return rc;
}
