// Whole-row selection helpers shared by the beam-search and verify-logits kernels: a vocabulary
// row lives in the registers of one 1024-thread workgroup; reductions go through wave shuffles and
// a few LDS words; the k-th largest value is found from a pivoted candidate list or, when that
// overflows, by bisection on the value bits.
#pragma once

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "rd_common.h"

namespace {

constexpr int kRowThreads = 1024;
constexpr int kRowWaves = kRowThreads / 64;
constexpr int kCap = 2048;       // LDS candidate list

template <typename T> struct Num;
template <> struct Num<float> {
  static __device__ float load(const float* p) { return *p; }
  static __device__ float round(float v) { return v; }
};
template <> struct Num<__hip_bfloat16> {
  static __device__ float load(const __hip_bfloat16* p) { return __bfloat162float(*p); }
  static __device__ float round(float v) { return __bfloat162float(__float2bfloat16(v)); }
};
template <> struct Num<__half> {
  static __device__ float load(const __half* p) { return __half2float(*p); }
  static __device__ float round(float v) { return __half2float(__float2half(v)); }
};

// Monotone map float -> uint32 (larger float, larger integer; -inf lowest of the finite order).
__device__ inline uint32_t ord(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ inline float unord(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}
// (score desc, index asc) as one integer: larger key = earlier in the result.
__device__ inline uint64_t key64(float score, uint32_t idx) {
  return ((uint64_t)ord(score) << 32) | (uint64_t)(0xffffffffu - idx);
}

__device__ inline float wave_max(float v) {
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  return v;
}
__device__ inline float wave_sum(float v) {
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

struct RowShared {
  float cval[kCap];
  int cidx[kCap];
  float red[kRowWaves];
  unsigned long long red64[kRowWaves];
  int ired[kRowWaves];
  int count;
  int n_surv;
  float thr;
  float logsum;
};

__device__ inline float block_max(float v, RowShared& sh) {
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sh.red[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = sh.red[0];
  for (int w = 1; w < kRowWaves; ++w) r = fmaxf(r, sh.red[w]);
  return r;
}
__device__ inline float block_min(float v, RowShared& sh) { return -block_max(-v, sh); }
__device__ inline float block_sum(float v, RowShared& sh) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sh.red[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = 0.f;
  for (int w = 0; w < kRowWaves; ++w) r += sh.red[w];  // fixed order
  return r;
}
__device__ inline int block_isum(int v, RowShared& sh) {
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sh.ired[threadIdx.x >> 6] = v;
  __syncthreads();
  int r = 0;
  for (int w = 0; w < kRowWaves; ++w) r += sh.ired[w];
  return r;
}
__device__ inline uint64_t block_max64(uint64_t v, RowShared& sh) {
  for (int off = 32; off > 0; off >>= 1) {
    const uint64_t o = __shfl_xor(v, off);
    v = o > v ? o : v;
  }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sh.red64[threadIdx.x >> 6] = v;
  __syncthreads();
  uint64_t r = sh.red64[0];
  for (int w = 1; w < kRowWaves; ++w) r = sh.red64[w] > r ? sh.red64[w] : r;
  return r;
}


// Row index held in register j of this thread: 16-byte vectors interleaved over the workgroup.
template <int VEC>
__device__ inline int row_index_of(int j) {
  return ((j / VEC) * kRowThreads + (int)threadIdx.x) * VEC + (j % VEC);
}

// Loads one row (V elements of T) into x[ITEMS] as float; slots past V hold -inf.
template <typename T, int ITEMS>
__device__ inline void load_row(const T* __restrict__ x_row, int V, float (&x)[ITEMS]) {
  constexpr int VEC = 16 / sizeof(T);
  constexpr int NV = ITEMS / VEC;
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int i0 = (c * kRowThreads + (int)threadIdx.x) * VEC;
    if (i0 + VEC <= V) {
      struct alignas(16) Pack { T v[VEC]; };
      const Pack p = *reinterpret_cast<const Pack*>(x_row + i0);
#pragma unroll
      for (int e = 0; e < VEC; ++e) x[c * VEC + e] = Num<T>::load(&p.v[e]);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) x[c * VEC + e] = (i0 + e < V) ? Num<T>::load(x_row + i0 + e) : -INFINITY;
    }
  }
}

// k-th largest value (with multiplicity) of the row held in x; every thread gets the result.
// Ordinary rows: pivot + LDS candidate list + counting.  Overflowing rows: 32-step bisection.
template <int ITEMS, int VEC>
__device__ inline float row_kth_largest(const float (&x)[ITEMS], int V, int k_eff, RowShared& sh,
                                        bool force_fallback) {
  const int tid = threadIdx.x, lane = tid & 63;
  float tmax = -INFINITY;
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) tmax = fmaxf(tmax, x[j]);
  const int rounds = (k_eff + kRowWaves - 1) / kRowWaves;
  float cur = tmax, wave_pivot = -INFINITY;
  for (int it = 0; it < rounds; ++it) {
    const float wm = wave_max(cur);
    wave_pivot = wm;
    const uint64_t holders = __ballot(cur == wm);
    if (holders != 0 && lane == __builtin_ctzll(holders)) cur = -INFINITY;
  }
  const float pivot = block_min(wave_pivot, sh);
  if (tid == 0) sh.count = 0;
  __syncthreads();
  if (!force_fallback) {
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      if (x[j] >= pivot && row_index_of<VEC>(j) < V) {
        const int pos = atomicAdd(&sh.count, 1);
        if (pos < kCap) sh.cval[pos] = x[j];
      }
    }
  }
  __syncthreads();
  const int n_c = force_fallback ? kCap + 1 : sh.count;
  if (n_c <= kCap) {
    for (int c = tid; c < n_c; c += kRowThreads) {
      const float v = sh.cval[c];
      int gt = 0, ge = 0;
      for (int o = 0; o < n_c; ++o) {
        const float ov = sh.cval[o];
        gt += ov > v;
        ge += ov >= v;
      }
      if (gt < k_eff && k_eff <= ge) sh.thr = v;
    }
    __syncthreads();
    return sh.thr;
  }
  uint32_t lo_k = 0u, hi_k = 0xffffffffu;  // invariant: count(>= lo_k) >= k_eff
  while (lo_k < hi_k) {
    const uint32_t mid = lo_k + (uint32_t)(((uint64_t)hi_k - lo_k + 1) >> 1);
    int cnt = 0;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) cnt += (row_index_of<VEC>(j) < V) && ord(x[j]) >= mid;
    cnt = block_isum(cnt, sh);
    if (cnt >= k_eff) lo_k = mid; else hi_k = mid - 1;
  }
  return unord(lo_k);
}

}  // namespace
