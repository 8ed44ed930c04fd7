// Whole-row selection helpers shared by the beam-search and verify-logits kernels: a vocabulary
// row lives in the registers of one workgroup (THREADS threads, ITEMS values each).  The largest
// entries are found without sorting the row: a pivot with at least k entries above it comes from
// the per-thread maxima, entries >= pivot go to an LDS list (a private segment per wave: no
// atomics, a deterministic order), and the list is sorted by counting.  The per-element work is a
// load, a max and a compare; everything else touches only the ~2k listed entries.  Rows whose list
// overflows take a bisection on the value bits over the row in memory: slow, exact for any input.
#pragma once

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "rd_common.h"

namespace {

constexpr int kMaxRowWaves = 16;
constexpr int kCap = 2048;  // LDS candidate list
constexpr int kPivotMargin = 16;  // thread maxima taken beyond k when the pivot is chosen

template <typename T> struct Num;
// kValueBits: the leading bits of the float that can differ between two values of the type (the
// rest are zero): bf16 is the upper half of a float; a half has 10 mantissa bits behind the float's
// sign and 8 exponent bits (its subnormals become normal floats of at most 10 mantissa bits).
template <> struct Num<float> {
  static constexpr int kValueBits = 32;
  static __device__ float load(const float* p) { return *p; }
  static __device__ float round(float v) { return v; }
};
template <> struct Num<__hip_bfloat16> {
  static constexpr int kValueBits = 16;
  static __device__ float load(const __hip_bfloat16* p) { return __bfloat162float(*p); }
  static __device__ float round(float v) { return __bfloat162float(__float2bfloat16(v)); }
};
template <> struct Num<__half> {
  static constexpr int kValueBits = 19;
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

// Wave-wide reductions on the cross-lane data path of the vector ALU (no LDS round trips): two
// quad permutes and two mirrors reduce each row of 16 lanes, row_bcast:15 / row_bcast:31 carry the
// row results up to lane 63, which is read back as a wave-uniform value.
template <int CTRL, int ROW_MASK>
__device__ inline float dpp_move(float old, float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(old), __float_as_int(v), CTRL,
                                                    ROW_MASK, 0xf, false));
}
__device__ inline float wave_max(float v) {
  v = fmaxf(v, dpp_move<0xB1, 0xf>(v, v));   // quad_perm [1,0,3,2]
  v = fmaxf(v, dpp_move<0x4E, 0xf>(v, v));   // quad_perm [2,3,0,1]
  v = fmaxf(v, dpp_move<0x141, 0xf>(v, v));  // row_half_mirror
  v = fmaxf(v, dpp_move<0x140, 0xf>(v, v));  // row_mirror
  v = fmaxf(v, dpp_move<0x142, 0xa>(v, v));  // row_bcast:15 into rows 1 and 3
  v = fmaxf(v, dpp_move<0x143, 0xc>(v, v));  // row_bcast:31 into rows 2 and 3
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
__device__ inline float wave_sum(float v) {
  v += dpp_move<0xB1, 0xf>(0.f, v);
  v += dpp_move<0x4E, 0xf>(0.f, v);
  v += dpp_move<0x141, 0xf>(0.f, v);
  v += dpp_move<0x140, 0xf>(0.f, v);
  v += dpp_move<0x142, 0xa>(0.f, v);
  v += dpp_move<0x143, 0xc>(0.f, v);
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

constexpr int kKeyPad = 16;  // key lists are padded with zero keys to a multiple of this many

// Number of keys in list[0 .. n_pad) that are greater than `mine`.  n_pad is a multiple of kKeyPad
// (the list is padded with zero keys, which are below every real key).  Eight 16-byte LDS reads are
// issued before their results are used: one read per iteration would leave the loop waiting for
// the LDS latency every time (4 us for 256 keys; 0.5 us this way).
__device__ inline int count_greater(const unsigned long long* list, int n_pad, unsigned long long mine) {
  const ulonglong2* k2 = reinterpret_cast<const ulonglong2*>(list);
  int before = 0;
  for (int o = 0; 2 * o < n_pad; o += kKeyPad / 2) {
    ulonglong2 kk[kKeyPad / 2];
#pragma unroll
    for (int u = 0; u < kKeyPad / 2; ++u) kk[u] = k2[o + u];
#pragma unroll
    for (int u = 0; u < kKeyPad / 2; ++u) before += (kk[u].x > mine) + (kk[u].y > mine);
  }
  return before;
}
__device__ inline int pad_keys(int n) { return (n + kKeyPad - 1) / kKeyPad * kKeyPad; }

// Candidate list: WAVES segments of kCap / WAVES keys (+kKeyPad so that a segment can be padded
// with zero keys for count_greater); skey receives the same keys sorted descending.
template <int CAP>
struct RowSharedT {
  static constexpr int kCapacity = CAP;
  unsigned long long ckey[CAP + kKeyPad * kMaxRowWaves];
  unsigned long long skey[CAP];
  float red[kMaxRowWaves];
  unsigned long long red64[kMaxRowWaves];
  int ired[kMaxRowWaves];
  int seg_count[kMaxRowWaves];
  int n_surv;
  float logsum;
};
using RowShared = RowSharedT<kCap>;

__device__ inline float key_value(unsigned long long k) { return unord((uint32_t)(k >> 32)); }
__device__ inline int key_index(unsigned long long k) { return (int)(0xffffffffu - (uint32_t)k); }

template <int THREADS, typename SH>
__device__ inline float block_max(float v, SH& sh) {
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sh.red[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = sh.red[0];
  for (int w = 1; w < THREADS / 64; ++w) r = fmaxf(r, sh.red[w]);
  return r;
}
template <int THREADS, typename SH>
__device__ inline float block_min(float v, SH& sh) { return -block_max<THREADS>(-v, sh); }
template <int THREADS, typename SH>
__device__ inline float block_sum(float v, SH& sh) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sh.red[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = 0.f;
  for (int w = 0; w < THREADS / 64; ++w) r += sh.red[w];  // fixed order
  return r;
}
template <int THREADS, typename SH>
__device__ inline int block_isum(int v, SH& sh) {
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sh.ired[threadIdx.x >> 6] = v;
  __syncthreads();
  int r = 0;
  for (int w = 0; w < THREADS / 64; ++w) r += sh.ired[w];
  return r;
}
template <int THREADS, typename SH>
__device__ inline uint64_t block_max64(uint64_t v, SH& sh) {
  for (int off = 32; off > 0; off >>= 1) {
    const uint64_t o = __shfl_xor(v, off);
    v = o > v ? o : v;
  }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sh.red64[threadIdx.x >> 6] = v;
  __syncthreads();
  uint64_t r = sh.red64[0];
  for (int w = 1; w < THREADS / 64; ++w) r = sh.red64[w] > r ? sh.red64[w] : r;
  return r;
}

// Register j of a thread holds row index (j / VEC * THREADS + threadIdx.x) * VEC + j % VEC: 16-byte
// vectors interleaved over the workgroup.  row_index_at() gives that index from an opaque copy of
// threadIdx.x * VEC.  Loops over the register row call
// row_base() right before they start: with a plain threadIdx.x the compiler computes all ITEMS
// indices of every later loop at the top of the kernel and keeps them in registers.
template <int VEC>
__device__ inline int row_base() {
  int base = (int)threadIdx.x * VEC;
  asm volatile("" : "+v"(base));
  return base;
}
template <int VEC, int THREADS>
__device__ inline int row_index_at(int base, int j) {
  return base + (j / VEC) * THREADS * VEC + (j % VEC);
}

// Loads one row (V elements of T) into x[ITEMS] as float; slots past V hold NaN, which no
// comparison selects and fmaxf skips.
template <typename T, int ITEMS, int THREADS>
__device__ inline void load_row(const T* __restrict__ x_row, int V, float (&x)[ITEMS]) {
  constexpr int VEC = 16 / sizeof(T);
  constexpr int NV = ITEMS / VEC;
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int i0 = (c * THREADS + (int)threadIdx.x) * VEC;
    if (i0 + VEC <= V) {
      struct alignas(16) Pack { T v[VEC]; };
      const Pack p = *reinterpret_cast<const Pack*>(x_row + i0);
#pragma unroll
      for (int e = 0; e < VEC; ++e) x[c * VEC + e] = Num<T>::load(&p.v[e]);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) x[c * VEC + e] = (i0 + e < V) ? Num<T>::load(x_row + i0 + e) : __builtin_nanf("");
    }
  }
}

// Pivot with at least k_eff row entries >= it, from the per-thread maxima: the minimum over waves
// of each wave's r-th largest maximum, r = ceil(k_eff / waves) (-inf when a wave holds fewer).
// A wave finds its r-th largest by bisection on the bits of the ordered value: per bit one
// compare, one ballot and one scalar population count -- no LDS traffic, no cross-lane reductions
// (taking the maxima out one by one, r rounds of wave reductions, cost 2.4 us of the 9 us a quarter
// row took; ranking all maxima against each other through LDS was bound by the LDS bandwidth once
// eight workgroups shared a compute unit).  VALUE_BITS: Num<T>::kValueBits, the leading bits of the
// float in which two values of the row's type can differ (with fewer bits the result would still
// be a valid, only lower, pivot: longer candidate lists).
template <int THREADS, int VALUE_BITS, typename SH>
__device__ inline float row_pivot(float tmax, int k_eff, SH& sh) {
  constexpr int WAVES = THREADS / 64;
  const int r = (k_eff + WAVES - 1) / WAVES;
  const uint32_t key = ord(tmax);
  uint32_t found = 0u;  // wave-uniform: the largest value v with at least r lanes >= v
#pragma unroll
  for (int bit = 31; bit >= 32 - VALUE_BITS; --bit) {
    const uint32_t cand = found | (1u << bit);
    const int n = __builtin_popcountll(__ballot(key >= cand));
    found = n >= r ? cand : found;
  }
  // at or below the key of -inf: fewer than r lanes hold data
  const float wave_pivot = found <= 0x007fffffu ? -INFINITY : unord(found);
  return block_min<THREADS>(wave_pivot, sh);
}

// Lists key_of(x[j], row index) for every register entry >= pivot in per-wave segments of sh.ckey
// (sh.seg_count holds the segment lengths; a count above the segment size means overflow).  Ends
// with a barrier.  Returns the total, or -1 on overflow.
template <int ITEMS, int VEC, int THREADS, typename SH, typename KeyFn>
__device__ inline int row_list_candidates(const float (&x)[ITEMS], float pivot, SH& sh, KeyFn key_of) {
  constexpr int WAVES = THREADS / 64, SEG = SH::kCapacity / WAVES, STRIDE = SEG + kKeyPad;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  unsigned long long* seg = sh.ckey + wave * STRIDE;
  const int base = row_base<VEC>();
  int count = 0;  // wave-uniform
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const bool take = x[j] >= pivot;
    const uint64_t votes = __ballot(take);
    if (votes != 0) {
      if (take) {
        const int pos = count + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(votes >> 32),
                                     __builtin_amdgcn_mbcnt_lo((uint32_t)votes, 0u));
        if (pos < SEG) seg[pos] = key_of(x[j], row_index_at<VEC, THREADS>(base, j));
      }
      count += __builtin_popcountll(votes);
    }
  }
  if (lane == 0) sh.seg_count[wave] = count;
  // pad to a multiple of kKeyPad with keys below every real key
  if (lane < kKeyPad && count <= SEG) seg[count + lane] = 0ull;
  __syncthreads();
  int n = 0;
  bool overflow = false;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    const int c = sh.seg_count[w];
    overflow |= c > SEG;
    n += c;
  }
  return overflow ? -1 : n;
}
// The c-th listed key, c < total, in segment order.
template <int THREADS, typename SH>
__device__ inline unsigned long long row_listed_key(int c, const SH& sh) {
  constexpr int WAVES = THREADS / 64, SEG = SH::kCapacity / WAVES, STRIDE = SEG + kKeyPad;
  int w = 0, off = c;
  while (off >= sh.seg_count[w]) off -= sh.seg_count[w++];
  return sh.ckey[w * STRIDE + off];
}

// Lists key_of(x[j], row index) for every register entry >= pivot and sorts the list descending
// into sh.skey.  Returns the number of keys, or -1 when a wave's segment overflowed.  Keys must be
// distinct and nonzero (key64 of distinct indices is).  Ends with a barrier.
template <int ITEMS, int VEC, int THREADS, typename SH, typename KeyFn>
__device__ inline int row_sorted_candidates(const float (&x)[ITEMS], float pivot, SH& sh,
                                            KeyFn key_of) {
  constexpr int WAVES = THREADS / 64, SEG = SH::kCapacity / WAVES, STRIDE = SEG + kKeyPad;
  const int n = row_list_candidates<ITEMS, VEC, THREADS>(x, pivot, sh, key_of);
  if (n < 0) return -1;
  for (int c = threadIdx.x; c < n; c += THREADS) {
    const unsigned long long mine = row_listed_key<THREADS>(c, sh);
    int before = 0;
    for (int w2 = 0; w2 < WAVES; ++w2) before += count_greater(sh.ckey + w2 * STRIDE, pad_keys(sh.seg_count[w2]), mine);
    sh.skey[before] = mine;
  }
  __syncthreads();
  return n;
}

// Number of sorted keys whose value part is >= the value part of sh.skey[k - 1] (k <= n): the
// entries that are >= the k-th largest value, ties included.  Ends with a barrier.
template <int THREADS, typename SH>
__device__ inline int row_survivors(int n, int k, SH& sh) {
  const uint32_t thr_hi = (uint32_t)(sh.skey[k - 1] >> 32);
  for (int r = threadIdx.x; r < n; r += THREADS) {
    const bool in = (uint32_t)(sh.skey[r] >> 32) >= thr_hi;
    const bool next_in = r + 1 < n && (uint32_t)(sh.skey[r + 1] >> 32) >= thr_hi;
    if (in && !next_in) sh.n_surv = r + 1;
  }
  __syncthreads();
  return sh.n_surv;
}

// k-th largest value of round_T(x_row[i] - shift), i < V, for any input: radix selection on the
// ordered bit pattern, four passes over the row in memory (it sits in L2) with a 256-bin LDS
// histogram each.  This is the rare path; it reads memory rather than the caller's register copy so
// that it adds nothing to the caller's register budget.  Uses sh.ckey as the histogram.
template <typename T, int THREADS, typename SH>
__device__ inline float row_kth_radix(const T* __restrict__ x_row, int V, float shift, int k_eff,
                                      SH& sh) {
  int* hist = reinterpret_cast<int*>(sh.ckey);
  const int tid = threadIdx.x, lane = tid & 63;
  uint32_t prefix = 0u, known = 0u;  // bits of the answer found so far, and their mask
  int k = k_eff;                     // rank of the answer among the keys that match the prefix
  for (int shift_bits = 24; shift_bits >= 0; shift_bits -= 8) {
    __syncthreads();
    for (int i = tid; i < 256; i += THREADS) hist[i] = 0;
    __syncthreads();
    for (int i0 = 0; i0 < V; i0 += THREADS) {
      const int i = i0 + tid;
      bool live = false;
      int bin = 0;
      if (i < V) {
        const uint32_t key = ord(Num<T>::round(Num<T>::load(x_row + i) - shift));
        live = (key & known) == prefix;
        bin = (key >> shift_bits) & 255;
      }
      // tied rows put whole waves into one bin: the first live lane's bin is added once per wave
      const uint64_t lives = __ballot(live);
      if (lives == 0) continue;
      const int lead_bin = __shfl(bin, __builtin_ctzll(lives));
      const uint64_t same = __ballot(live && bin == lead_bin);
      if (lane == __builtin_ctzll(lives)) atomicAdd(&hist[lead_bin], __builtin_popcountll(same));
      if (live && bin != lead_bin) atomicAdd(&hist[bin], 1);
    }
    __syncthreads();
    if (tid == 0) {
      int above = 0, b = 255;
      for (; b > 0; --b) {
        if (above + hist[b] >= k) break;
        above += hist[b];
      }
      sh.ired[0] = b;
      sh.ired[1] = k - above;
    }
    __syncthreads();
    prefix |= (uint32_t)sh.ired[0] << shift_bits;
    known |= 255u << shift_bits;
    k = sh.ired[1];
  }
  __syncthreads();
  return unord(prefix);
}

// Launch geometry for a vocabulary of V elements: threads per row x values per thread (a multiple
// of the 16-byte vector for every dtype).  -1 when V is beyond the compiled limit.
//   V <= 8192        256 threads x 32
//   V <= 32768       256 threads x 128   (two workgroups per compute unit); the beam search uses
//                    512 threads x 64 when it has at most 512 rows
//   V <= 65536      1024 threads x 64
inline int row_geometry(int V) { return V <= 8192 ? 0 : (V <= 32768 ? 1 : (V <= 65536 ? 2 : -1)); }

}  // namespace
