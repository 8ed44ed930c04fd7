// Tree-masked verification attention over the pre-allocated KV cache (gfx950).
//
//   O[b,q,h,:] = softmax_k( Q[b,h,q,:] . K[b,hk,k,:] * scale  masked by bits[b,q,k] ) V[b,hk,k,:]
//
// K and V are strided views into the cache (no repeat_interleave copy, no additive bias tensor);
// the mask arrives as one uint64 per (query row, 64 keys) and is applied to the scores in
// registers; 64-key tiles in front of a row's first attended key are never loaded.
//
// Two kernels behind one entry point:
//   attn_mfma_kernel      bf16, head_dim 128: S^T = K Q^T and O^T = V^T P^T on
//                         v_mfma_f32_32x32x16_bf16.  512 threads = 8 waves, each wave owns 32 query
//                         rows; a 64-key K tile and the transposed V tile are staged in LDS (double
//                         buffered) and shared by the 8 waves; online softmax in fp32.  With the transposed
//                         products a query row lives in one lane pair, so the row maximum and sum
//                         need a single cross-lane exchange, and P^T is already laid out as the
//                         B operand of the second product.
//   attn_generic_kernel   any dtype, head_dim <= 256, one workgroup per (row, head, query); the
//                         correctness path for shapes the MFMA kernel does not cover.
// Work items come from the plan (attn_plan.h): (batch row, key range) chunks, longest first; rows
// whose keys are split over several items write fp32 partials that attn_combine_kernel merges.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "attn_plan.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct AttnArgs {
  const void* q; int64_t q_sb, q_sh, q_ss;
  const void* k; int64_t k_sb, k_sh, k_ss;
  const void* v; int64_t v_sb, v_sh, v_ss;
  void* out; int64_t o_sb, o_sh, o_ss;
  const uint64_t* bits;
  const int32_t* plan;
  float* part_o;   // [slot][n_q][D]
  float* part_ml;  // [slot][n_q][2]
  int B, H, Hkv, n_q, kv_len, words, max_splits, D;
  float scale;  // softmax scale; the MFMA kernel works in log2 units (scale * log2 e)
};

__device__ inline float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ---------------------------------------------------------------------------------------------
// MFMA kernel
// ---------------------------------------------------------------------------------------------
constexpr int kD = 128;
constexpr int kTile = 64;                  // keys per tile
constexpr int kWaves = 8;
constexpr int kMfmaThreads = kWaves * 64;  // 512
constexpr int kRowsPerWG = kWaves * 32;    // 256 query rows: K/V tiles are staged once per key range
constexpr int kBuffers = 2;                // LDS tile buffers (2: stage tile t+1 while t is consumed)
constexpr int kKsStride = kD + 8;          // bf16 elements; 272-byte rows spread 16 lanes over all banks
constexpr int kVtStride = kTile + 4;       // bf16 elements; 136-byte rows

// max over the two lanes (l, l^32) that share a query row
__device__ inline float pair_max(float v) {
  const unsigned u = __float_as_uint(v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);  // r[0]: low half's value, r[1]: high half's
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ inline float pair_sum(float v) {
  const unsigned u = __float_as_uint(v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

__global__ __launch_bounds__(kMfmaThreads) void attn_mfma_kernel(AttnArgs a) {
  __shared__ __attribute__((aligned(16))) __bf16 s_k[kBuffers][kTile * kKsStride];
  __shared__ __attribute__((aligned(16))) __bf16 s_vt[kBuffers][kD * kVtStride];

  const int item = blockIdx.y;
  if (item >= a.plan[0]) return;
  const int32_t* it = a.plan + RD_PLAN_HDR + 4 * a.B + 4 * item;
  const int b = it[0], lo = it[1], hi = it[2], split = it[3];
  const int n_splits = a.plan[RD_PLAN_HDR + 4 * b + 1];
  // query tiles of one (row, head, key range) are neighbours in dispatch order, so they run
  // together and the second read of the K/V tiles is served by the L2
  const int q_tiles = gridDim.x / a.H;
  const int h = blockIdx.x / q_tiles, q_tile = blockIdx.x - h * q_tiles;
  const int hk = h / (a.H / a.Hkv);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, r = lane & 31;
  const int q_row = q_tile * kRowsPerWG + wave * 32 + r;
  const bool wave_active = q_tile * kRowsPerWG + wave * 32 < a.n_q;
  const bool row_valid = q_row < a.n_q;

  const __bf16* kbase = reinterpret_cast<const __bf16*>(a.k) + (int64_t)b * a.k_sb + (int64_t)hk * a.k_sh;
  const __bf16* vbase = reinterpret_cast<const __bf16*>(a.v) + (int64_t)b * a.v_sb + (int64_t)hk * a.v_sh;

  // Q fragments: B operand of S^T = K Q^T; lane (r,g) holds Q[q_row][16*ks + 8*g .. +8)
  bf16x8 qf[8];
  {
    const __bf16* qp = reinterpret_cast<const __bf16*>(a.q) + (int64_t)b * a.q_sb + (int64_t)h * a.q_sh +
                       (int64_t)(row_valid ? q_row : 0) * a.q_ss + 8 * g;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
      qf[ks] = row_valid ? *reinterpret_cast<const bf16x8*>(qp + 16 * ks) : z;
    }
  }
  const uint64_t* brow = a.bits + ((int64_t)b * a.n_q + (row_valid ? q_row : 0)) * a.words;

  f32x16 o[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
  float m = -INFINITY, l = 0.f;  // m in log2 units (already scaled)
  const float scale_log2 = a.scale * 1.4426950408889634f;

  // Loader roles: threads [0,256) stage K rows (keys lrow+16*i), threads [256,512) stage V
  // transposed (keys 4*lrow+i); four 16-byte chunks each per tile.
  const bool k_loader = tid < 256;
  const int lt = tid & 255;
  const int chunk = lt & 15;  // 16-byte column chunk of a 256-byte row
  const int lrow = lt >> 4;
  bf16x8 pre[4];
  auto prefetch = [&](int key0) {
    const bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = key0 + (k_loader ? lrow + 16 * i : 4 * lrow + i);
      const __bf16* p = (k_loader ? kbase + (int64_t)key * a.k_ss : vbase + (int64_t)key * a.v_ss) + 8 * chunk;
      pre[i] = key < a.kv_len ? *reinterpret_cast<const bf16x8*>(p) : z;
    }
  };
  auto stage = [&](int buf) {
    if (k_loader) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        *reinterpret_cast<bf16x8*>(&s_k[buf][(lrow + 16 * i) * kKsStride + 8 * chunk]) = pre[i];
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        bf16x4 t = {pre[0][e], pre[1][e], pre[2][e], pre[3][e]};
        *reinterpret_cast<bf16x4*>(&s_vt[buf][(8 * chunk + e) * kVtStride + 4 * lrow]) = t;
      }
    }
  };

  const int n_tiles = (hi - lo + kTile - 1) / kTile;
  // Vector-memory loads complete in issue order, so a load that is needed soon must be issued
  // BEFORE the long-latency tile prefetch: the mask word of tile t+1 is fetched one iteration
  // ahead, in front of the K/V loads of tile t+2.
  uint64_t word_next = 0ull;
  if (n_tiles > 0) {
    word_next = row_valid ? brow[lo >> 6] : 0ull;
    prefetch(lo);
    stage(0);
    if (kBuffers == 2 && n_tiles > 1) prefetch(lo + kTile);
  }
  __syncthreads();
  for (int t = 0; t < n_tiles; ++t) {
    const int key0 = lo + t * kTile;
    const int buf = kBuffers == 2 ? (t & 1) : 0;
    if (kBuffers == 2) {
      // the other buffer was last read in iteration t-1, which every wave has left
      if (t + 1 < n_tiles) stage(buf ^ 1);
    }
    const uint64_t word = word_next;
    if (t + 1 < n_tiles) word_next = row_valid ? brow[(key0 + kTile) >> 6] : 0ull;
    if (t + kBuffers < n_tiles) prefetch(key0 + kBuffers * kTile);
    if (wave_active) {
      const __bf16* sk = s_k[buf];
      const __bf16* sv = s_vt[buf];
      // S^T tile: 64 keys x 32 queries, two 32x32 blocks
      f32x16 s[2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int i = 0; i < 16; ++i) s[kb][i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
          const bf16x8 ka = *reinterpret_cast<const bf16x8*>(&sk[(32 * kb + r) * kKsStride + 16 * ks + 8 * g]);
          s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qf[ks], s[kb], 0, 0, 0);
        }
      }
      // accumulator i of block kb is key 32*kb + 8*(i/4) + 4*g + i%4 of the tile
      if (!__all(word == ~0ull)) {
        const uint32_t w[2] = {(uint32_t)(word >> (4 * g)), (uint32_t)(word >> (32 + 4 * g))};
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const bool on = (w[kb] >> (8 * (i >> 2) + (i & 3))) & 1u;
            s[kb][i] = on ? s[kb][i] : -INFINITY;
          }
      }
      float tmax = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, s[kb][i]);
      tmax = pair_max(tmax) * scale_log2;
      // The running maximum only has to bound the exponents, not equal the true maximum: it is
      // raised (and O, l rescaled) only when the tile exceeds it by more than kSlack, so most
      // tiles skip the 64-register rescale.  p <= 2^kSlack stays far inside bf16/fp32 range.
      constexpr float kSlack = 8.f;
      const bool raise = tmax > m + kSlack || m == -INFINITY;
      if (__any(raise)) {
        const float m_new = raise ? tmax : m;
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = fast_exp2(m - m_safe);  // m == -inf -> 0 (o and l are 0 then)
        l *= alpha;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[db][i] *= alpha;
        m = m_new;
      }
      const float m_use = m == -INFINITY ? 0.f : m;
      float psum = 0.f;
      bf16x8 pf[4];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          const float p0 = fast_exp2(fmaf(s[kb][i], scale_log2, -m_use));
          const float p1 = fast_exp2(fmaf(s[kb][i + 1], scale_log2, -m_use));
          psum += p0 + p1;
          const f32x2 pp = {p0, p1};
          const bf16x2 pb = __builtin_convertvector(pp, bf16x2);
          pf[2 * kb + (i >> 3)][i & 7] = pb[0];
          pf[2 * kb + (i >> 3)][(i & 7) + 1] = pb[1];
        }
      l += psum;
      // O^T += V^T P^T ; k-slot j of lane group g is key 16*t + 4*g + (j%4) + 8*(j/4)
#pragma unroll
      for (int db = 0; db < 4; ++db) {
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
          const __bf16* vp = &sv[(32 * db + r) * kVtStride + 16 * tt + 4 * g];
          const bf16x4 v0 = *reinterpret_cast<const bf16x4*>(vp);
          const bf16x4 v1 = *reinterpret_cast<const bf16x4*>(vp + 8);
          const bf16x8 va = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
          o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pf[tt], o[db], 0, 0, 0);
        }
      }
    }
    __syncthreads();
    if (kBuffers == 1 && t + 1 < n_tiles) {
      stage(0);  // every wave has left tile t
      __syncthreads();
    }
  }

  if (!wave_active) return;
  l = pair_sum(l);
  if (!row_valid) return;
  // accumulator i of block db is d = 32*db + 8*(i/4) + 4*g + i%4
  if (n_splits == 1) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    __bf16* op = reinterpret_cast<__bf16*>(a.out) + (int64_t)b * a.o_sb + (int64_t)h * a.o_sh +
                 (int64_t)q_row * a.o_ss + 4 * g;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        bf16x4 w = {static_cast<__bf16>(o[db][4 * i4 + 0] * inv), static_cast<__bf16>(o[db][4 * i4 + 1] * inv),
                    static_cast<__bf16>(o[db][4 * i4 + 2] * inv), static_cast<__bf16>(o[db][4 * i4 + 3] * inv)};
        *reinterpret_cast<bf16x4*>(op + 32 * db + 8 * i4) = w;
      }
  } else {
    const int64_t slot = ((int64_t)b * a.H + h) * a.max_splits + split;
    float* po = a.part_o + (slot * a.n_q + q_row) * kD + 4 * g;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        f32x4 w = {o[db][4 * i4 + 0], o[db][4 * i4 + 1], o[db][4 * i4 + 2], o[db][4 * i4 + 3]};
        *reinterpret_cast<f32x4*>(po + 32 * db + 8 * i4) = w;
      }
    if (g == 0) {
      float* pm = a.part_ml + (slot * a.n_q + q_row) * 2;
      pm[0] = m;
      pm[1] = l;
    }
  }
}

// Merges the partials of rows whose keys were split (m in log2 units).  One workgroup per
// (head, batch row, query slice); rows that were not split cost one early exit per workgroup.
constexpr int kCombineSlices = 32;
__global__ __launch_bounds__(kD) void attn_combine_kernel(AttnArgs a) {
  const int h = blockIdx.x, b = blockIdx.y;
  const int n_splits = a.plan[RD_PLAN_HDR + 4 * b + 1];
  if (n_splits <= 1) return;
  const int d = threadIdx.x;
  const int64_t slot0 = ((int64_t)b * a.H + h) * a.max_splits;
  for (int q = blockIdx.z; q < a.n_q; q += kCombineSlices) {
    float mx = -INFINITY;
    for (int s = 0; s < n_splits; ++s) mx = fmaxf(mx, a.part_ml[((slot0 + s) * a.n_q + q) * 2]);
    float acc = 0.f, lsum = 0.f;
    if (mx > -INFINITY) {
      for (int s = 0; s < n_splits; ++s) {
        const float* pm = a.part_ml + ((slot0 + s) * a.n_q + q) * 2;
        const float w = fast_exp2(pm[0] - mx);
        lsum += w * pm[1];
        acc += w * a.part_o[((slot0 + s) * a.n_q + q) * kD + d];
      }
    }
    __bf16* op = reinterpret_cast<__bf16*>(a.out) + (int64_t)b * a.o_sb + (int64_t)h * a.o_sh + (int64_t)q * a.o_ss;
    op[d] = static_cast<__bf16>(lsum > 0.f ? acc / lsum : 0.f);
  }
}

// ---------------------------------------------------------------------------------------------
// Generic kernel: one workgroup per (query, head, batch row); keys in chunks of 256.
// ---------------------------------------------------------------------------------------------
constexpr int kGenThreads = 256;

template <typename T> __device__ inline float ld(const T* p);
template <> __device__ inline float ld<float>(const float* p) { return *p; }
template <> __device__ inline float ld<__hip_bfloat16>(const __hip_bfloat16* p) { return __bfloat162float(*p); }
template <> __device__ inline float ld<__half>(const __half* p) { return __half2float(*p); }
template <typename T> __device__ inline void st(T* p, float v);
template <> __device__ inline void st<float>(float* p, float v) { *p = v; }
template <> __device__ inline void st<__hip_bfloat16>(__hip_bfloat16* p, float v) { *p = __float2bfloat16(v); }
template <> __device__ inline void st<__half>(__half* p, float v) { *p = __float2half(v); }

__device__ inline float block_reduce(float v, bool is_max, float* s_tmp) {
  for (int off = 32; off > 0; off >>= 1) {
    const float o = __shfl_xor(v, off);
    v = is_max ? fmaxf(v, o) : v + o;
  }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) s_tmp[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = s_tmp[0];
  for (int w = 1; w < kGenThreads / 64; ++w) r = is_max ? fmaxf(r, s_tmp[w]) : r + s_tmp[w];
  return r;
}

template <typename T>
__global__ __launch_bounds__(kGenThreads) void attn_generic_kernel(AttnArgs a) {
  __shared__ float s_q[256];
  __shared__ float s_p[kGenThreads];
  __shared__ float s_tmp[kGenThreads / 64];
  const int q = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int hk = h / (a.H / a.Hkv);
  const int D = a.D, tid = threadIdx.x;
  const T* qp = reinterpret_cast<const T*>(a.q) + (int64_t)b * a.q_sb + (int64_t)h * a.q_sh + (int64_t)q * a.q_ss;
  const T* kb = reinterpret_cast<const T*>(a.k) + (int64_t)b * a.k_sb + (int64_t)hk * a.k_sh;
  const T* vb = reinterpret_cast<const T*>(a.v) + (int64_t)b * a.v_sb + (int64_t)hk * a.v_sh;
  if (tid < D) s_q[tid] = ld<T>(qp + tid) * a.scale;
  __syncthreads();
  const uint64_t* brow = a.bits + ((int64_t)b * a.n_q + q) * a.words;
  const int begin = a.plan[RD_PLAN_HDR + 4 * b + 0];
  float m = -INFINITY, l = 0.f, acc = 0.f;
  for (int c0 = begin; c0 < a.kv_len; c0 += kGenThreads) {
    const int j = c0 + tid;
    const bool on = j < a.kv_len && ((brow[j >> 6] >> (j & 63)) & 1ull);
    float sc = -INFINITY;
    if (on) {
      const T* kr = kb + (int64_t)j * a.k_ss;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot += s_q[d] * ld<T>(kr + d);
      sc = dot;
    }
    const float cmax = block_reduce(sc, true, s_tmp);
    const float m_new = fmaxf(m, cmax);
    if (m_new == -INFINITY) continue;  // uniform: nothing attended so far
    const float p = on ? __expf(sc - m_new) : 0.f;
    const float csum = block_reduce(p, false, s_tmp);
    const float alpha = __expf(m - m_new);
    l = l * alpha + csum;
    s_p[tid] = p;
    __syncthreads();
    if (tid < D) {
      acc *= alpha;
      const int n = (a.kv_len - c0) < kGenThreads ? (a.kv_len - c0) : kGenThreads;
      for (int jj = 0; jj < n; ++jj) {
        const float pj = s_p[jj];
        if (pj != 0.f) acc += pj * ld<T>(vb + (int64_t)(c0 + jj) * a.v_ss + tid);
      }
    }
    m = m_new;
    __syncthreads();
  }
  if (tid < D) {
    T* op = reinterpret_cast<T*>(a.out) + (int64_t)b * a.o_sb + (int64_t)h * a.o_sh + (int64_t)q * a.o_ss;
    st<T>(op + tid, l > 0.f ? acc / l : 0.f);
  }
}

bool mfma_eligible(const AttnArgs& a, int dtype) {
  auto al = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
  auto m8 = [](int64_t s) { return (s % 8) == 0; };
  return dtype == RD_BF16 && a.D == kD && al(a.q) && al(a.k) && al(a.v) && ((uintptr_t)a.out & 7) == 0 &&
         m8(a.q_sb) && m8(a.q_sh) && m8(a.q_ss) && m8(a.k_sb) && m8(a.k_sh) && m8(a.k_ss) &&
         m8(a.v_sb) && m8(a.v_sh) && m8(a.v_ss) && (a.o_sb % 4) == 0 && (a.o_sh % 4) == 0 &&
         (a.o_ss % 4) == 0;
}

}  // namespace

extern "C" size_t rd_attention_workspace_bytes(int batch, int n_heads, int n_q, int kv_len,
                                               int head_dim) {
  if (batch <= 0 || n_heads <= 0 || n_q <= 0 || kv_len <= 0 || head_dim <= 0) return 0;
  const size_t slots = (size_t)batch * n_heads * rd::attn_max_splits(kv_len);
  return rd::align_up(slots * n_q * head_dim * sizeof(float), 256) +
         rd::align_up(slots * n_q * 2 * sizeof(float), 256);
}

extern "C" int rd_verify_attention(const void* q, const int64_t* q_strides, const void* k,
                                   const int64_t* k_strides, const void* v,
                                   const int64_t* v_strides, void* out, const int64_t* o_strides,
                                   int dtype, int batch, int n_heads, int n_kv_heads, int n_q,
                                   int kv_len, int head_dim, float scale, const uint64_t* bits,
                                   const int32_t* plan, void* workspace, size_t workspace_bytes,
                                   int force_generic, void* stream) {
  RD_REQUIRE(batch > 0 && n_heads > 0 && n_kv_heads > 0 && n_q > 0 && kv_len > 0 && head_dim > 0,
             RD_EINVAL, "rd_verify_attention: bad sizes (batch %d heads %d kv_heads %d n_q %d kv %d D %d)",
             batch, n_heads, n_kv_heads, n_q, kv_len, head_dim);
  RD_REQUIRE(n_heads % n_kv_heads == 0, RD_EINVAL, "rd_verify_attention: heads %d not a multiple of kv heads %d",
             n_heads, n_kv_heads);
  RD_REQUIRE(head_dim <= 256, RD_ELIMIT, "rd_verify_attention: head_dim %d > 256", head_dim);
  RD_REQUIRE(batch <= 65535 && n_heads <= 65535, RD_ELIMIT, "rd_verify_attention: batch/heads > 65535");
  RD_REQUIRE(q && k && v && out && bits && plan && q_strides && k_strides && v_strides && o_strides,
             RD_EINVAL, "rd_verify_attention: null pointer");
  RD_REQUIRE(dtype == RD_BF16 || dtype == RD_F16 || dtype == RD_F32, RD_EINVAL,
             "rd_verify_attention: unknown dtype %d", dtype);
  AttnArgs a;
  a.q = q; a.q_sb = q_strides[0]; a.q_sh = q_strides[1]; a.q_ss = q_strides[2];
  a.k = k; a.k_sb = k_strides[0]; a.k_sh = k_strides[1]; a.k_ss = k_strides[2];
  a.v = v; a.v_sb = v_strides[0]; a.v_sh = v_strides[1]; a.v_ss = v_strides[2];
  a.out = out; a.o_sb = o_strides[0]; a.o_sh = o_strides[1]; a.o_ss = o_strides[2];
  a.bits = bits; a.plan = plan;
  a.B = batch; a.H = n_heads; a.Hkv = n_kv_heads; a.n_q = n_q; a.kv_len = kv_len;
  a.words = (kv_len + 63) / 64; a.max_splits = rd::attn_max_splits(kv_len); a.D = head_dim;
  a.scale = scale;
  a.part_o = nullptr; a.part_ml = nullptr;
  hipStream_t s = rd::as_stream(stream);

  if (!force_generic && mfma_eligible(a, dtype)) {
    const size_t need = rd_attention_workspace_bytes(batch, n_heads, n_q, kv_len, head_dim);
    RD_REQUIRE(workspace && workspace_bytes >= need, RD_EWORKSPACE,
               "rd_verify_attention: workspace %zu < %zu bytes", workspace_bytes, need);
    RD_REQUIRE(((uintptr_t)workspace & 255) == 0, RD_EINVAL, "rd_verify_attention: workspace not 256B aligned");
    const size_t slots = (size_t)batch * n_heads * a.max_splits;
    a.part_o = reinterpret_cast<float*>(workspace);
    a.part_ml = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) +
                                         rd::align_up(slots * n_q * head_dim * sizeof(float), 256));
    const int max_items = batch * a.max_splits;
    const int q_tiles = (n_q + kRowsPerWG - 1) / kRowsPerWG;
    RD_REQUIRE(max_items <= 65535 && (int64_t)q_tiles * n_heads <= 2147483647LL, RD_ELIMIT,
               "rd_verify_attention: grid too large");
    { rd::ScopedTiming rd_t("attn_mfma_kernel", s); hipLaunchKernelGGL(attn_mfma_kernel, dim3(n_heads * q_tiles, max_items), dim3(kMfmaThreads), 0, s, a); }
    if (int e = rd::check_launch("rd_verify_attention(mfma)")) return e;
    if (a.max_splits > 1) {
      { rd::ScopedTiming rd_t("attn_combine_kernel", s); hipLaunchKernelGGL(attn_combine_kernel, dim3(n_heads, batch, kCombineSlices), dim3(kD), 0, s, a); }
      return rd::check_launch("rd_verify_attention(combine)");
    }
    return RD_OK;
  }
  const dim3 grid(n_q, n_heads, batch);
  switch (dtype) {
    case RD_BF16: { rd::ScopedTiming rd_t("attn_generic_kernel", s); hipLaunchKernelGGL(attn_generic_kernel<__hip_bfloat16>, grid, dim3(kGenThreads), 0, s, a); } break;
    case RD_F16: { rd::ScopedTiming rd_t("attn_generic_kernel", s); hipLaunchKernelGGL(attn_generic_kernel<__half>, grid, dim3(kGenThreads), 0, s, a); } break;
    default: { rd::ScopedTiming rd_t("attn_generic_kernel", s); hipLaunchKernelGGL(attn_generic_kernel<float>, grid, dim3(kGenThreads), 0, s, a); } break;
  }
  return rd::check_launch("rd_verify_attention(generic)");
}
