// Rotary position embedding of the new queries and keys, fused with the in-place append of the new
// keys and values to the KV cache (gfx950).
//
// Upstream (modeling_llama.py:87-110, 148-159; kv_cache.py:24-32) gathers cos/sin rows by
// position id, forms q*cos + rotate_half(q)*sin and the same for k with seven elementwise kernels
// and two concatenations, then copies k and v into the cache.  Here one kernel reads q, k, v once,
// writes the rotated q in place, and writes the rotated k and v straight to their cache rows.
//
// Rounding: every product and the sum are rounded to the tensors' dtype, as the separate torch
// kernels do (a product of two bf16/fp16 values is exact in float32, so one rounding per product
// and one for the sum reproduce them bit for bit); float32 uses unfused multiplies and adds.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "rd_common.h"

namespace {

constexpr int kThreads = 256;

template <typename T> struct Elem;
template <> struct Elem<float> {
  static __device__ float load(float v) { return v; }
  static __device__ float store(float v) { return v; }
};
template <> struct Elem<__hip_bfloat16> {
  static __device__ float load(__hip_bfloat16 v) { return __bfloat162float(v); }
  static __device__ __hip_bfloat16 store(float v) { return __float2bfloat16(v); }
};
template <> struct Elem<__half> {
  static __device__ float load(__half v) { return __half2float(v); }
  static __device__ __half store(float v) { return __float2half(v); }
};

template <typename T>
struct alignas(16) Vec {
  static constexpr int N = 16 / sizeof(T);
  T v[N];
};

// round_T(a * b) as a float.  Contraction is off in this file's arithmetic: a fused multiply-add
// would skip the rounding of the product that the separate torch kernels perform.
template <typename T>
__device__ inline float mul_rounded(float a, float b) {
#pragma clang fp contract(off)
  const float p = a * b;
  return Elem<T>::load(Elem<T>::store(p));
}
__device__ inline float add_unfused(float a, float b) {
#pragma clang fp contract(off)
  return a + b;
}
__device__ inline float sub_unfused(float a, float b) {
#pragma clang fp contract(off)
  return a - b;
}

struct RopeArgs {
  const void* q; const void* k; const void* v;  // (B, n, heads, D), head_dim contiguous
  int64_t q_sb, q_st, k_sb, k_st, v_sb, v_st;   // element strides of batch and token; head stride D
  const void* cos; const void* sin;             // (table_rows, D)
  int64_t table_rows;
  const int64_t* position_ids; int64_t pos_sb;  // (B, n)
  void* q_out; int64_t qo_sb, qo_st;            // (B, n, heads, D); may be q itself
  void* k_cache; void* v_cache;                 // (B, kv_heads, max_len, D)
  int64_t c_sb, c_sh, c_st;
  int64_t row0;                                 // first cache row written (before the row's shift)
  int64_t max_len;
  // Per batch row (or null): token column c of row b lives in cache row c - kv_shift[b].
  const int32_t* kv_shift;
  // Packed token rows (or null): token t of batch row b is row row_start[b] + t of q, k, v and
  // q_out (their batch strides are unused) and exists only for t < row_start[b+1] - row_start[b];
  // the cache rows of tokens that do not exist are left as they are.
  const int32_t* row_start;
  int n_new, n_heads, n_kv_heads, head_dim;
};

// One workgroup per (token, batch row).  A rotation task covers one 16-byte vector of the first
// half of a head and its partner in the second half; a copy task moves one vector of v.
template <typename T>
__global__ __launch_bounds__(kThreads) void rope_append_kernel(RopeArgs a) {
#pragma clang fp contract(off)
  using V = Vec<T>;
  constexpr int N = V::N;
  const int t = blockIdx.x, b = blockIdx.y;
  const int D = a.head_dim, half = D / 2;
  const int per_head = half / N;  // rotation tasks per head
  const int q_tasks = a.n_heads * per_head, k_tasks = a.n_kv_heads * per_head;
  const int v_tasks = a.n_kv_heads * (D / N);
  int64_t pos = a.position_ids[b * a.pos_sb + t];
  pos = pos < 0 ? 0 : (pos >= a.table_rows ? a.table_rows - 1 : pos);  // never read outside the table
  const T* cos_row = reinterpret_cast<const T*>(a.cos) + pos * D;
  const T* sin_row = reinterpret_cast<const T*>(a.sin) + pos * D;
  int64_t tok = t, in_batch = b;  // token row within the batch row's block, and which block
  if (a.row_start != nullptr) {
    const int r0 = a.row_start[b];
    if (t >= a.row_start[b + 1] - r0) return;
    tok = (int64_t)r0 + t;
    in_batch = 0;
  }
  const T* q_tok = reinterpret_cast<const T*>(a.q) + in_batch * a.q_sb + tok * a.q_st;
  const T* k_tok = reinterpret_cast<const T*>(a.k) + in_batch * a.k_sb + tok * a.k_st;
  const T* v_tok = reinterpret_cast<const T*>(a.v) + in_batch * a.v_sb + tok * a.v_st;
  T* qo_tok = reinterpret_cast<T*>(a.q_out) + in_batch * a.qo_sb + tok * a.qo_st;
  int64_t cache_row = a.row0 + t - (a.kv_shift ? a.kv_shift[b] : 0);
  // a shift that leaves the slab is never followed: q is still rotated, k and v are dropped
  const bool in_cache = cache_row >= 0 && cache_row < a.max_len;
  cache_row = in_cache ? cache_row : 0;
  T* kc = reinterpret_cast<T*>(a.k_cache) + b * a.c_sb + cache_row * a.c_st;
  T* vc = reinterpret_cast<T*>(a.v_cache) + b * a.c_sb + cache_row * a.c_st;
  const int n_tasks = in_cache ? q_tasks + k_tasks + v_tasks : q_tasks;

  for (int task = threadIdx.x; task < n_tasks; task += kThreads) {
    if (task >= q_tasks + k_tasks) {
      const int c = task - q_tasks - k_tasks;
      const int h = c / (D / N), d = (c % (D / N)) * N;
      *reinterpret_cast<V*>(vc + h * a.c_sh + d) = *reinterpret_cast<const V*>(v_tok + (int64_t)h * D + d);
      continue;
    }
    const bool is_q = task < q_tasks;
    const int c = is_q ? task : task - q_tasks;
    const int h = c / per_head, d = (c % per_head) * N;
    const T* src = (is_q ? q_tok : k_tok) + (int64_t)h * D;
    T* dst = is_q ? qo_tok + (int64_t)h * D : kc + h * a.c_sh;
    const V x1 = *reinterpret_cast<const V*>(src + d);
    const V x2 = *reinterpret_cast<const V*>(src + half + d);
    const V c1 = *reinterpret_cast<const V*>(cos_row + d), c2 = *reinterpret_cast<const V*>(cos_row + half + d);
    const V s1 = *reinterpret_cast<const V*>(sin_row + d), s2 = *reinterpret_cast<const V*>(sin_row + half + d);
    V o1, o2;
#pragma unroll
    for (int e = 0; e < N; ++e) {
      const float a1 = Elem<T>::load(x1.v[e]), a2 = Elem<T>::load(x2.v[e]);
      // rotate_half: (-x2, x1); (-x2)*sin rounds to -(x2*sin), and a + (-b) is a - b
      o1.v[e] = Elem<T>::store(sub_unfused(mul_rounded<T>(a1, Elem<T>::load(c1.v[e])),
                                           mul_rounded<T>(a2, Elem<T>::load(s1.v[e]))));
      o2.v[e] = Elem<T>::store(add_unfused(mul_rounded<T>(a2, Elem<T>::load(c2.v[e])),
                                           mul_rounded<T>(a1, Elem<T>::load(s2.v[e]))));
    }
    *reinterpret_cast<V*>(dst + d) = o1;
    *reinterpret_cast<V*>(dst + half + d) = o2;
  }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

extern "C" int rd_rope_append(const void* q, const int64_t* q_strides, const void* k,
                              const int64_t* k_strides, const void* v, const int64_t* v_strides,
                              int dtype, int batch, int n_new, int n_heads, int n_kv_heads,
                              int head_dim, const void* cos, const void* sin, int64_t table_rows,
                              const int64_t* position_ids, int64_t pos_batch_stride, void* q_out,
                              const int64_t* q_out_strides, void* k_cache, void* v_cache,
                              const int64_t* cache_strides, int64_t row0, int64_t max_len,
                              const int32_t* row_start, const int32_t* kv_row_shift, void* stream) {
  RD_REQUIRE(batch > 0 && n_new > 0 && n_heads > 0 && n_kv_heads > 0 && head_dim > 0, RD_EINVAL,
             "rd_rope_append: bad sizes (batch %d n_new %d heads %d kv_heads %d head_dim %d)", batch, n_new,
             n_heads, n_kv_heads, head_dim);
  RD_REQUIRE(batch <= 65535, RD_ELIMIT, "rd_rope_append: batch %d > 65535", batch);
  RD_REQUIRE(dtype == RD_F32 || dtype == RD_BF16 || dtype == RD_F16, RD_EINVAL, "rd_rope_append: unknown dtype %d", dtype);
  const int es = dtype == RD_F32 ? 4 : 2, vec = 16 / es;
  RD_REQUIRE(head_dim % (2 * vec) == 0, RD_ELIMIT, "rd_rope_append: head_dim %d must be a multiple of %d", head_dim, 2 * vec);
  RD_REQUIRE(q && k && v && cos && sin && position_ids && q_out && k_cache && v_cache && q_strides && k_strides &&
                 v_strides && q_out_strides && cache_strides, RD_EINVAL, "rd_rope_append: null pointer");
  RD_REQUIRE(table_rows > 0, RD_EINVAL, "rd_rope_append: empty cos/sin table");
  RD_REQUIRE(row0 >= 0 && row0 + n_new <= max_len, RD_EINVAL,
             "rd_rope_append: rows [%lld, %lld) do not fit max_len %lld", (long long)row0,
             (long long)(row0 + n_new), (long long)max_len);
  RD_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(cos) && aligned16(sin) && aligned16(q_out) &&
                 aligned16(k_cache) && aligned16(v_cache), RD_EINVAL, "rd_rope_append: pointers must be 16-byte aligned");
  const int64_t* all[] = {q_strides, k_strides, v_strides, q_out_strides};
  for (const int64_t* s : all)
    RD_REQUIRE(s[0] % vec == 0 && s[1] % vec == 0 && s[0] >= 0 && s[1] >= 0, RD_EINVAL,
               "rd_rope_append: token and batch strides must be non-negative multiples of %d elements", vec);
  RD_REQUIRE(cache_strides[0] % vec == 0 && cache_strides[1] % vec == 0 && cache_strides[2] % vec == 0 &&
                 cache_strides[2] >= head_dim, RD_EINVAL, "rd_rope_append: bad cache strides");
  RopeArgs a;
  a.q = q; a.k = k; a.v = v;
  a.q_sb = q_strides[0]; a.q_st = q_strides[1];
  a.k_sb = k_strides[0]; a.k_st = k_strides[1];
  a.v_sb = v_strides[0]; a.v_st = v_strides[1];
  a.cos = cos; a.sin = sin; a.table_rows = table_rows;
  a.position_ids = position_ids; a.pos_sb = pos_batch_stride;
  a.q_out = q_out; a.qo_sb = q_out_strides[0]; a.qo_st = q_out_strides[1];
  a.k_cache = k_cache; a.v_cache = v_cache;
  a.c_sb = cache_strides[0]; a.c_sh = cache_strides[1]; a.c_st = cache_strides[2];
  a.row0 = row0;
  a.max_len = max_len;
  a.kv_shift = kv_row_shift;
  a.row_start = row_start;
  a.n_new = n_new; a.n_heads = n_heads; a.n_kv_heads = n_kv_heads; a.head_dim = head_dim;
  hipStream_t s = rd::as_stream(stream);
  const dim3 grid(n_new, batch);
  {
    rd::ScopedTiming rd_t("rope_append_kernel", s);
    switch (dtype) {
      case RD_F32: hipLaunchKernelGGL(rope_append_kernel<float>, grid, dim3(kThreads), 0, s, a); break;
      case RD_BF16: hipLaunchKernelGGL(rope_append_kernel<__hip_bfloat16>, grid, dim3(kThreads), 0, s, a); break;
      default: hipLaunchKernelGGL(rope_append_kernel<__half>, grid, dim3(kThreads), 0, s, a); break;
    }
  }
  return rd::check_launch("rd_rope_append");
}
