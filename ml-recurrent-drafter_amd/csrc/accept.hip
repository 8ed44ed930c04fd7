// Candidate acceptance and sequence re-alignment planning (gfx950).  Integer / index work plus one
// bandwidth-bound reduction (row argmax over the vocabulary).
//   argmax_rows_kernel     first maximal index of every row (HBM-bound read of the logits)
//   accept_greedy_kernel   longest drafted prefix the LLM agrees with; first best beam
//   count_pads_kernel      leading pad run of every row of the token ids
//   realign_plan_kernel    new right-aligned ids, per-row shift plan for the KV cache
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "rd_common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;

template <typename T>
__device__ inline float to_float(T v);
template <>
__device__ inline float to_float<float>(float v) { return v; }
template <>
__device__ inline float to_float<__hip_bfloat16>(__hip_bfloat16 v) { return __bfloat162float(v); }
template <>
__device__ inline float to_float<__half>(__half v) { return __half2float(v); }

// Order used by torch.argmax: NaN is larger than everything; among equals the lower index wins.
__device__ inline bool better(float v, int64_t i, float bv, int64_t bi) {
  const bool vn = v != v, bn = bv != bv;
  if (vn || bn) return vn && (!bn || i < bi);
  return v > bv || (v == bv && i < bi);
}

template <typename T, int VEC>
__global__ __launch_bounds__(kThreads) void argmax_rows_kernel(const T* __restrict__ x,
                                                               int64_t row_stride, int64_t V,
                                                               int64_t* __restrict__ out,
                                                               const int64_t* __restrict__ out_index) {
  const T* row = x + (int64_t)blockIdx.x * row_stride;
  float bv = -INFINITY;
  int64_t bi = INT64_MAX;
  const int64_t nvec = V / VEC;
  struct alignas(sizeof(T) * VEC) Pack { T v[VEC]; };
  const Pack* rv = reinterpret_cast<const Pack*>(row);
  // A thread meets its elements in increasing index order, so within the thread "strictly greater,
  // or the first NaN" is the whole rule and the index can stay 32 bits wide (the vector ALU work per
  // element, not the memory, was what held this kernel at 3.5 TB/s); `better` settles the rest.
  if (V < 2147483647LL) {
    float tv = -INFINITY;
    int ti = -1;
    bool t_nan = false;
    for (int c = threadIdx.x; c < (int)nvec; c += kThreads) {
      const Pack p = rv[c];
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float v = to_float<T>(p.v[e]);
        const bool take = !t_nan && (v > tv || v != v || ti < 0);
        t_nan = t_nan || (take && v != v);
        tv = take ? v : tv;
        ti = take ? c * VEC + e : ti;
      }
    }
    if (ti >= 0) { bv = tv; bi = ti; }
  } else {
    for (int64_t c = threadIdx.x; c < nvec; c += kThreads) {
      const Pack p = rv[c];
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float v = to_float<T>(p.v[e]);
        const int64_t i = c * VEC + e;
        if (better(v, i, bv, bi)) { bv = v; bi = i; }
      }
    }
  }
  for (int64_t i = nvec * VEC + threadIdx.x; i < V; i += kThreads) {
    const float v = to_float<T>(row[i]);
    if (better(v, i, bv, bi)) { bv = v; bi = i; }
  }
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off);
    const int64_t oi = __shfl_xor(bi, off);
    if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
  }
  __shared__ float s_v[kWaves];
  __shared__ int64_t s_i[kWaves];
  if ((threadIdx.x & 63) == 0) { s_v[threadIdx.x >> 6] = bv; s_i[threadIdx.x >> 6] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kWaves; ++w)
      if (better(s_v[w], s_i[w], bv, bi)) { bv = s_v[w]; bi = s_i[w]; }
    out[out_index ? out_index[blockIdx.x] : (int64_t)blockIdx.x] = bi == INT64_MAX ? 0 : bi;
  }
}

// One workgroup per batch row, thread i scores beam i.
__global__ __launch_bounds__(kThreads) void accept_greedy_kernel(
    const int64_t* __restrict__ beams, const int64_t* __restrict__ llm_tokens,
    int64_t llm_row_stride, const int64_t* __restrict__ unpacker, int W, int L,
    int64_t* __restrict__ n_tokens_in_seq, int64_t* __restrict__ seq_in_beam,
    int64_t* __restrict__ next_token, int64_t* __restrict__ last_slot) {
  const int b = blockIdx.x;
  const int64_t* bm = beams + (int64_t)b * W * L;
  const int64_t* un = unpacker ? unpacker + (int64_t)b * W * L : nullptr;
  const int64_t* lt = llm_tokens + (int64_t)b * llm_row_stride;
  auto llm_at = [&](int i, int k) -> int64_t { return un ? lt[un[i * L + k]] : lt[i * L + k]; };
  // key = n * 2^16 + (65535 - i): the maximum is the longest match, lowest beam on ties
  int key = -1;
  for (int i = threadIdx.x; i < W; i += kThreads) {
    int n = 0;
    while (n < L - 1 && bm[i * L + n + 1] == llm_at(i, n)) ++n;
    const int k2 = (n << 16) | (65535 - i);
    key = k2 > key ? k2 : key;
  }
  for (int off = 32; off > 0; off >>= 1) {
    const int o = __shfl_xor(key, off);
    key = o > key ? o : key;
  }
  __shared__ int s_key[kWaves];
  if ((threadIdx.x & 63) == 0) s_key[threadIdx.x >> 6] = key;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kWaves; ++w) key = s_key[w] > key ? s_key[w] : key;
    const int n = key >> 16, s = 65535 - (key & 65535);
    n_tokens_in_seq[b] = n;
    seq_in_beam[b] = s;
    if (next_token) next_token[b] = llm_at(s, n);
    if (last_slot) last_slot[b] = un ? un[s * L + n] : (int64_t)s * L + n;
  }
}

__device__ inline int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

// pads[b] = index of the first id that is not the pad id (prev if the row is all pads).
__global__ __launch_bounds__(kThreads) void count_pads_kernel(const int64_t* __restrict__ ids,
                                                              int64_t row_stride, int64_t prev,
                                                              int64_t pad, int32_t* __restrict__ pads) {
  const int64_t* row = ids + (int64_t)blockIdx.x * row_stride;
  __shared__ int s_first;
  if (threadIdx.x == 0) s_first = (int)prev;
  __syncthreads();
  // chunks in increasing order; stop at the first chunk that holds a non-pad id
  for (int64_t base = 0; base < prev; base += kThreads) {
    const int64_t j = base + threadIdx.x;
    if (j < prev && row[j] != pad) atomicMin(&s_first, (int)j);
    __syncthreads();
    const int first = s_first;  // read between two barriers: the next round's atomics cannot race
    __syncthreads();
    if (first < prev) break;
  }
  if (threadIdx.x == 0) pads[blockIdx.x] = s_first;
}

// position_ids[b, t] = (prev - leading pads of row b) + offsets[b, t]: the pad count of
// count_pads_kernel and the two elementwise steps that follow it upstream, in one launch.
__global__ __launch_bounds__(kThreads) void position_ids_kernel(
    const int64_t* __restrict__ ids, int64_t row_stride, int64_t prev, int64_t pad,
    const int64_t* __restrict__ offsets, int64_t offsets_row_stride, int n,
    int64_t* __restrict__ out) {
  const int64_t* row = ids + (int64_t)blockIdx.x * row_stride;
  __shared__ int s_first;
  if (threadIdx.x == 0) s_first = (int)prev;
  __syncthreads();
  for (int64_t base = 0; base < prev; base += kThreads) {
    const int64_t j = base + threadIdx.x;
    if (j < prev && row[j] != pad) atomicMin(&s_first, (int)j);
    __syncthreads();
    const int first = s_first;
    __syncthreads();
    if (first < prev) break;
  }
  const int64_t start = prev - s_first;
  const int64_t* off = offsets + (int64_t)blockIdx.x * offsets_row_stride;
  for (int t = threadIdx.x; t < n; t += kThreads) out[(int64_t)blockIdx.x * n + t] = start + off[t];
}

// plan layout (int32): [0]=M, [1]=prev, [2]=L, [3]=0, then per row 4+L ints:
//   {old_pads, new_pads, n_new, live_len, src_row[0..L)}
__global__ __launch_bounds__(kThreads) void realign_plan_kernel(
    const int64_t* __restrict__ ids, int64_t ids_row_stride, int64_t prev,
    const int64_t* __restrict__ n_tokens_in_seq, const int64_t* __restrict__ seq_in_beam,
    const int64_t* __restrict__ beams, const int64_t* __restrict__ unpacker, int B, int W, int L,
    int64_t pad, const int32_t* __restrict__ pads, int32_t* __restrict__ plan,
    int64_t* __restrict__ new_ids, int32_t* __restrict__ kv_shift, int32_t* __restrict__ step_out) {
  const int b = blockIdx.x;
  int m = 0, accepted = 0;
  for (int r = threadIdx.x; r < B; r += kThreads) {
    const int n = clampi((int)n_tokens_in_seq[r], 0, L - 1);
    const int sl = (int)prev - pads[r] + n + 1;
    m = sl > m ? sl : m;
    accepted += n;
  }
  for (int off = 32; off > 0; off >>= 1) {
    const int o = __shfl_xor(m, off);
    m = o > m ? o : m;
    accepted += __shfl_xor(accepted, off);
  }
  __shared__ int s_m[kWaves], s_accepted[kWaves];
  if ((threadIdx.x & 63) == 0) { s_m[threadIdx.x >> 6] = m; s_accepted[threadIdx.x >> 6] = accepted; }
  __syncthreads();
  m = 0;
  accepted = 0;
  for (int w = 0; w < kWaves; ++w) { m = s_m[w] > m ? s_m[w] : m; accepted += s_accepted[w]; }

  const int old_pads = pads[b];
  // out-of-range inputs are clamped so that no access below can leave its buffer
  const int n_new = clampi((int)n_tokens_in_seq[b], 0, L - 1) + 1;
  const int live = (int)prev - old_pads;
  const int new_pads = m - live - n_new;
  const int s = clampi((int)seq_in_beam[b], 0, W - 1);
  int32_t* row_plan = plan + 4 + (int64_t)b * (4 + L);
  // With kv_shift the cache rows stay where they are: token column c of this row lives in cache row
  // c - kv_shift[b], the plan is written in cache rows (nothing moves, the accepted rows are appended
  // behind the live ones) and the shift takes up the change of the left padding instead.
  const int shift = kv_shift ? kv_shift[b] : 0;
  if (threadIdx.x == 0) {
    if (b == 0) {
      plan[0] = m; plan[1] = (int)prev; plan[2] = L; plan[3] = 0;
      if (step_out) { step_out[0] = m; step_out[1] = accepted; }
    }
    row_plan[0] = old_pads - shift;
    row_plan[1] = (kv_shift ? old_pads : new_pads) - shift;
    row_plan[2] = n_new; row_plan[3] = live;
  }
  for (int j = threadIdx.x; j < L; j += kThreads)
    row_plan[4 + j] = (int)prev - shift + (unpacker ? (int)unpacker[((int64_t)b * W + s) * L + j] : s * L + j);
  __syncthreads();  // every thread has read the old shift
  if (kv_shift && threadIdx.x == 0) kv_shift[b] = shift + new_pads - old_pads;

  int64_t* out = new_ids + (int64_t)b * m;
  const int64_t* in = ids + (int64_t)b * ids_row_stride;
  const int64_t* acc = beams + ((int64_t)b * W + s) * L;
  for (int p = threadIdx.x; p < m; p += kThreads) {
    const int q = p - new_pads;
    out[p] = q < 0 ? pad : (q < live ? in[old_pads + q] : acc[q - live]);
  }
}

template <typename T>
int launch_argmax(const void* x, int64_t rows, int64_t V, int64_t row_stride, int64_t* out,
                  const int64_t* out_index, hipStream_t s) {
  constexpr int VEC = 16 / sizeof(T);
  const bool vec_ok = ((uintptr_t)x % 16 == 0) && (row_stride % VEC == 0);
  if (vec_ok)
    { rd::ScopedTiming rd_t("argmax_rows_kernel", s); hipLaunchKernelGGL((argmax_rows_kernel<T, VEC>), dim3(rows), dim3(kThreads), 0, s,
                       reinterpret_cast<const T*>(x), row_stride, V, out, out_index); }
  else
    { rd::ScopedTiming rd_t("argmax_rows_kernel", s); hipLaunchKernelGGL((argmax_rows_kernel<T, 1>), dim3(rows), dim3(kThreads), 0, s,
                       reinterpret_cast<const T*>(x), row_stride, V, out, out_index); }
  return rd::check_launch("rd_argmax_rows");
}

}  // namespace

extern "C" int rd_argmax_rows(const void* x, int dtype, int64_t rows, int64_t vocab,
                              int64_t row_stride, int64_t* out, const int64_t* out_index, void* stream) {
  RD_REQUIRE(rows > 0 && vocab > 0 && row_stride >= vocab, RD_EINVAL,
             "rd_argmax_rows: rows %lld vocab %lld row_stride %lld", (long long)rows,
             (long long)vocab, (long long)row_stride);
  RD_REQUIRE(rows <= 2147483647LL, RD_ELIMIT, "rd_argmax_rows: too many rows");
  RD_REQUIRE(x && out, RD_EINVAL, "rd_argmax_rows: null pointer");
  hipStream_t s = rd::as_stream(stream);
  switch (dtype) {
    case RD_F32: return launch_argmax<float>(x, rows, vocab, row_stride, out, out_index, s);
    case RD_BF16: return launch_argmax<__hip_bfloat16>(x, rows, vocab, row_stride, out, out_index, s);
    case RD_F16: return launch_argmax<__half>(x, rows, vocab, row_stride, out, out_index, s);
    default: return rd::fail(RD_EINVAL, "rd_argmax_rows: unknown dtype %d", dtype);
  }
}

extern "C" int rd_accept_greedy(const int64_t* beams, const int64_t* llm_tokens,
                                int64_t llm_row_stride, const int64_t* unpacker, int batch,
                                int width, int length, int64_t* n_tokens_in_seq,
                                int64_t* seq_in_beam, int64_t* next_token, int64_t* last_slot,
                                void* stream) {
  RD_REQUIRE(batch > 0 && width > 0 && length > 0, RD_EINVAL,
             "rd_accept_greedy: batch/width/length must be positive (%d,%d,%d)", batch, width,
             length);
  RD_REQUIRE(width <= 65535 && length <= 32767, RD_ELIMIT, "rd_accept_greedy: width %d length %d",
             width, length);
  RD_REQUIRE(beams && llm_tokens && n_tokens_in_seq && seq_in_beam, RD_EINVAL,
             "rd_accept_greedy: null pointer");
  RD_REQUIRE(unpacker || llm_row_stride >= (int64_t)width * length, RD_EINVAL,
             "rd_accept_greedy: llm_row_stride %lld < width*length", (long long)llm_row_stride);
  { rd::ScopedTiming rd_t("accept_greedy_kernel", rd::as_stream(stream)); hipLaunchKernelGGL(accept_greedy_kernel, dim3(batch), dim3(kThreads), 0, rd::as_stream(stream),
                     beams, llm_tokens, llm_row_stride, unpacker, width, length, n_tokens_in_seq,
                     seq_in_beam, next_token, last_slot); }
  return rd::check_launch("rd_accept_greedy");
}

extern "C" size_t rd_realign_plan_ints(int batch, int length) {
  if (batch <= 0 || length <= 0) return 0;
  return 4 + (size_t)batch * (4 + length) + (size_t)batch;  // header, rows, scratch pad counts
}

extern "C" int rd_realign_plan(const int64_t* input_ids, int64_t ids_row_stride, int64_t prev,
                               const int64_t* n_tokens_in_seq, const int64_t* seq_in_beam,
                               const int64_t* beams, const int64_t* unpacker, int batch, int width,
                               int length, int64_t pad_token_id, int32_t* plan, int64_t* new_ids,
                               int32_t* kv_row_shift, const int32_t* left_pads, int32_t* step_out,
                               void* stream) {
  RD_REQUIRE(batch > 0 && width > 0 && length > 0 && prev >= 0, RD_EINVAL,
             "rd_realign_plan: bad sizes (batch %d width %d length %d prev %lld)", batch, width,
             length, (long long)prev);
  RD_REQUIRE(prev + length < 2147483647LL, RD_ELIMIT, "rd_realign_plan: prev too large");
  RD_REQUIRE(prev == 0 || ids_row_stride >= prev, RD_EINVAL, "rd_realign_plan: ids_row_stride < prev");
  RD_REQUIRE((prev == 0 || input_ids) && n_tokens_in_seq && seq_in_beam && beams && plan && new_ids,
             RD_EINVAL, "rd_realign_plan: null pointer");
  hipStream_t s = rd::as_stream(stream);
  const int32_t* pads = left_pads;
  if (pads == nullptr) {
    int32_t* own = plan + 4 + (size_t)batch * (4 + length);
    { rd::ScopedTiming rd_t("count_pads_kernel", s); hipLaunchKernelGGL(count_pads_kernel, dim3(batch), dim3(kThreads), 0, s, input_ids,
                       ids_row_stride, prev, pad_token_id, own); }
    if (int e = rd::check_launch("rd_realign_plan(pads)")) return e;
    pads = own;
  }
  { rd::ScopedTiming rd_t("realign_plan_kernel", s); hipLaunchKernelGGL(realign_plan_kernel, dim3(batch), dim3(kThreads), 0, s, input_ids,
                     ids_row_stride, prev, n_tokens_in_seq, seq_in_beam, beams, unpacker, batch,
                     width, length, pad_token_id, pads, plan, new_ids, kv_row_shift, step_out); }
  return rd::check_launch("rd_realign_plan");
}

extern "C" int rd_position_ids(const int64_t* input_ids, int64_t ids_row_stride, int64_t prev,
                               int batch, int64_t pad_token_id, const int64_t* position_offsets,
                               int64_t offsets_row_stride, int n, int64_t* position_ids,
                               void* stream) {
  RD_REQUIRE(batch > 0 && n > 0 && prev >= 0 && prev < 2147483647LL, RD_EINVAL,
             "rd_position_ids: batch %d n %d prev %lld", batch, n, (long long)prev);
  RD_REQUIRE((prev == 0 || input_ids) && position_offsets && position_ids, RD_EINVAL,
             "rd_position_ids: null pointer");
  RD_REQUIRE((prev == 0 || ids_row_stride >= prev) && offsets_row_stride >= n, RD_EINVAL,
             "rd_position_ids: a row stride is shorter than its row");
  { rd::ScopedTiming rd_t("position_ids_kernel", rd::as_stream(stream)); hipLaunchKernelGGL(position_ids_kernel, dim3(batch), dim3(kThreads), 0, rd::as_stream(stream),
                     input_ids, ids_row_stride, prev, pad_token_id, position_offsets,
                     offsets_row_stride, n, position_ids); }
  return rd::check_launch("rd_position_ids");
}

extern "C" int rd_count_left_paddings(const int64_t* input_ids, int64_t ids_row_stride,
                                      int64_t prev, int batch, int64_t pad_token_id,
                                      int32_t* pads, void* stream) {
  RD_REQUIRE(batch > 0 && prev >= 0 && prev < 2147483647LL, RD_EINVAL,
             "rd_count_left_paddings: batch %d prev %lld", batch, (long long)prev);
  RD_REQUIRE((prev == 0 || input_ids) && pads, RD_EINVAL, "rd_count_left_paddings: null pointer");
  RD_REQUIRE(prev == 0 || ids_row_stride >= prev, RD_EINVAL,
             "rd_count_left_paddings: ids_row_stride < prev");
  { rd::ScopedTiming rd_t("count_pads_kernel", rd::as_stream(stream)); hipLaunchKernelGGL(count_pads_kernel, dim3(batch), dim3(kThreads), 0, rd::as_stream(stream),
                     input_ids, ids_row_stride, prev, pad_token_id, pads); }
  return rd::check_launch("rd_count_left_paddings");
}
