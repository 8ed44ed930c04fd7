// Speculative-sampling acceptance without the (batch, width, length, vocab) tensors (gfx950).
//
// Upstream filters the verify logits to their top 50 per row, unpacks them to every candidate
// position, takes a log-softmax of logits/T over the vocabulary, and then reads 4*B*W scalars and
// one vocabulary row per batch row out of those tensors.  Here:
//   row_stats_kernel       one pass over each PACKED logits row: 50th largest value, maximum and
//                          log-sum of the filtered, tempered row -> 4 floats per row
//   accept_sample_kernel   per batch row: u < exp(P - Q) at every drafted token, leading accepted
//                          run per beam, first beam with the longest run
//   residual_probs_kernel  per batch row: relu(P - Q) at the first rejected position, or P at the
//                          bonus position when a whole beam was accepted
// log P of a token is rebuilt on the fly from its logit and the row's 4 floats; a dense log P
// tensor is accepted as well (the form the upstream helper functions take).
#include "row_select.h"

namespace {

constexpr int kThreads = 256;

struct RowStats { float thr, zmax, log_sum, mask_z; };  // of z = filtered logits / T

template <typename T, int ITEMS, int THREADS>
__global__ __launch_bounds__(THREADS) void row_stats_kernel(
    const T* __restrict__ logits, int64_t row_stride, int V, int top_k, float mask_value,
    float temperature, RowStats* __restrict__ stats, int force_fallback) {
  constexpr int VEC = 16 / sizeof(T);
  __shared__ RowShared sh;
  const int tid = threadIdx.x;
  const T* x_row = logits + (int64_t)blockIdx.x * row_stride;
  float x[ITEMS];
  load_row<T, ITEMS, THREADS>(x_row, V, x);
  float tmax = -INFINITY;
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) tmax = fmaxf(tmax, x[j]);
  const float row_max = block_max<THREADS>(tmax, sh);
  const int k_eff = top_k < V ? top_k : V;
  const float zmax = row_max / temperature;
  const float mask_z = mask_value / temperature;
  // (a few more maxima than k_eff: the k-th largest key then sits well above the pivot's key, and
  // a tie between the two, which costs the slow path, takes that many equal values in a row)
  const float pivot = row_pivot<THREADS, Num<T>::kValueBits>(tmax, k_eff + kPivotMargin < THREADS ? k_eff + kPivotMargin : THREADS, sh);
  int n_c = -1;
  if (!force_fallback)
    n_c = row_sorted_candidates<ITEMS, VEC, THREADS>(
        x, pivot, sh, [](float v, int i) { return key64(v, (uint32_t)i); });
  if (n_c >= k_eff) {
    // the filter keeps skey[0 .. n_s); every other entry of the row counts as mask_z
    const int n_s = row_survivors<THREADS>(n_c, k_eff, sh);
    if (tid < 64) {
      float part = 0.f;
      for (int o = tid; o < n_s; o += 64) part += expf(key_value(sh.skey[o]) / temperature - zmax);
      part = wave_sum(part);
      if (tid == 0) {
        const float sum = part + (float)(V - n_s) * expf(mask_z - zmax);
        stats[blockIdx.x] = RowStats{key_value(sh.skey[k_eff - 1]), zmax, logf(sum), mask_z};
      }
    }
    return;
  }
  // exact path from memory
  const float thr = row_kth_radix<T, THREADS>(x_row, V, 0.f, k_eff, sh);
  float part = 0.f;
  for (int i = tid; i < V; i += THREADS) {
    const float v = Num<T>::load(x_row + i);
    part += expf((v >= thr ? v / temperature : mask_z) - zmax);
  }
  const float sum = block_sum<THREADS>(part, sh);
  if (tid == 0) stats[blockIdx.x] = RowStats{thr, zmax, logf(sum), mask_z};
}

__device__ inline float load_any(const void* p, int dtype, int64_t i) {
  switch (dtype) {
    case RD_BF16: return __bfloat162float(reinterpret_cast<const __hip_bfloat16*>(p)[i]);
    case RD_F16: return __half2float(reinterpret_cast<const __half*>(p)[i]);
    default: return reinterpret_cast<const float*>(p)[i];
  }
}

// Where log P comes from: a dense (B,W,L,V) float tensor, or packed logits + per-row stats.
struct LogPSource {
  const float* dense; int64_t d_sb, d_sw, d_sk;  // element strides; vocabulary contiguous
  const void* logits; int dtype; int64_t l_sb, l_sr;  // packed (B, n, V): batch and row strides
  const RowStats* stats; int n_rows;              // (B, n_rows)
  const int64_t* unpacker;                        // (B, W, L)
  float temperature;
};

__device__ inline float log_p(const LogPSource& s, int b, int i, int k, int W, int L, int64_t tok) {
  if (s.dense) return s.dense[b * s.d_sb + i * s.d_sw + k * s.d_sk + tok];
  const int64_t slot = s.unpacker[((int64_t)b * W + i) * L + k];
  const RowStats st = s.stats[(int64_t)b * s.n_rows + slot];
  const float x = load_any(s.logits, s.dtype, b * s.l_sb + slot * s.l_sr + tok);
  return (x >= st.thr ? x / s.temperature : st.mask_z) - st.zmax - st.log_sum;
}

__global__ __launch_bounds__(kThreads) void accept_sample_kernel(
    const int64_t* __restrict__ beams, LogPSource p, const float* __restrict__ log_q, int64_t q_sb,
    int64_t q_sw, int64_t q_sk, const float* __restrict__ uniforms, int W, int L, int V,
    int64_t* __restrict__ n_tokens_in_seq, int64_t* __restrict__ seq_in_beam) {
  const int b = blockIdx.x;
  int key = -1;
  for (int i = threadIdx.x; i < W; i += kThreads) {
    int n = 0;
    for (int k = 0; k < L - 1; ++k) {
      int64_t tok = beams[((int64_t)b * W + i) * L + k + 1];
      tok = tok < 0 ? 0 : (tok >= V ? V - 1 : tok);  // a corrupt id must not leave the row
      const float lp = log_p(p, b, i, k, W, L, tok);
      const float lq = log_q[b * q_sb + i * q_sw + k * q_sk + tok];
      if (uniforms[((int64_t)b * W + i) * (L - 1) + k] < expf(lp - lq)) ++n; else break;
    }
    const int k2 = (n << 16) | (65535 - i);
    key = k2 > key ? k2 : key;
  }
  for (int off = 32; off > 0; off >>= 1) {
    const int o = __shfl_xor(key, off);
    key = o > key ? o : key;
  }
  __shared__ int s_key[kThreads / 64];
  if ((threadIdx.x & 63) == 0) s_key[threadIdx.x >> 6] = key;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kThreads / 64; ++w) key = s_key[w] > key ? s_key[w] : key;
    n_tokens_in_seq[b] = key >> 16;
    seq_in_beam[b] = 65535 - (key & 65535);
  }
}

__global__ __launch_bounds__(kThreads) void residual_probs_kernel(
    LogPSource p, const float* __restrict__ log_q, int64_t q_sb, int64_t q_sw, int64_t q_sk,
    const int64_t* __restrict__ seq_in_beam, const int64_t* __restrict__ n_tokens_in_seq, int W,
    int L, int V, float* __restrict__ probs) {
  const int b = blockIdx.y;
  int s = (int)seq_in_beam[b], n = (int)n_tokens_in_seq[b];
  s = s < 0 ? 0 : (s >= W ? W - 1 : s);
  n = n < 0 ? 0 : (n > L - 1 ? L - 1 : n);
  const bool whole = n == L - 1;  // the whole beam was accepted: sample the bonus position
  const int k = n;                // position of P: first rejected, or the bonus position L-1
  float* out = probs + (int64_t)b * V;
  for (int v = blockIdx.x * kThreads + threadIdx.x; v < V; v += gridDim.x * kThreads) {
    const float pv = expf(log_p(p, b, s, k, W, L, v));
    if (whole) out[v] = pv;
    else {
      const float d = pv - expf(log_q[b * q_sb + s * q_sw + n * q_sk + v]);
      out[v] = d > 0.f ? d : 0.f;
    }
  }
}

int fill_source(LogPSource& src, const float* dense, const int64_t* dense_strides, const void* logits,
                int dtype, const int64_t* logits_strides, const void* stats, int n_rows,
                const int64_t* unpacker, float temperature, const char* who) {
  src = LogPSource{};
  src.temperature = temperature;
  if (dense) {
    RD_REQUIRE(dense_strides, RD_EINVAL, "%s: dense log-probs need strides", who);
    src.dense = dense; src.d_sb = dense_strides[0]; src.d_sw = dense_strides[1]; src.d_sk = dense_strides[2];
    return RD_OK;
  }
  RD_REQUIRE(logits && logits_strides && stats && unpacker && n_rows > 0, RD_EINVAL,
             "%s: need either dense log-probs or packed logits + stats + unpacker", who);
  RD_REQUIRE(dtype == RD_BF16 || dtype == RD_F16 || dtype == RD_F32, RD_EINVAL, "%s: unknown dtype %d", who, dtype);
  RD_REQUIRE(temperature > 0.f, RD_EINVAL, "%s: temperature must be positive", who);
  src.logits = logits; src.dtype = dtype; src.l_sb = logits_strides[0]; src.l_sr = logits_strides[1];
  src.stats = reinterpret_cast<const RowStats*>(stats); src.n_rows = n_rows; src.unpacker = unpacker;
  return RD_OK;
}

template <typename T>
int launch_stats(const void* logits, int64_t row_stride, int64_t rows, int V, int top_k, float mask_value,
                 float temperature, void* stats, int force_fallback, hipStream_t s) {
  const T* x = reinterpret_cast<const T*>(logits);
  RowStats* st = reinterpret_cast<RowStats*>(stats);
#define RD_STATS(ITEMS, THREADS)                                                                     \
  do { rd::ScopedTiming rd_t("row_stats_kernel", s);                                                 \
    hipLaunchKernelGGL((row_stats_kernel<T, ITEMS, THREADS>), dim3(rows), dim3(THREADS), 0, s, x,    \
                       row_stride, V, top_k, mask_value, temperature, st, force_fallback); } while (0)
  switch (row_geometry(V)) {
    case 0: RD_STATS(32, 256); break;
    case 1: RD_STATS(128, 256); break;
    default: RD_STATS(64, 1024); break;
  }
#undef RD_STATS
  return rd::check_launch("rd_verify_row_stats");
}

}  // namespace

extern "C" int rd_verify_row_stats(const void* logits, int dtype, int64_t row_stride, int64_t rows,
                                   int vocab, int top_k, float mask_value, float temperature,
                                   float* stats, int force_fallback, void* stream) {
  RD_REQUIRE(rows > 0 && vocab > 0 && top_k > 0 && rows <= 2147483647LL, RD_EINVAL,
             "rd_verify_row_stats: bad sizes (rows %lld vocab %d top_k %d)", (long long)rows, vocab, top_k);
  RD_REQUIRE(row_geometry(vocab) >= 0 && top_k <= 512, RD_ELIMIT,
             "rd_verify_row_stats: vocab %d (<= 65536), top_k %d (<= 512)", vocab, top_k);
  RD_REQUIRE(logits && stats, RD_EINVAL, "rd_verify_row_stats: null pointer");
  RD_REQUIRE(temperature > 0.f, RD_EINVAL, "rd_verify_row_stats: temperature must be positive");
  RD_REQUIRE(dtype == RD_F32 || dtype == RD_BF16 || dtype == RD_F16, RD_EINVAL, "rd_verify_row_stats: unknown dtype %d", dtype);
  const int es = dtype == RD_F32 ? 4 : 2;
  RD_REQUIRE(row_stride >= vocab && ((uintptr_t)logits % 16) == 0 && (row_stride * es) % 16 == 0, RD_EINVAL,
             "rd_verify_row_stats: rows must be 16-byte aligned (row_stride %lld)", (long long)row_stride);
  hipStream_t s = rd::as_stream(stream);
  switch (dtype) {
    case RD_F32: return launch_stats<float>(logits, row_stride, rows, vocab, top_k, mask_value, temperature, stats, force_fallback, s);
    case RD_BF16: return launch_stats<__hip_bfloat16>(logits, row_stride, rows, vocab, top_k, mask_value, temperature, stats, force_fallback, s);
    default: return launch_stats<__half>(logits, row_stride, rows, vocab, top_k, mask_value, temperature, stats, force_fallback, s);
  }
}

extern "C" int rd_accept_sample(const int64_t* beams, const float* log_p_dense,
                                const int64_t* log_p_strides, const void* logits, int dtype,
                                const int64_t* logits_strides, const float* stats, int n_rows,
                                const int64_t* unpacker, float temperature, const float* log_q,
                                const int64_t* log_q_strides, const float* uniforms, int batch,
                                int width, int length, int vocab, int64_t* n_tokens_in_seq,
                                int64_t* seq_in_beam, void* stream) {
  RD_REQUIRE(batch > 0 && width > 0 && length > 1 && vocab > 0, RD_EINVAL,
             "rd_accept_sample: bad sizes (batch %d width %d length %d vocab %d)", batch, width, length, vocab);
  RD_REQUIRE(width <= 65535 && length <= 32767, RD_ELIMIT, "rd_accept_sample: width %d length %d", width, length);
  RD_REQUIRE(beams && log_q && log_q_strides && uniforms && n_tokens_in_seq && seq_in_beam, RD_EINVAL,
             "rd_accept_sample: null pointer");
  LogPSource src;
  if (int e = fill_source(src, log_p_dense, log_p_strides, logits, dtype, logits_strides, stats, n_rows,
                          unpacker, temperature, "rd_accept_sample")) return e;
  hipStream_t s = rd::as_stream(stream);
  { rd::ScopedTiming rd_t("accept_sample_kernel", s);
    hipLaunchKernelGGL(accept_sample_kernel, dim3(batch), dim3(kThreads), 0, s, beams, src, log_q,
                       log_q_strides[0], log_q_strides[1], log_q_strides[2], uniforms, width, length, vocab,
                       n_tokens_in_seq, seq_in_beam); }
  return rd::check_launch("rd_accept_sample");
}

extern "C" int rd_residual_probs(const float* log_p_dense, const int64_t* log_p_strides,
                                 const void* logits, int dtype, const int64_t* logits_strides,
                                 const float* stats, int n_rows, const int64_t* unpacker,
                                 float temperature, const float* log_q, const int64_t* log_q_strides,
                                 const int64_t* seq_in_beam, const int64_t* n_tokens_in_seq, int batch,
                                 int width, int length, int vocab, float* probs, void* stream) {
  RD_REQUIRE(batch > 0 && width > 0 && length > 1 && vocab > 0 && batch <= 65535, RD_EINVAL,
             "rd_residual_probs: bad sizes (batch %d width %d length %d vocab %d)", batch, width, length, vocab);
  RD_REQUIRE(log_q && log_q_strides && seq_in_beam && n_tokens_in_seq && probs, RD_EINVAL,
             "rd_residual_probs: null pointer");
  LogPSource src;
  if (int e = fill_source(src, log_p_dense, log_p_strides, logits, dtype, logits_strides, stats, n_rows,
                          unpacker, temperature, "rd_residual_probs")) return e;
  hipStream_t s = rd::as_stream(stream);
  const int blocks = (vocab + kThreads * 4 - 1) / (kThreads * 4);
  { rd::ScopedTiming rd_t("residual_probs_kernel", s);
    hipLaunchKernelGGL(residual_probs_kernel, dim3(blocks, batch), dim3(kThreads), 0, s, src, log_q,
                       log_q_strides[0], log_q_strides[1], log_q_strides[2], seq_in_beam, n_tokens_in_seq,
                       width, length, vocab, probs); }
  return rd::check_launch("rd_residual_probs");
}
