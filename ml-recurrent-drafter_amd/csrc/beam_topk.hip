// Drafter beam search, post-GEMM chain of one iteration (gfx950): one read of the logits.
//
//   per beam row : x -= max(x); entries below the 50th largest become -50000; log-softmax;
//                  score = log-prob + running beam score
//   per batch row: top-W of the W*V scores, sorted descending; token = idx % V, parent = idx / V;
//                  beams gathered by parent and extended by the token
//
// beam_row_kernel (one 1024-thread workgroup per beam row, the whole row in registers):
//   After the filter only ~50 entries of a row differ from one constant, so the row's contribution
//   to the batch row's top-W is: its W best survivors, then (if W exceeds them) filtered tokens in
//   increasing id order, all with the same score.  Survivors are found without sorting the row:
//   a pivot p -- the minimum over waves of each wave's r-th largest per-thread maximum,
//   r = ceil(50/16) -- has at least 50 entries above it and, on ordinary data, not many more;
//   entries >= p are appended to an LDS list, which is ranked by counting.  If the list overflows
//   (heavy ties, adversarial layouts) the row falls back to a bisection on the value bits plus W
//   rounds of block-wide argmax: slow, exact for any input.
// beam_merge_kernel (one workgroup per batch row): the W sorted lists are cut at
//   max(min head, max tail), the few entries above the cut are ranked by counting.
//
// Rounding follows the drafter's dtype T at the points where a tensor in that dtype is
// materialised upstream (after the max subtraction, the filter value, the log-softmax output); the
// beam score is float32.  Equal scores are ordered by the lower flat index beam*V + token.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "row_select.h"

namespace {

constexpr int kMaxWidth = 64;    // beam width limit of the merge kernel (W*W <= 4096 LDS keys)
constexpr int kMergeThreads = 256;

// ITEMS elements per thread, held as ITEMS/VEC vectors of VEC = 16 bytes / sizeof(T).
template <typename T, int ITEMS>
__global__ __launch_bounds__(kRowThreads) void beam_row_kernel(
    const T* __restrict__ logits, int64_t row_stride, int V, const float* __restrict__ log_p_beam,
    int W, int top_k, float mask_value, float* __restrict__ cand_score,
    int32_t* __restrict__ cand_tok, float* __restrict__ logp_out, int64_t logp_row_stride,
    int force_fallback) {
  constexpr int VEC = 16 / sizeof(T);
  constexpr int NV = ITEMS / VEC;
  __shared__ RowShared sh;
  const int row = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const T* x_row = logits + (int64_t)row * row_stride;
  auto index_of = [&](int j) { return ((j / VEC) * kRowThreads + tid) * VEC + (j % VEC); };

  // ---- load the row, row maximum ------------------------------------------------------------
  float x[ITEMS];
  float tmax = -INFINITY;
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int i0 = (c * kRowThreads + tid) * VEC;
    if (i0 + VEC <= V) {
      struct alignas(16) Pack { T v[VEC]; };
      const Pack p = *reinterpret_cast<const Pack*>(x_row + i0);
#pragma unroll
      for (int e = 0; e < VEC; ++e) x[c * VEC + e] = Num<T>::load(&p.v[e]);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) x[c * VEC + e] = (i0 + e < V) ? Num<T>::load(x_row + i0 + e) : -INFINITY;
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) tmax = fmaxf(tmax, x[c * VEC + e]);
  }
  const float row_max = block_max(tmax, sh);
  tmax = -INFINITY;
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    x[j] = index_of(j) < V ? Num<T>::round(x[j] - row_max) : -INFINITY;
    tmax = fmaxf(tmax, x[j]);
  }
  const int k_eff = top_k < V ? top_k : V;
  const float mask_t = Num<T>::round(mask_value);
  const float lpb = log_p_beam[row];
  float* c_score = cand_score + (int64_t)row * W;
  int32_t* c_tok = cand_tok + (int64_t)row * W;

  // ---- pivot: at least k_eff entries are >= pivot ----------------------------------------------
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
      if (x[j] >= pivot && index_of(j) < V) {
        const int pos = atomicAdd(&sh.count, 1);
        if (pos < kCap) { sh.cval[pos] = x[j]; sh.cidx[pos] = index_of(j); }
      }
    }
  }
  __syncthreads();
  const int n_c = force_fallback ? kCap + 1 : sh.count;

  if (n_c <= kCap) {
    // ---- ranked candidate list -------------------------------------------------------------
    // order: value descending, index ascending.  rank = number of candidates strictly before.
    int my_rank = -1;
    float my_v = 0.f;
    int my_i = 0;
    if (tid < n_c) {
      my_v = sh.cval[tid];
      my_i = sh.cidx[tid];
      int gt = 0, ge = 0, before = 0;
      for (int o = 0; o < n_c; ++o) {
        const float ov = sh.cval[o];
        const int oi = sh.cidx[o];
        gt += ov > my_v;
        ge += ov >= my_v;
        before += (ov > my_v) || (ov == my_v && oi < my_i);
      }
      my_rank = before;
      if (gt < k_eff && k_eff <= ge) { sh.thr = my_v; sh.n_surv = ge; }
    }
    // entries beyond the first 1024 candidates (tid covers only kRowThreads of up to kCap)
    int my_rank2 = -1;
    float my_v2 = 0.f;
    int my_i2 = 0;
    if (tid + kRowThreads < n_c) {
      my_v2 = sh.cval[tid + kRowThreads];
      my_i2 = sh.cidx[tid + kRowThreads];
      int gt = 0, ge = 0, before = 0;
      for (int o = 0; o < n_c; ++o) {
        const float ov = sh.cval[o];
        const int oi = sh.cidx[o];
        gt += ov > my_v2;
        ge += ov >= my_v2;
        before += (ov > my_v2) || (ov == my_v2 && oi < my_i2);
      }
      my_rank2 = before;
      if (gt < k_eff && k_eff <= ge) { sh.thr = my_v2; sh.n_surv = ge; }
    }
    __syncthreads();
    const float thr = sh.thr;
    const int n_s = sh.n_surv;
    // survivors, sorted, back into the list (all reads of the unsorted list are done)
    if (my_rank >= 0 && my_v >= thr) { sh.cval[my_rank] = my_v; sh.cidx[my_rank] = my_i; }
    if (my_rank2 >= 0 && my_v2 >= thr) { sh.cval[my_rank2] = my_v2; sh.cidx[my_rank2] = my_i2; }
    __syncthreads();
    // log-sum-exp over the survivors in sorted order (filtered entries add exp(-5e4) == 0)
    if (wave == 0) {
      float part = 0.f;
      for (int o = lane; o < n_s; o += 64) part += expf(sh.cval[o]);
      part = wave_sum(part);
      if (lane == 0) sh.logsum = logf(part);
    }
    __syncthreads();
    const float logsum = sh.logsum;
    const float masked_score = Num<T>::round(mask_t - logsum) + lpb;
    // survivors -> scores; equal scores are re-ordered by index (rounding can merge values)
    for (int s = tid; s < n_s; s += kRowThreads) {
      const float sc = Num<T>::round(sh.cval[s] - logsum) + lpb;
      const int si = sh.cidx[s];
      // entries with the same rounded score are contiguous in the sorted list
      int lo = s, pos = s;
      while (lo > 0 && Num<T>::round(sh.cval[lo - 1] - logsum) + lpb == sc) --lo;
      int hi = s;
      while (hi + 1 < n_s && Num<T>::round(sh.cval[hi + 1] - logsum) + lpb == sc) ++hi;
      pos = lo;
      for (int o = lo; o <= hi; ++o) pos += sh.cidx[o] < si;
      if (pos < W) { c_score[pos] = sc; c_tok[pos] = si; }
    }
    // W beyond the survivors: filtered tokens in increasing id, all with masked_score
    if (n_s < W) {
      const int need = W - n_s;
      for (int u = tid; u < need + n_s && u < V; u += kRowThreads) {
        bool surv = false;
        int before = 0;
        for (int o = 0; o < n_s; ++o) { surv |= sh.cidx[o] == u; before += sh.cidx[o] < u; }
        const int pos = u - before;
        if (!surv && pos < need) { c_score[n_s + pos] = masked_score; c_tok[n_s + pos] = u; }
      }
      const int avail = V - n_s;  // fewer tokens than W in a tiny vocabulary
      for (int u = tid; u < need; u += kRowThreads)
        if (u >= avail) { c_score[n_s + u] = -INFINITY; c_tok[n_s + u] = -1; }
    }
    if (logp_out) {
      float* lo_row = logp_out + (int64_t)row * logp_row_stride;
      const float masked_lp = Num<T>::round(mask_t - logsum);
#pragma unroll
      for (int j = 0; j < ITEMS; ++j) {
        const int i = index_of(j);
        if (i < V) lo_row[i] = x[j] >= thr ? Num<T>::round(x[j] - logsum) : masked_lp;
      }
    }
    return;
  }

  // ---- fallback: exact for any input -----------------------------------------------------------
  // k-th largest value by bisection on the ordered bit pattern
  uint32_t lo_k = 0u, hi_k = 0xffffffffu;  // invariant: count(>= lo_k) >= k_eff
  while (lo_k < hi_k) {
    const uint32_t mid = lo_k + (uint32_t)(((uint64_t)hi_k - lo_k + 1) >> 1);
    int cnt = 0;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) cnt += (index_of(j) < V) && ord(x[j]) >= mid;
    cnt = block_isum(cnt, sh);
    if (cnt >= k_eff) lo_k = mid; else hi_k = mid - 1;
  }
  const float thr = unord(lo_k);
  float part = 0.f;
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) part += (index_of(j) < V && x[j] >= thr) ? expf(x[j]) : 0.f;
  const float logsum = logf(block_sum(part, sh));
  const float masked_lp = Num<T>::round(mask_t - logsum);
  auto score_of = [&](int j) { return (x[j] >= thr ? Num<T>::round(x[j] - logsum) : masked_lp) + lpb; };
  uint64_t last = ~0ull;
  for (int w = 0; w < W; ++w) {
    uint64_t best = 0ull;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const int i = index_of(j);
      if (i < V) {
        const uint64_t k = key64(score_of(j), (uint32_t)i);
        if (k < last && k > best) best = k;
      }
    }
    best = block_max64(best, sh);
    if (tid == 0) {
      if (best == 0ull) { c_score[w] = -INFINITY; c_tok[w] = -1; }
      else { c_score[w] = unord((uint32_t)(best >> 32)); c_tok[w] = (int32_t)(0xffffffffu - (uint32_t)best); }
    }
    last = best == 0ull ? 0ull : best;
  }
  if (logp_out) {
    float* lo_row = logp_out + (int64_t)row * logp_row_stride;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const int i = index_of(j);
      if (i < V) lo_row[i] = x[j] >= thr ? Num<T>::round(x[j] - logsum) : masked_lp;
    }
  }
}

// One workgroup per batch row.
__global__ __launch_bounds__(kMergeThreads) void beam_merge_kernel(
    const float* __restrict__ cand_score, const int32_t* __restrict__ cand_tok, int W, int V,
    const int64_t* __restrict__ beams_in, int t_len, float* __restrict__ new_log_p_beam,
    int64_t* __restrict__ tokens, int64_t* __restrict__ parents, int64_t* __restrict__ beams_out) {
  __shared__ unsigned long long s_keys[kMaxWidth * kMaxWidth];
  __shared__ unsigned long long s_cut[2][kMergeThreads / 64];
  __shared__ int s_count;
  __shared__ int s_parent[kMaxWidth];
  const int b = blockIdx.x, tid = threadIdx.x;
  const float* cs = cand_score + (int64_t)b * W * W;
  const int32_t* ct = cand_tok + (int64_t)b * W * W;
  auto key_at = [&](int w, int j) -> uint64_t {
    const int tok = ct[w * W + j];
    return tok < 0 ? 0ull : key64(cs[w * W + j], (uint32_t)(w * V + tok));
  };
  // cut = max(min over rows of the head, max over rows of the tail): the W-th best key is >= cut
  uint64_t min_head = ~0ull, max_tail = 0ull;
  for (int w = tid; w < W; w += kMergeThreads) {
    const uint64_t h = key_at(w, 0), t = key_at(w, W - 1);
    min_head = h < min_head ? h : min_head;
    max_tail = t > max_tail ? t : max_tail;
  }
  for (int off = 32; off > 0; off >>= 1) {
    const uint64_t a = __shfl_xor(min_head, off), c = __shfl_xor(max_tail, off);
    min_head = a < min_head ? a : min_head;
    max_tail = c > max_tail ? c : max_tail;
  }
  if ((tid & 63) == 0) { s_cut[0][tid >> 6] = min_head; s_cut[1][tid >> 6] = max_tail; }
  if (tid == 0) s_count = 0;
  __syncthreads();
  for (int w = 0; w < kMergeThreads / 64; ++w) {
    min_head = s_cut[0][w] < min_head ? s_cut[0][w] : min_head;
    max_tail = s_cut[1][w] > max_tail ? s_cut[1][w] : max_tail;
  }
  const uint64_t cut = min_head > max_tail ? min_head : max_tail;
  for (int c = tid; c < W * W; c += kMergeThreads) {
    const uint64_t k = key_at(c / W, c % W);
    if (k >= cut && k != 0ull) s_keys[atomicAdd(&s_count, 1)] = k;
  }
  __syncthreads();
  const int n = s_count;
  for (int c = tid; c < n; c += kMergeThreads) {
    const uint64_t k = s_keys[c];
    int rank = 0;
    for (int o = 0; o < n; ++o) rank += s_keys[o] > k;
    if (rank < W) {
      const uint32_t flat = 0xffffffffu - (uint32_t)k;
      const int parent = (int)(flat / (uint32_t)V);
      const int64_t o = (int64_t)b * W + rank;
      new_log_p_beam[o] = unord((uint32_t)(k >> 32));
      tokens[o] = flat - (uint32_t)parent * (uint32_t)V;
      parents[o] = parent;
      s_parent[rank] = parent;
    }
  }
  if (!beams_out) return;
  __syncthreads();
  // beams_out[b,w,:t_len] = beams_in[b,parent[w],:]; beams_out[b,w,t_len] = token
  const int t_out = t_len + 1;
  for (int c = tid; c < W * t_out; c += kMergeThreads) {
    const int w = c / t_out, k = c - w * t_out;
    beams_out[((int64_t)b * W + w) * t_out + k] =
        k < t_len ? beams_in[((int64_t)b * W + s_parent[w]) * t_len + k] : tokens[(int64_t)b * W + w];
  }
}

template <typename T>
int launch_rows(const void* logits, int64_t row_stride, int rows, int V, const float* lpb, int W,
                int top_k, float mask_value, float* cs, int32_t* ct, float* logp_out,
                int64_t logp_row_stride, int force_fallback, hipStream_t s) {
  const T* x = reinterpret_cast<const T*>(logits);
  constexpr int VEC = 16 / sizeof(T);
  const int per_thread = (V + kRowThreads - 1) / kRowThreads;
#define RD_ROWS(ITEMS)                                                                              \
  do { rd::ScopedTiming rd_t("beam_row_kernel", s); hipLaunchKernelGGL((beam_row_kernel<T, ITEMS>), dim3(rows), dim3(kRowThreads), 0, s, x, row_stride, \
                     V, lpb, W, top_k, mask_value, cs, ct, logp_out, logp_row_stride, force_fallback); } while (0)
  if (per_thread <= 8 && VEC <= 8) RD_ROWS(8);
  else if (per_thread <= 32) RD_ROWS(32);
  else RD_ROWS(64);
#undef RD_ROWS
  return rd::check_launch("rd_beam_topk(rows)");
}

}  // namespace

extern "C" size_t rd_beam_topk_workspace_bytes(int batch, int width) {
  if (batch <= 0 || width <= 0) return 0;
  const size_t n = (size_t)batch * width * width;
  return rd::align_up(n * sizeof(float), 256) + rd::align_up(n * sizeof(int32_t), 256);
}

extern "C" int rd_beam_topk(const void* logits, int dtype, int64_t row_stride, int batch, int width,
                            int vocab, const float* log_p_beam, int top_k, float mask_value,
                            const int64_t* beams_in, int t_len, float* new_log_p_beam,
                            int64_t* tokens, int64_t* parents, int64_t* beams_out, float* logp_out,
                            int64_t logp_row_stride, void* workspace, size_t workspace_bytes,
                            int force_fallback, void* stream) {
  RD_REQUIRE(batch > 0 && width > 0 && vocab > 0 && top_k > 0, RD_EINVAL,
             "rd_beam_topk: bad sizes (batch %d width %d vocab %d top_k %d)", batch, width, vocab, top_k);
  RD_REQUIRE(width <= kMaxWidth, RD_ELIMIT, "rd_beam_topk: width %d > %d", width, kMaxWidth);
  RD_REQUIRE(vocab <= 64 * kRowThreads, RD_ELIMIT, "rd_beam_topk: vocab %d > %d", vocab, 64 * kRowThreads);
  RD_REQUIRE((int64_t)width * vocab < 4294967295LL, RD_ELIMIT, "rd_beam_topk: width*vocab too large");
  RD_REQUIRE(top_k <= 512, RD_ELIMIT, "rd_beam_topk: top_k %d > 512", top_k);
  RD_REQUIRE(logits && log_p_beam && new_log_p_beam && tokens && parents && workspace, RD_EINVAL,
             "rd_beam_topk: null pointer");
  RD_REQUIRE(!beams_out || (beams_in && t_len > 0), RD_EINVAL, "rd_beam_topk: beams_out needs beams_in and t_len > 0");
  RD_REQUIRE(row_stride >= vocab, RD_EINVAL, "rd_beam_topk: row_stride %lld < vocab %d", (long long)row_stride, vocab);
  const int es = dtype == RD_F32 ? 4 : 2;
  RD_REQUIRE(dtype == RD_F32 || dtype == RD_BF16 || dtype == RD_F16, RD_EINVAL, "rd_beam_topk: unknown dtype %d", dtype);
  RD_REQUIRE(((uintptr_t)logits % 16) == 0 && (row_stride * es) % 16 == 0, RD_EINVAL,
             "rd_beam_topk: logits rows must be 16-byte aligned (row_stride %lld)", (long long)row_stride);
  RD_REQUIRE(!logp_out || logp_row_stride >= vocab, RD_EINVAL, "rd_beam_topk: logp_row_stride < vocab");
  RD_REQUIRE(workspace_bytes >= rd_beam_topk_workspace_bytes(batch, width), RD_EWORKSPACE,
             "rd_beam_topk: workspace %zu < %zu bytes", workspace_bytes,
             rd_beam_topk_workspace_bytes(batch, width));
  RD_REQUIRE(((uintptr_t)workspace & 255) == 0, RD_EINVAL, "rd_beam_topk: workspace not 256B aligned");
  const size_t n = (size_t)batch * width * width;
  float* cs = reinterpret_cast<float*>(workspace);
  int32_t* ct = reinterpret_cast<int32_t*>(reinterpret_cast<char*>(workspace) + rd::align_up(n * sizeof(float), 256));
  hipStream_t s = rd::as_stream(stream);
  const int rows = batch * width;
  int e;
  switch (dtype) {
    case RD_F32: e = launch_rows<float>(logits, row_stride, rows, vocab, log_p_beam, width, top_k, mask_value, cs, ct, logp_out, logp_row_stride, force_fallback, s); break;
    case RD_BF16: e = launch_rows<__hip_bfloat16>(logits, row_stride, rows, vocab, log_p_beam, width, top_k, mask_value, cs, ct, logp_out, logp_row_stride, force_fallback, s); break;
    default: e = launch_rows<__half>(logits, row_stride, rows, vocab, log_p_beam, width, top_k, mask_value, cs, ct, logp_out, logp_row_stride, force_fallback, s); break;
  }
  if (e) return e;
  { rd::ScopedTiming rd_t("beam_merge_kernel", s); hipLaunchKernelGGL(beam_merge_kernel, dim3(batch), dim3(kMergeThreads), 0, s, cs, ct, width, vocab,
                     beams_in, t_len, new_log_p_beam, tokens, parents, beams_out); }
  return rd::check_launch("rd_beam_topk(merge)");
}
