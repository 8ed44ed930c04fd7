// Drafter beam search, post-GEMM chain of one iteration (gfx950): one read of the logits.
//
//   per beam row : x -= max(x); entries below the 50th largest become -50000; log-softmax;
//                  score = log-prob + running beam score
//   per batch row: top-W of the W*V scores, sorted descending; token = idx % V, parent = idx / V;
//                  beams gathered by parent and extended by the token
//
// beam_row_kernel (one workgroup per beam row, the whole row in registers: 256 threads x 128 values
// up to a vocabulary of 32768, so that several rows share a compute unit; 1024 x 64 above):
//   After the filter only ~50 entries of a row differ from one constant, so the row's contribution
//   to the batch row's top-W is: its W best survivors, then (if W exceeds them) filtered tokens in
//   increasing id order, all with the same score.  Survivors are found without sorting the row:
//   a pivot p -- the minimum over waves of each wave's r-th largest per-thread maximum,
//   r = ceil(50/waves) -- has at least 50 entries above it and, on ordinary data, not many more;
//   entries >= p go to an LDS list, which is sorted by counting.  The max subtraction and the
//   rounding are applied to the listed entries only.  If the list overflows or cannot decide a tie
//   at the 50th value (heavy ties, adversarial layouts) the row falls back to a radix selection
//   over the row in memory: several passes, exact for any input.
// beam_merge_kernel (one workgroup per batch row): the W sorted lists are cut at the W-th largest
//   of their leading entries, the few entries above the cut are ranked by counting.
//
// Rounding follows the drafter's dtype T at the points where a tensor in that dtype is
// materialised upstream (after the max subtraction, the filter value, the log-softmax output); the
// beam score is float32.  Equal scores are ordered by the lower flat index beam*V + token.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include <mutex>

#include "row_select.h"

namespace {

constexpr int kMaxWidth = 64;    // beam width limit of the merge kernel (W*W <= 4096 LDS keys)
constexpr int kMergeThreads = 256;

// The exact path for rows whose candidate list overflows or cannot settle a tie.  Works from memory
// (the row is in L2), not from the caller's register copy, so that it costs the common path no
// registers.  With t = round_T(x - max) and thr = the k-th largest t, the first W entries in
// (score descending, index ascending) order are among: every entry with t > thr (fewer than k),
// the first W entries by index with t == thr, and the first W by index with t < thr (the filtered
// class, one common score).  Those are listed, scored and ranked by counting.
template <typename T, int THREADS>
__device__ void beam_row_fallback(const T* __restrict__ x_row, int V, float row_max, int k_eff,
                                  float mask_t, float lpb, int W, float* __restrict__ c_score,
                                  int32_t* __restrict__ c_tok, float* __restrict__ lo_row,
                                  RowShared& sh) {
  const int tid = threadIdx.x;
  auto value = [&](int i) { return Num<T>::round(Num<T>::load(x_row + i) - row_max); };
  const float thr = row_kth_radix<T, THREADS>(x_row, V, row_max, k_eff, sh);
  // every thread owns a contiguous index range, so that "first by index" is a prefix over threads
  const int span = (V + THREADS - 1) / THREADS;
  const int i_lo = tid * span < V ? tid * span : V, i_hi = i_lo + span < V ? i_lo + span : V;
  int* n_eq = reinterpret_cast<int*>(sh.ckey);  // [THREADS] entries equal to thr per thread
  int* n_lt = n_eq + THREADS;                   // [THREADS] entries below thr per thread
  if (tid == 0) sh.n_surv = 0;                  // length of the list of entries above thr
  __syncthreads();
  float part = 0.f;
  int eq = 0, lt = 0;
  for (int i = i_lo; i < i_hi; ++i) {
    const float t = value(i);
    if (t >= thr) part += expf(t);
    if (t > thr) sh.skey[atomicAdd(&sh.n_surv, 1)] = key64(t, (uint32_t)i);  // fewer than k_eff <= 512
    eq += t == thr;
    lt += t < thr;
  }
  n_eq[tid] = eq;
  n_lt[tid] = lt;
  const float logsum = logf(block_sum<THREADS>(part, sh));  // has barriers
  const float masked_lp = Num<T>::round(mask_t - logsum);
  const int n_gt = sh.n_surv;
  int eq_before = 0, lt_before = 0, eq_all = 0, lt_all = 0;
  for (int j = 0; j < THREADS; ++j) {
    const int e = n_eq[j], l = n_lt[j];
    if (j < tid) { eq_before += e; lt_before += l; }
    eq_all += e;
    lt_all += l;
  }
  const int take_eq = eq_all < W ? eq_all : W, take_lt = lt_all < W ? lt_all : W;
  // list: [0, n_gt) above thr, [n_gt, n_gt + take_eq) equal, then take_lt filtered entries
  if ((eq_before < W && eq > 0) || (lt_before < W && lt > 0)) {
    int e = eq_before, l = lt_before;
    for (int i = i_lo; i < i_hi; ++i) {
      const float t = value(i);
      if (t == thr) { if (e < W) sh.skey[n_gt + e] = key64(t, (uint32_t)i); ++e; }
      else if (t < thr) { if (l < W) sh.skey[n_gt + take_eq + l] = key64(t, (uint32_t)i); ++l; }
    }
  }
  __syncthreads();
  // score keys (the per-thread counts in ckey are dead after the barrier above)
  const int n_list = n_gt + take_eq + take_lt;
  for (int c = tid; c < n_list; c += THREADS) {
    const unsigned long long e = sh.skey[c];
    const float lp = c < n_gt + take_eq ? Num<T>::round(key_value(e) - logsum) : masked_lp;
    sh.ckey[c] = key64(lp + lpb, (uint32_t)key_index(e));
  }
  if (tid < kKeyPad) sh.ckey[n_list + tid] = 0ull;
  __syncthreads();
  for (int c = tid; c < n_list; c += THREADS) {
    const unsigned long long mine = sh.ckey[c];
    const int rank = count_greater(sh.ckey, pad_keys(n_list), mine);
    if (rank < W) { c_score[rank] = key_value(mine); c_tok[rank] = key_index(mine); }
  }
  for (int w = n_list + tid; w < W; w += THREADS) { c_score[w] = -INFINITY; c_tok[w] = -1; }  // V < W
  if (lo_row)
    for (int i = tid; i < V; i += THREADS) {
      const float t = value(i);
      lo_row[i] = t >= thr ? Num<T>::round(t - logsum) : masked_lp;
    }
}

// ITEMS elements per thread, held as ITEMS/VEC vectors of VEC = 16 bytes / sizeof(T).
template <typename T, int ITEMS, int THREADS>
__global__ __launch_bounds__(THREADS) void beam_row_kernel(
    const T* __restrict__ logits, int64_t row_stride, int64_t batch_stride, int V,
    const float* __restrict__ log_p_beam, int W, int top_k, float mask_value,
    float* __restrict__ cand_score,
    int32_t* __restrict__ cand_tok, float* __restrict__ logp_out, int64_t logp_row_stride,
    int force_fallback) {
  constexpr int VEC = 16 / sizeof(T);
  __shared__ RowShared sh;
  const int row = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const T* x_row = logits + (int64_t)(row / W) * batch_stride + (int64_t)(row % W) * row_stride;

  // ---- load the row; maximum; pivot on the raw values -------------------------------------------
  float x[ITEMS];
  load_row<T, ITEMS, THREADS>(x_row, V, x);
  float tmax = -INFINITY;
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) tmax = fmaxf(tmax, x[j]);
  const float row_max = block_max<THREADS>(tmax, sh);
  const int k_eff = top_k < V ? top_k : V;
  const float mask_t = Num<T>::round(mask_value);
  const float lpb = log_p_beam[row];
  float* c_score = cand_score + (int64_t)row * W;
  int32_t* c_tok = cand_tok + (int64_t)row * W;
  // (a few more maxima than k_eff: the k-th largest key then sits well above the pivot's key, and
  // a tie between the two, which costs the slow path, takes that many equal values in a row)
  const float pivot = row_pivot<THREADS, Num<T>::kValueBits>(tmax, k_eff + kPivotMargin < THREADS ? k_eff + kPivotMargin : THREADS, sh);

  // ---- candidates: entries >= pivot, keyed by their value after the max subtraction ------------
  // t(x) = round_T(x - max) is monotone, so the k-th largest t comes from the list; an entry
  // below the pivot could only tie with it when that k-th value equals t(pivot).
  int n_c = -1;
  if (!force_fallback)
    n_c = row_sorted_candidates<ITEMS, VEC, THREADS>(
        x, pivot, sh, [&](float v, int i) { return key64(Num<T>::round(v - row_max), (uint32_t)i); });
  bool fast = n_c >= k_eff;
  if (fast && n_c < V) fast = key_value(sh.skey[k_eff - 1]) > Num<T>::round(pivot - row_max);

  if (fast) {
    const int n_s = row_survivors<THREADS>(n_c, k_eff, sh);  // skey[0 .. n_s) survive the filter
    const float thr = key_value(sh.skey[k_eff - 1]);
    auto s_val = [&](int o) { return key_value(sh.skey[o]); };
    auto s_idx = [&](int o) { return key_index(sh.skey[o]); };
    // log-sum-exp over the survivors in sorted order (filtered entries add exp(-5e4) == 0)
    if (wave == 0) {
      float part = 0.f;
      for (int o = lane; o < n_s; o += 64) part += expf(s_val(o));
      part = wave_sum(part);
      if (lane == 0) sh.logsum = logf(part);
    }
    __syncthreads();
    const float logsum = sh.logsum;
    const float masked_score = Num<T>::round(mask_t - logsum) + lpb;
    // survivors -> scores; equal scores are re-ordered by index (rounding can merge values)
    for (int s = tid; s < n_s; s += THREADS) {
      const float sc = Num<T>::round(s_val(s) - logsum) + lpb;
      const int si = s_idx(s);
      // entries with the same rounded score are contiguous in the sorted list
      int lo = s;
      while (lo > 0 && Num<T>::round(s_val(lo - 1) - logsum) + lpb == sc) --lo;
      int hi = s;
      while (hi + 1 < n_s && Num<T>::round(s_val(hi + 1) - logsum) + lpb == sc) ++hi;
      int pos = lo;
      for (int o = lo; o <= hi; ++o) pos += s_idx(o) < si;
      if (pos < W) { c_score[pos] = sc; c_tok[pos] = si; }
    }
    // W beyond the survivors: filtered tokens in increasing id, all with masked_score
    if (n_s < W) {
      const int need = W - n_s;
      for (int u = tid; u < need + n_s && u < V; u += THREADS) {
        bool surv = false;
        int before = 0;
        for (int o = 0; o < n_s; ++o) { surv |= s_idx(o) == u; before += s_idx(o) < u; }
        const int pos = u - before;
        if (!surv && pos < need) { c_score[n_s + pos] = masked_score; c_tok[n_s + pos] = u; }
      }
      const int avail = V - n_s;  // fewer tokens than W in a tiny vocabulary
      for (int u = tid; u < need; u += THREADS)
        if (u >= avail) { c_score[n_s + u] = -INFINITY; c_tok[n_s + u] = -1; }
    }
    if (logp_out) {
      float* lo_row = logp_out + (int64_t)row * logp_row_stride;
      const float masked_lp = Num<T>::round(mask_t - logsum);
      const int base = row_base<VEC>();
#pragma unroll
      for (int c = 0; c < ITEMS / 4; ++c) {
        // float4 stores where the four values are contiguous in the row (VEC is 4 or 8)
        const int i = row_index_at<VEC, THREADS>(base, c * 4);
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float t = Num<T>::round(x[c * 4 + e] - row_max);
          o[e] = t >= thr ? Num<T>::round(t - logsum) : masked_lp;
        }
        if (i + 4 <= V && ((reinterpret_cast<uintptr_t>(lo_row + i) & 15) == 0)) {
          *reinterpret_cast<float4*>(lo_row + i) = make_float4(o[0], o[1], o[2], o[3]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) if (i + e < V) lo_row[i + e] = o[e];
        }
      }
    }
    return;
  }

  beam_row_fallback<T, THREADS>(x_row, V, row_max, k_eff, mask_t, lpb, W, c_score, c_tok,
                                logp_out ? logp_out + (int64_t)row * logp_row_stride : nullptr, sh);
}

// One workgroup per batch row: top-W of W sorted lists of W candidates.
//   1. the W-th largest key of a subset (the first m entries of every list, m*W <= threads) is a
//      lower bound of the W-th largest key overall: the cut;
//   2. the keys >= cut -- usually not many more than W -- are listed and ranked by counting.
__global__ __launch_bounds__(kMergeThreads) void beam_merge_kernel(
    const float* __restrict__ cand_score, const int32_t* __restrict__ cand_tok, int W, int V,
    const int64_t* __restrict__ beams_in, int t_len, float* __restrict__ new_log_p_beam,
    int64_t* __restrict__ tokens, int64_t* __restrict__ parents, int64_t* __restrict__ beams_out) {
  __shared__ __attribute__((aligned(16))) unsigned long long s_keys[kMaxWidth * kMaxWidth + 2];
  __shared__ __attribute__((aligned(16))) unsigned long long s_head[kMergeThreads + 2];
  __shared__ unsigned long long s_cut;
  __shared__ int s_count;
  __shared__ int s_parent[kMaxWidth];
  const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
  const float* cs = cand_score + (int64_t)b * W * W;
  const int32_t* ct = cand_tok + (int64_t)b * W * W;
  auto key_at = [&](int w, int j) -> uint64_t {
    const int tok = ct[w * W + j];
    return tok < 0 ? 0ull : key64(cs[w * W + j], (uint32_t)(w * V + tok));
  };
  auto count_above = [&](const unsigned long long* keys, int n, uint64_t mine) {
    const ulonglong2* k2 = reinterpret_cast<const ulonglong2*>(keys);  // keys[n] is a zero pad
    int before = 0;
    for (int o = 0; 2 * o < n; ++o) {
      const ulonglong2 kk = k2[o];
      before += (kk.x > mine) + (kk.y > mine);
    }
    return before;
  };
  const int m = W < kMergeThreads / W ? W : kMergeThreads / W;
  const int n_sub = W * m;
  uint64_t mine = 0ull;
  if (tid < n_sub) mine = key_at(tid / m, tid % m);
  s_head[tid] = mine;
  if (tid == 0) { s_head[kMergeThreads] = 0ull; s_count = 0; s_cut = 0ull; }
  __syncthreads();
  // distinct nonzero keys: exactly one thread has W - 1 keys above it (none if fewer than W exist)
  if (mine != 0ull && count_above(s_head, kMergeThreads, mine) == W - 1) s_cut = mine;
  __syncthreads();
  const uint64_t cut = s_cut;
  for (int c0 = 0; c0 < W * W; c0 += kMergeThreads) {
    const int c = c0 + tid;
    const uint64_t k = c < W * W ? key_at(c / W, c % W) : 0ull;
    const bool take = k != 0ull && k >= cut;
    const uint64_t votes = __ballot(take);
    if (votes == 0) continue;
    int first = 0;
    const int leader = __builtin_ctzll(votes);
    if (lane == leader) first = atomicAdd(&s_count, __builtin_popcountll(votes));
    first = __shfl(first, leader);
    if (take) s_keys[first + __builtin_popcountll(votes & ((1ull << lane) - 1ull))] = k;
  }
  __syncthreads();
  const int n = s_count;
  if (tid == 0) s_keys[n] = 0ull;
  __syncthreads();
  for (int c = tid; c < n; c += kMergeThreads) {
    const uint64_t k = s_keys[c];
    const int rank = count_above(s_keys, n, k);
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
int launch_rows(const void* logits, int64_t row_stride, int64_t batch_stride, int rows, int V,
                const float* lpb, int W,
                int top_k, float mask_value, float* cs, int32_t* ct, float* logp_out,
                int64_t logp_row_stride, int force_fallback, hipStream_t s) {
  const T* x = reinterpret_cast<const T*>(logits);
#define RD_ROWS(ITEMS, THREADS)                                                                     \
  do { rd::ScopedTiming rd_t("beam_row_kernel", s);                                                  \
    hipLaunchKernelGGL((beam_row_kernel<T, ITEMS, THREADS>), dim3(rows), dim3(THREADS), 0, s, x,     \
                       row_stride, batch_stride, V, lpb, W, top_k, mask_value, cs, ct, logp_out,     \
                       logp_row_stride,                                                              \
                       force_fallback); } while (0)
  switch (row_geometry(V)) {
    case 0: RD_ROWS(32, 256); break;
    // few rows (batch*width below two per compute unit): twice the threads per row hide more of the
    // per-row latency (360 rows of 32000: 22.5 -> 18.7 us); with many rows the smaller workgroup wins
    case 1: if (rows <= 512) RD_ROWS(64, 512); else RD_ROWS(128, 256); break;
    default: RD_ROWS(64, 1024); break;
  }
#undef RD_ROWS
  return rd::check_launch("rd_beam_topk(rows)");
}

// Scratch of rd_beam_topk_static: the candidate lists (scores, tokens) of every beam row, in device
// memory that belongs to the library and exists from the moment it is loaded, one copy per GPU.
constexpr int kStaticMaxRows = 4096;  // batch * width
constexpr size_t kStaticScratchBytes = 2 * (size_t)kStaticMaxRows * kMaxWidth * 4;  // 2 MiB
}  // namespace

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
// The array's name is only a host-side stand-in: its address on a GPU is asked for once per device
// (with that device current) and kept; every GPU holds its own copy at its own address.
void* static_scratch(int* error) {
  static std::mutex mu;
  static void* ptr[kMaxDevices] = {nullptr};
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    *error = rd::fail(RD_ELAUNCH, "rd_beam_topk_static: no current device (or an ordinal above %d)", kMaxDevices - 1);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (ptr[dev] == nullptr) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      *error = rd::fail(RD_ELAUNCH, "rd_beam_topk_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
      return nullptr;
    }
    ptr[dev] = p;
  }
  return ptr[dev];
}
}  // namespace

namespace {

// One workgroup per (batch row, beam): the row's prompt state into the context half of the head's
// input, zeros into the recurrent state, the beam's first token and score.
constexpr int kInitThreads = 256;
__global__ __launch_bounds__(kInitThreads) void beam_init_kernel(const char* prompt_state, int64_t ps_row_bytes,
                                                                 const int64_t* init_token, int width, int64_t hidden_bytes,
                                                                 float mask_value, float* log_p_beam, int64_t* beams,
                                                                 char* head_in, int64_t head_in_row_bytes, char* state,
                                                                 int state_rows) {
  const int w = blockIdx.x, b = blockIdx.y;
  const int64_t row = (int64_t)b * width + w;
  const uint4* src = reinterpret_cast<const uint4*>(prompt_state + (int64_t)b * ps_row_bytes);
  uint4* dst = reinterpret_cast<uint4*>(head_in + row * head_in_row_bytes);
  const int64_t chunks = hidden_bytes / 16;
  for (int64_t i = threadIdx.x; i < chunks; i += kInitThreads) dst[i] = src[i];
  if (w < state_rows) {
    uint4* z = reinterpret_cast<uint4*>(state + ((int64_t)b * state_rows + w) * hidden_bytes);
    for (int64_t i = threadIdx.x; i < chunks; i += kInitThreads) z[i] = make_uint4(0u, 0u, 0u, 0u);
  }
  if (threadIdx.x == 0) {
    log_p_beam[row] = w == 0 ? 0.f : mask_value;
    beams[row] = init_token[b];
  }
}

}  // namespace

extern "C" int rd_beam_init(const void* prompt_state, int64_t ps_row_bytes, const int64_t* init_token, int batch,
                            int width, int64_t hidden_bytes, float mask_value, float* log_p_beam, int64_t* beams,
                            void* head_in, int64_t head_in_row_bytes, void* state, int state_rows, void* stream) {
  RD_REQUIRE(batch > 0 && width > 0 && hidden_bytes > 0 && state_rows > 0 && state_rows <= width, RD_EINVAL,
             "rd_beam_init: bad sizes (batch %d width %d hidden bytes %lld state rows %d)", batch, width,
             (long long)hidden_bytes, state_rows);
  RD_REQUIRE(batch <= 65535, RD_ELIMIT, "rd_beam_init: batch %d > 65535", batch);
  RD_REQUIRE(prompt_state && init_token && log_p_beam && beams && head_in && state, RD_EINVAL, "rd_beam_init: null pointer");
  auto al = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
  RD_REQUIRE(hidden_bytes % 16 == 0 && ps_row_bytes % 16 == 0 && head_in_row_bytes % 16 == 0 && al(prompt_state) &&
                 al(head_in) && al(state) && ps_row_bytes >= hidden_bytes && head_in_row_bytes >= hidden_bytes,
             RD_EINVAL, "rd_beam_init: rows must be 16-byte aligned multiples of 16 bytes, strides at least a row");
  hipStream_t s = rd::as_stream(stream);
  {
    rd::ScopedTiming rd_t("beam_init_kernel", s);
    hipLaunchKernelGGL(beam_init_kernel, dim3(width, batch), dim3(kInitThreads), 0, s,
                       reinterpret_cast<const char*>(prompt_state), ps_row_bytes, init_token, width, hidden_bytes,
                       mask_value, log_p_beam, beams, reinterpret_cast<char*>(head_in), head_in_row_bytes,
                       reinterpret_cast<char*>(state), state_rows);
  }
  return rd::check_launch("rd_beam_init");
}

extern "C" size_t rd_beam_topk_workspace_bytes(int batch, int width) {
  if (batch <= 0 || width <= 0) return 0;
  const size_t n = (size_t)batch * width * width;
  return rd::align_up(n * sizeof(float), 256) + rd::align_up(n * sizeof(int32_t), 256);
}

extern "C" int rd_beam_topk(const void* logits, int dtype, int64_t row_stride, int64_t batch_stride,
                            int batch, int width, int vocab, const float* log_p_beam, int top_k, float mask_value,
                            const int64_t* beams_in, int t_len, float* new_log_p_beam,
                            int64_t* tokens, int64_t* parents, int64_t* beams_out, float* logp_out,
                            int64_t logp_row_stride, void* workspace, size_t workspace_bytes,
                            int force_fallback, void* stream) {
  RD_REQUIRE(batch > 0 && width > 0 && vocab > 0 && top_k > 0, RD_EINVAL,
             "rd_beam_topk: bad sizes (batch %d width %d vocab %d top_k %d)", batch, width, vocab, top_k);
  RD_REQUIRE(width <= kMaxWidth, RD_ELIMIT, "rd_beam_topk: width %d > %d", width, kMaxWidth);
  RD_REQUIRE(row_geometry(vocab) >= 0, RD_ELIMIT, "rd_beam_topk: vocab %d > 65536", vocab);
  RD_REQUIRE((int64_t)width * vocab < 4294967295LL, RD_ELIMIT, "rd_beam_topk: width*vocab too large");
  RD_REQUIRE(top_k <= 512, RD_ELIMIT, "rd_beam_topk: top_k %d > 512", top_k);
  RD_REQUIRE(logits && log_p_beam && new_log_p_beam && tokens && parents && workspace, RD_EINVAL,
             "rd_beam_topk: null pointer");
  RD_REQUIRE(!beams_out || (beams_in && t_len > 0), RD_EINVAL, "rd_beam_topk: beams_out needs beams_in and t_len > 0");
  if (batch_stride == 0) batch_stride = (int64_t)width * row_stride;
  RD_REQUIRE(row_stride >= vocab || (row_stride == 0 && batch_stride >= vocab), RD_EINVAL,
             "rd_beam_topk: row_stride %lld < vocab %d (0 is allowed with a batch stride: every beam of a row reads the same logits)",
             (long long)row_stride, vocab);
  RD_REQUIRE(batch_stride >= 0, RD_EINVAL, "rd_beam_topk: negative batch_stride");
  const int es = dtype == RD_F32 ? 4 : 2;
  RD_REQUIRE(dtype == RD_F32 || dtype == RD_BF16 || dtype == RD_F16, RD_EINVAL, "rd_beam_topk: unknown dtype %d", dtype);
  RD_REQUIRE(((uintptr_t)logits % 16) == 0 && (row_stride * es) % 16 == 0 && (batch_stride * es) % 16 == 0, RD_EINVAL,
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
    case RD_F32: e = launch_rows<float>(logits, row_stride, batch_stride, rows, vocab, log_p_beam, width, top_k, mask_value, cs, ct, logp_out, logp_row_stride, force_fallback, s); break;
    case RD_BF16: e = launch_rows<__hip_bfloat16>(logits, row_stride, batch_stride, rows, vocab, log_p_beam, width, top_k, mask_value, cs, ct, logp_out, logp_row_stride, force_fallback, s); break;
    default: e = launch_rows<__half>(logits, row_stride, batch_stride, rows, vocab, log_p_beam, width, top_k, mask_value, cs, ct, logp_out, logp_row_stride, force_fallback, s); break;
  }
  if (e) return e;
  { rd::ScopedTiming rd_t("beam_merge_kernel", s); hipLaunchKernelGGL(beam_merge_kernel, dim3(batch), dim3(kMergeThreads), 0, s, cs, ct, width, vocab,
                     beams_in, t_len, new_log_p_beam, tokens, parents, beams_out); }
  return rd::check_launch("rd_beam_topk(merge)");
}

extern "C" int rd_beam_topk_static(const void* logits, int dtype, int64_t row_stride, int64_t batch_stride,
                                   int batch, int width, int vocab, const float* log_p_beam, int top_k,
                                   float mask_value, const int64_t* beams_in, int t_len,
                                   float* new_log_p_beam, int64_t* tokens, int64_t* parents,
                                   int64_t* beams_out, float* logp_out, int64_t logp_row_stride,
                                   int force_fallback, void* stream) {
  RD_REQUIRE(batch > 0 && width > 0, RD_EINVAL, "rd_beam_topk_static: bad sizes (batch %d width %d)", batch, width);
  const size_t need = rd_beam_topk_workspace_bytes(batch, width);
  RD_REQUIRE((int64_t)batch * width <= kStaticMaxRows && width <= kMaxWidth && need <= kStaticScratchBytes, RD_ELIMIT,
             "rd_beam_topk_static: batch %d x width %d is beyond the built-in scratch (batch*width <= %d, width <= %d); "
             "use rd_beam_topk with a workspace", batch, width, kStaticMaxRows, kMaxWidth);
  int error = RD_OK;
  void* ws = static_scratch(&error);
  if (ws == nullptr) return error;
  // every beam row writes all `width` entries of its two lists, so nothing of an earlier call is read
  return rd_beam_topk(logits, dtype, row_stride, batch_stride, batch, width, vocab, log_p_beam, top_k, mask_value,
                      beams_in, t_len, new_log_p_beam, tokens, parents, beams_out, logp_out, logp_row_stride, ws,
                      kStaticScratchBytes, force_fallback, stream);
}
