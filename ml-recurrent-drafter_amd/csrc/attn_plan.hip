// Mask compression and work planning for the verification attention (gfx950).
//   mask_bits_kernel   bool mask (batch, n_q, kv) -> one uint64 per (row, 64 keys); a wave reads 64
//                      mask bytes coalesced and a ballot turns them into the word
//   attn_plan_kernel   per batch row: the span of keys that any query attends to (whole 64-key tiles
//                      of left padding or behind the row's last tree slot are never loaded), split
//                      of that span into near-equal chunks, and the chunk list sorted longest-first
#include "attn_plan.h"
#include "rd_common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;

__global__ __launch_bounds__(kThreads) void mask_bits_kernel(
    const uint8_t* __restrict__ mask, int64_t stride_b, int64_t stride_q, int n_q, int kv_len,
    int words, int fix_empty_rows, uint64_t* __restrict__ bits, int32_t* __restrict__ row_first,
    int32_t* __restrict__ row_last) {
  const int q = blockIdx.x, b = blockIdx.y;
  const uint8_t* row = mask + (int64_t)b * stride_b + (int64_t)q * stride_q;
  uint64_t* out = bits + ((int64_t)b * n_q + q) * words;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int first = kv_len, last = -1;
  for (int w = wave; w < words; w += kWaves) {
    const int j = w * 64 + lane;
    const bool on = j < kv_len && row[j] != 0;
    const uint64_t word = __ballot(on);
    if (lane == 0) out[w] = word;
    if (word != 0) {
      const int f = w * 64 + __builtin_ctzll(word), l = w * 64 + 63 - __builtin_clzll(word);
      first = f < first ? f : first;
      last = l > last ? l : last;
    }
  }
  __shared__ int s_first[kWaves], s_last[kWaves];
  if (lane == 0) { s_first[wave] = first; s_last[wave] = last; }
  __syncthreads();
  first = kv_len; last = -1;
  for (int w = 0; w < kWaves; ++w) {
    first = s_first[w] < first ? s_first[w] : first;
    last = s_last[w] > last ? s_last[w] : last;
  }
  if (first == kv_len && fix_empty_rows) {
    // a query that attends to nothing attends to everything (finite-minimum bias semantics)
    for (int w = threadIdx.x; w < words; w += kThreads) {
      const int rem = kv_len - w * 64;
      out[w] = rem >= 64 ? ~0ull : ((1ull << rem) - 1ull);
    }
    first = 0;
    last = kv_len - 1;
  }
  if (threadIdx.x == 0) {
    row_first[(int64_t)b * n_q + q] = first;
    row_last[(int64_t)b * n_q + q] = last;
  }
}

// The plan from the span of attended keys of every batch row (s_key_min[b], s_key_end[b], in LDS,
// written before the call; the call begins with a barrier).  Whole workgroup of kThreads.
// s_rows: 2 * B more ints of LDS (the rows' split counts and first items; global memory is only
// written here, never read back: a serial loop over rows would pay a trip to memory per row).
__device__ __forceinline__ void build_plan(const int* s_key_min, const int* s_key_end, int* s_rows, int B, int n_q, int kv_len,
                           int words, int min_chunk, int max_splits, int n_heads, int n_cu,
                           const int32_t* __restrict__ kv_shift, int32_t* __restrict__ plan) {
  __shared__ int s_n_items;
  __shared__ int s_chunk;
  __shared__ int s_len[rd::kAttnSortLimit];
  int32_t* per_row = plan + RD_PLAN_HDR;
  int* s_splits = s_rows;
  int* s_first_item = s_rows + B;
  auto begin_of = [&](int b) __attribute__((always_inline)) { return rd::plan_begin(s_key_min[b]); };
  int32_t* items = plan + RD_PLAN_HDR + 4 * B;
  __syncthreads();
  for (int b = threadIdx.x; b < B; b += kThreads) {
    per_row[4 * b + 0] = begin_of(b);
    per_row[4 * b + 3] = kv_shift ? kv_shift[b] : 0;  // cache row of key c is c - shift
  }
  __syncthreads();
  __shared__ int s_share;
  __shared__ bool s_search;
  if (threadIdx.x == 0) {
    // keys per work item, first guess: one compute unit's even share (attn_plan.h)
    long long total = 0;
    for (int b = 0; b < B; ++b) total += s_key_end[b] - begin_of(b);
    s_share = rd::plan_share(total, n_heads, n_cu, min_chunk);
    // The search below is for ragged rows: with no row split at the share and one workgroup per
    // compute unit at most (every decode step of equal rows) the share stands.  It walks over
    // every piece of every candidate: only where that is a short walk.
    const long long smallest = s_share;
    const int q_tiles = n_q <= 256 ? 1 : (n_q + 255) / 256;
    bool split_at_share = false;
    for (int b = 0; b < B && !split_at_share; ++b)
      split_at_share = rd::plan_splits(s_key_end[b] - begin_of(b), s_share, max_splits) > 1;
    const bool one_round = (long long)B * n_heads * q_tiles <= n_cu;
    s_search = B <= 32 && (total / smallest + B) * 32 <= 8192 && !(one_round && !split_at_share);
  }
  __syncthreads();
  auto splits_of = [&](int live, int chunk) __attribute__((always_inline)) { return rd::plan_splits(live, chunk, max_splits); };
  // Ragged rows: the even share is only a guess, because the items run in rounds (every compute
  // unit holds one workgroup) and each costs a fixed part on top of its tiles.  A few chunk sizes
  // from the share upwards are therefore tried on a model of the launch, one thread each: the pieces of
  // every row, longest first, go to the least loaded of the n_cu / (heads * query tiles) groups
  // of compute units that an item's workgroups fill together; a piece costs its 64-key tiles plus
  // kFixed (launch of the item, first tiles, store), a piece of a split row kSplit more (partials,
  // fence and count: the fences slow the whole XCD, so the price is high), and a split row's
  // merge kMerge at the end, all in half tiles, fitted to measured launches.  The share stands
  // unless another size is at least 5 % better.  (Same box, eight rows of 500-2548 keys, 32
  // heads: 86 -> 67 us at 168 query rows, 63 -> 48 us at 88.)
  constexpr int kCands = rd::kPlanCandidates, kMaxRows = 32, kMaxGroups = 32;
  constexpr int kTile = 2, kFixed = 10, kSplit = 16, kMerge = 8;
  __shared__ int s_est[kCands];
  __shared__ int s_plen[kCands][2 * kMaxRows], s_pcnt[kCands][2 * kMaxRows], s_load[kCands][kMaxGroups];
  __shared__ int s_sorted_len[kCands][2 * kMaxRows], s_sorted_cnt[kCands][2 * kMaxRows];
  auto candidate = [&](int c) __attribute__((always_inline)) {
    return rd::plan_candidate(s_share, c);
  };
  // Three short phases instead of one thread per candidate walking through everything: (1) a
  // thread per (candidate, row) forms the row's two classes of pieces (whole pieces, and the
  // rest) at fixed slots, (2) a thread per (candidate, class) finds the class's rank by length,
  // (3) a thread per candidate deals the pieces out, longest first.
  __shared__ int s_any_split[kCands];
  if (s_search) {
    for (int i = threadIdx.x; i < kCands; i += kThreads) s_any_split[i] = 0;
    for (int idx = threadIdx.x; idx < kCands * B; idx += kThreads) {
      const int c = idx / B, b = idx - c * B, chunk = candidate(c);
      const int live = s_key_end[b] - begin_of(b);
      const int splits = splits_of(live, chunk);
      const int per = rd::plan_per(live, splits);
      const int whole = per > 0 ? live / per : 0;  // pieces of full length
      const int rest = live - whole * per;
      const int extra = splits > 1 ? kSplit : 0;
      s_plen[c][2 * b] = whole > 0 ? ((per + 63) / 64) * kTile + kFixed + extra : 0;
      s_pcnt[c][2 * b] = whole;
      s_plen[c][2 * b + 1] = rest > 0 ? ((rest + 63) / 64) * kTile + kFixed + extra : 0;
      s_pcnt[c][2 * b + 1] = rest > 0 ? 1 : 0;
      if (splits > 1) s_any_split[c] = 1;  // (every writer writes the same value)
    }
  }
  __syncthreads();
  if (s_search) {
    const int n_classes = 2 * B;
    for (int idx = threadIdx.x; idx < kCands * n_classes; idx += kThreads) {
      const int c = idx / n_classes, i = idx - c * n_classes;
      const int* plen = s_plen[c];
      const int l = plen[i];
      int rank = 0;
      for (int j = 0; j < n_classes; ++j) rank += plen[j] > l || (plen[j] == l && j < i);
      s_sorted_len[c][rank] = l;
      s_sorted_cnt[c][rank] = s_pcnt[c][i];
    }
  }
  __syncthreads();
  if (s_search && threadIdx.x < kCands) {
    const int c = threadIdx.x;
    const int q_tiles = n_q <= 256 ? 1 : (n_q + 255) / 256;
    const long long per_item = (long long)n_heads * q_tiles;  // workgroups of one item
    int groups = per_item >= n_cu ? 1 : (int)(n_cu / per_item);
    groups = groups > kMaxGroups ? kMaxGroups : groups;
    const int rounds_per_item = per_item >= n_cu ? (int)((per_item + n_cu - 1) / n_cu) : 1;
    const int* slen = s_sorted_len[c];
    const int* scnt = s_sorted_cnt[c];
    int* load = s_load[c];
    for (int g = 0; g < groups; ++g) load[g] = 0;
    int end = 0;
    for (int i = 0; i < 2 * B && slen[i] > 0; ++i)
      for (int k = 0; k < scnt[i]; ++k) {
        int least = 0, least_load = load[0];
        for (int g = 1; g < groups; ++g) {
          const int l = load[g];
          if (l < least_load) { least = g; least_load = l; }
        }
        least_load += slen[i] * rounds_per_item;
        load[least] = least_load;
        end = least_load > end ? least_load : end;
      }
    s_est[c] = end + (s_any_split[c] ? kMerge : 0);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int chunk = s_share;
    if (s_search) {
      const int at_share = s_est[0];  // candidate 0 is the share itself
      int best = at_share - at_share / 20;  // 5 % better or stay
      for (int c = 0; c < kCands; ++c)
        if (s_est[c] < best) { best = s_est[c]; chunk = candidate(c); }
    }
    s_chunk = chunk;
  }
  __syncthreads();
  const int chunk = s_chunk;
  for (int b = threadIdx.x; b < B; b += kThreads) per_row[4 * b + 1] = s_splits[b] = splits_of(s_key_end[b] - begin_of(b), chunk);
  __syncthreads();
  if (threadIdx.x == 0) {
    int n = 0;
    for (int b = 0; b < B; ++b) {
      per_row[4 * b + 2] = s_first_item[b] = n;  // first item of this row (before sorting)
      n += s_splits[b];
    }
    s_n_items = n;
    plan[0] = n; plan[1] = n_q; plan[2] = kv_len; plan[3] = words;
    plan[4] = max_splits; plan[5] = chunk; plan[6] = 0; plan[7] = 0;
  }
  __syncthreads();
  const int n_items = s_n_items;
  // every item computes its own extent and its rank (longest first, ties by index)
  auto extent = [&](int it, int& b, int& s, int& lo, int& hi) __attribute__((always_inline)) {
    b = 0;
    while (b + 1 < B && s_first_item[b + 1] <= it) ++b;
    s = it - s_first_item[b];
    rd::plan_extent(begin_of(b), s_key_end[b], s_splits[b], s, &lo, &hi);
  };
  const bool sorted = n_items <= rd::kAttnSortLimit;
  if (sorted) {
    for (int it = threadIdx.x; it < n_items; it += kThreads) {
      int b, s, lo, hi;
      extent(it, b, s, lo, hi);
      s_len[it] = hi - lo;
    }
  }
  __syncthreads();
  for (int it = threadIdx.x; it < n_items; it += kThreads) {
    int b, s, lo, hi;
    extent(it, b, s, lo, hi);
    int rank = it;
    if (sorted) {
      const int len = hi - lo;
      rank = 0;
      for (int o = 0; o < n_items; ++o) {
        const int olen = s_len[o];
        rank += (olen > len) || (olen == len && o < it);
      }
    }
    int32_t* rec = items + RD_ITEM_INTS * rank;
    rec[0] = b; rec[1] = lo; rec[2] = hi; rec[3] = s;
    rec[4] = kv_shift ? kv_shift[b] : 0;
    rec[5] = s_key_min[b];
    rec[6] = s_splits[b];
    rec[7] = s_key_end[b];
  }
}

__global__ __launch_bounds__(kThreads) void attn_plan_kernel(const int32_t* __restrict__ row_first,
                                                             const int32_t* __restrict__ row_last,
                                                             int B, int n_q, int kv_len, int words,
                                                             int min_chunk, int max_splits,
                                                             int n_heads, int n_cu,
                                                             const int32_t* __restrict__ kv_shift,
                                                             int32_t* __restrict__ plan) {
  extern __shared__ int s_span[];  // [4][B]: first key any query of the row attends to, last such key + 1, build_plan's rows
  int* s_key_min = s_span;
  int* s_key_end = s_span + B;
  // per batch row, the span of attended keys: the minimum / maximum over its query rows
  // (one wave per batch row at a time)
  for (int b = threadIdx.x >> 6; b < B; b += kThreads / 64) {
    int first = kv_len, last = -1;
    for (int q = threadIdx.x & 63; q < n_q; q += 64) {
      const int f = row_first[(int64_t)b * n_q + q], l = row_last[(int64_t)b * n_q + q];
      first = f < first ? f : first;
      last = l > last ? l : last;
    }
    for (int off = 32; off > 0; off >>= 1) {
      const int o = __shfl_xor(first, off), p = __shfl_xor(last, off);
      first = o < first ? o : first;
      last = p > last ? p : last;
    }
    if ((threadIdx.x & 63) == 0) {
      if (last < first) { first = kv_len - 1; last = kv_len - 1; }  // a row in which nobody attends to anything
      s_key_min[b] = first;
      s_key_end[b] = last + 1;
    }
  }
  build_plan(s_key_min, s_key_end, s_span + 2 * B, B, n_q, kv_len, words, min_chunk, max_splits, n_heads, n_cu, kv_shift, plan);
}

// ---------------------------------------------------------------------------------------------
// The packed tree straight to mask bits, position ids and plan: what tree_mask_kernel (bytes),
// mask_bits_kernel, position_ids_kernel and attn_plan_kernel produce one after the other, in one
// launch and without the (batch, n, prev + n) byte mask.
//   workgroups (x, b < B): kTreeSlots packed slots of batch row b, a wave per slot at a time: the
//     words of the left part are the same for every slot of a row (ballots of "is not padding",
//     computed once per workgroup into LDS); the tree part of slot q sets the bits of the packed
//     slots of its source beam's positions 0..k.  position_ids[b, q] = prev - leading pads + k.
//   workgroup (0, B): the plan.  The span of attended keys of a row follows from its left padding
//     and its tree size: first attended key = first key that is not padding (prev when there is
//     none: slot 0 attends to itself), last = its last tree slot (which attends to itself).
// ---------------------------------------------------------------------------------------------
constexpr int kTreeSlots = 16;
constexpr int kMaxLeftWords = 2048;  // left part of at most 131072 keys

template <typename PM>
__device__ inline int left_words(const PM* __restrict__ pm, int64_t prev, PM pad, uint64_t* s_left, int* s_first) {
  // words of "key j < prev is not padding" into s_left; returns nothing, *s_first = first such key (prev if none)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nw = (int)((prev + 63) >> 6);
  int first = (int)prev;
  for (int w = wave; w < nw; w += kWaves) {
    const int64_t j = (int64_t)w * 64 + lane;
    const bool on = j < prev && pm[j] != pad;
    const uint64_t word = __ballot(on);
    if (lane == 0) s_left[w] = word;
    if (word != 0) {
      const int f = w * 64 + __builtin_ctzll(word);
      first = f < first ? f : first;
    }
  }
  if (lane == 0) atomicMin(s_first, first);
  return nw;
}

template <typename PM>
__global__ __launch_bounds__(kThreads) void tree_prepare_kernel(
    const int64_t* __restrict__ unpacker, const int64_t* __restrict__ packed_token_indices,
    const int32_t* __restrict__ counts, const PM* __restrict__ padding_mask, int64_t pm_row_stride,
    int64_t pm_pad_value, int64_t prev, int B, int WL, int L, int n, int words, int n_heads, int n_cu,
    int min_chunk, int max_splits, const int32_t* __restrict__ kv_shift, uint64_t* __restrict__ bits,
    int32_t* __restrict__ plan,
    int64_t* __restrict__ position_ids, int32_t* __restrict__ left_pads) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kv_len = (int)prev + n;
  if (blockIdx.y == B) {
    // ---- the plan ------------------------------------------------------------------------------
    if (blockIdx.x != 0) return;
    extern __shared__ int s_span[];  // [4][B]
    int* s_key_min = s_span;
    int* s_key_end = s_span + B;
    for (int b = wave; b < B; b += kWaves) {
      const PM* pm = padding_mask + (int64_t)b * pm_row_stride;
      int first = (int)prev;
      for (int64_t base = 0; base < prev && first == (int)prev; base += 64) {
        const int64_t j = base + lane;
        const uint64_t word = __ballot(j < prev && pm[j] != (PM)pm_pad_value);
        if (word != 0) first = (int)base + __builtin_ctzll(word);
      }
      if (lane == 0) {
        s_key_min[b] = first;  // (== prev when no key of the left part is attended: slot 0 attends to itself)
        s_key_end[b] = (int)prev + counts[b];
        if (left_pads) left_pads[b] = first;
      }
    }
    build_plan(s_key_min, s_key_end, s_span + 2 * B, B, n, kv_len, words, min_chunk, max_splits, n_heads, n_cu, kv_shift, plan);
    return;
  }
  // ---- mask bits and position ids of kTreeSlots slots of one batch row -------------------------
  __shared__ uint64_t s_left[kMaxLeftWords];
  __shared__ int s_first;
  const int b = blockIdx.y;
  if (threadIdx.x == 0) s_first = (int)prev;
  __syncthreads();
  const int nw_left = left_words<PM>(padding_mask + (int64_t)b * pm_row_stride, prev, (PM)pm_pad_value, s_left, &s_first);
  __syncthreads();
  const int64_t start = prev - s_first;  // tokens of the row so far: its length minus its left padding
  const int q_end = (blockIdx.x + 1) * kTreeSlots < n ? (blockIdx.x + 1) * kTreeSlots : n;
  for (int q = blockIdx.x * kTreeSlots + wave; q < q_end; q += kWaves) {
    const int f = (int)packed_token_indices[(int64_t)b * n + q];
    const int i = f / L, k = f - i * L;
    // lane kk <= k holds the packed slot of position kk of the source beam
    const int tgt = lane <= k ? (int)unpacker[(int64_t)b * WL + i * L + lane] : -1;
    uint64_t* out = bits + ((int64_t)b * n + q) * words;
    // left part from LDS; tree part: bit prev + tgt[kk] for kk <= k (every lane looks at every
    // target and keeps the bits that fall into its word)
    const int w_tree = (int)(prev >> 6);  // first word that can hold a tree bit
    for (int w0 = 0; w0 < words; w0 += 64) {
      const int w = w0 + lane;
      uint64_t word = w < nw_left ? s_left[w] : 0ull;
      if (w0 + 63 >= w_tree) {
        for (int kk = 0; kk <= k; ++kk) {
          const int c = (int)prev + __shfl(tgt, kk);
          if ((c >> 6) == w) word |= 1ull << (c & 63);
        }
      }
      if (w < words) out[w] = word;
    }
    if (lane == 0 && position_ids) position_ids[(int64_t)b * n + q] = start + k;
  }
}

}  // namespace

extern "C" size_t rd_attn_plan_ints(int batch, int n_q, int kv_len) {
  if (batch <= 0 || n_q <= 0 || kv_len <= 0) return 0;
  return rd::attn_plan_ints(batch, n_q, kv_len);
}

extern "C" size_t rd_attn_bits_words(int batch, int n_q, int kv_len) {
  if (batch <= 0 || n_q <= 0 || kv_len <= 0) return 0;
  return (size_t)batch * n_q * ((kv_len + 63) / 64);
}

namespace {
int compute_units() {
  static int n = 0;
  if (n == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
      n = prop.multiProcessorCount;
    if (n <= 0) n = 256;
  }
  return n;
}
}  // namespace

extern "C" int rd_attn_prepare(const uint8_t* mask, int64_t mask_stride_b, int64_t mask_stride_q,
                               int batch, int n_q, int kv_len, int n_heads, int fix_empty_rows,
                               uint64_t* bits, int32_t* plan, const int32_t* kv_row_shift,
                               void* stream) {
  RD_REQUIRE(batch > 0 && n_q > 0 && kv_len > 0 && n_heads > 0, RD_EINVAL,
             "rd_attn_prepare: bad sizes (batch %d n_q %d kv_len %d n_heads %d)", batch, n_q, kv_len,
             n_heads);
  RD_REQUIRE(batch <= 2048 && batch * (int64_t)rd::attn_max_splits(kv_len) <= 32768, RD_ELIMIT,
             "rd_attn_prepare: batch %d too large (2048 rows; %d for kv_len %d)", batch,
             32768 / rd::attn_max_splits(kv_len), kv_len);
  RD_REQUIRE(mask && bits && plan, RD_EINVAL, "rd_attn_prepare: null pointer");
  RD_REQUIRE(mask_stride_q >= kv_len && mask_stride_b >= 0, RD_EINVAL,
             "rd_attn_prepare: mask_stride_q %lld < kv_len %d", (long long)mask_stride_q, kv_len);
  const int words = (kv_len + 63) / 64;
  const int max_splits = rd::attn_max_splits(kv_len);
  int32_t* row_first = plan + RD_PLAN_HDR + 4 * (size_t)batch + RD_ITEM_INTS * (size_t)batch * max_splits;
  int32_t* row_last = row_first + (size_t)batch * n_q;
  hipStream_t s = rd::as_stream(stream);
  { rd::ScopedTiming rd_t("mask_bits_kernel", s); hipLaunchKernelGGL(mask_bits_kernel, dim3(n_q, batch), dim3(kThreads), 0, s, mask, mask_stride_b,
                     mask_stride_q, n_q, kv_len, words, fix_empty_rows, bits, row_first, row_last); }
  if (int e = rd::check_launch("rd_attn_prepare(bits)")) return e;
  { rd::ScopedTiming rd_t("attn_plan_kernel", s); hipLaunchKernelGGL(attn_plan_kernel, dim3(1), dim3(kThreads), 4 * batch * sizeof(int), s, row_first, row_last, batch, n_q, kv_len,
                     words, rd::kAttnChunk, max_splits, n_heads, compute_units(), kv_row_shift, plan); }
  return rd::check_launch("rd_attn_prepare(plan)");
}

extern "C" int rd_tree_attn_prepare(const int64_t* unpacker, const int64_t* packed_token_indices,
                                    const int32_t* counts, const void* padding_mask, int pm_elem_bytes,
                                    int64_t pm_row_stride, int64_t pm_pad_value, int64_t prev, int batch,
                                    int width, int length, int n, int n_heads, uint64_t* bits,
                                    int32_t* plan, int64_t* position_ids, int32_t* left_pads,
                                    const int32_t* kv_row_shift, void* stream) {
  RD_REQUIRE(batch > 0 && width > 0 && length > 0 && prev >= 0 && n > 0 && n_heads > 0, RD_EINVAL,
             "rd_tree_attn_prepare: bad sizes (batch %d width %d length %d prev %lld n %d n_heads %d)", batch,
             width, length, (long long)prev, n, n_heads);
  RD_REQUIRE(length <= 64 && n <= width * length, RD_ELIMIT, "rd_tree_attn_prepare: length %d (<= 64), n %d (<= width*length)",
             length, n);
  RD_REQUIRE(prev <= (int64_t)kMaxLeftWords * 64 && prev + n < 2147483647LL, RD_ELIMIT,
             "rd_tree_attn_prepare: prev %lld > %d (use rd_tree_mask + rd_attn_prepare)", (long long)prev, kMaxLeftWords * 64);
  const int kv_len = (int)prev + n;
  RD_REQUIRE(batch <= 1024 && batch * (int64_t)rd::attn_max_splits(kv_len) <= 32768, RD_ELIMIT,
             "rd_tree_attn_prepare: batch %d too large (1024 rows; %d for kv_len %d)", batch,
             32768 / rd::attn_max_splits(kv_len), kv_len);
  RD_REQUIRE(unpacker && packed_token_indices && counts && bits && plan, RD_EINVAL, "rd_tree_attn_prepare: null pointer");
  RD_REQUIRE(prev == 0 || (padding_mask && pm_row_stride >= prev), RD_EINVAL,
             "rd_tree_attn_prepare: padding_mask missing or pm_row_stride %lld < prev %lld", (long long)pm_row_stride, (long long)prev);
  RD_REQUIRE(pm_elem_bytes == 1 || pm_elem_bytes == 4 || pm_elem_bytes == 8, RD_EINVAL,
             "rd_tree_attn_prepare: pm_elem_bytes must be 1, 4 or 8 (got %d)", pm_elem_bytes);
  const int words = (kv_len + 63) / 64;
  const int max_splits = rd::attn_max_splits(kv_len);
  hipStream_t s = rd::as_stream(stream);
  const dim3 grid((n + kTreeSlots - 1) / kTreeSlots, batch + 1);
#define RD_LAUNCH_TP(T)                                                                               \
  do { rd::ScopedTiming rd_t("tree_prepare_kernel", s);                                               \
    hipLaunchKernelGGL(tree_prepare_kernel<T>, grid, dim3(kThreads), 4 * batch * sizeof(int), s, unpacker, \
                       packed_token_indices, counts, reinterpret_cast<const T*>(padding_mask), pm_row_stride,  \
                       pm_pad_value, prev, batch, width * length, length, n, words, n_heads, compute_units(),  \
                       rd::kAttnChunk, max_splits, kv_row_shift, bits, plan, position_ids, \
                       left_pads); } while (0)
  if (pm_elem_bytes == 1) RD_LAUNCH_TP(uint8_t);
  else if (pm_elem_bytes == 4) RD_LAUNCH_TP(int32_t);
  else RD_LAUNCH_TP(int64_t);
#undef RD_LAUNCH_TP
  return rd::check_launch("rd_tree_attn_prepare");
}
