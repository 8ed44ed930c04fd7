// Draft beams -> prefix tree -> packed tokens -> tree attention mask (gfx950).
//
// Integer, byte and index work only.  One workgroup per batch row keeps the row's beams in LDS;
// nothing is reshaped into a matrix product.  Three kernels:
//   tree_rows_kernel   per row: owner of every prefix, unpacker, the row's own packed list
//   tree_fill_kernel   per row: batch-wide offsets, max over rows, spill-over fill of the padding
//   tree_mask_kernel   per packed row: one row of the (batch, max_n, prev+max_n) byte mask
#include "rd_common.h"

namespace {

constexpr int kMaxWidth = 1024;
constexpr int kMaxLength = 64;
constexpr int kMaxTokens = 4096;  // width * length held in LDS
constexpr int kThreads = 256;

// ---------------------------------------------------------------------------------------------
// Per batch row.  Thread i owns beam i for the dedup; ownership of a beam is always a suffix of
// it, so slot(i,k) = start[owner] + k - (L - n_owned[owner]).
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void tree_rows_kernel(
    const int64_t* __restrict__ beams, int W, int L, int64_t* __restrict__ prefix_tree,
    int64_t* __restrict__ unpacker, int64_t* __restrict__ sel_tok, int32_t* __restrict__ sel_idx,
    int32_t* __restrict__ counts) {
  __shared__ int64_t s_tok[kMaxTokens];
  __shared__ int32_t s_owner[kMaxTokens];
  __shared__ int16_t s_nown[kMaxWidth];
  __shared__ int32_t s_start[kMaxWidth];

  const int b = blockIdx.x;
  const int WL = W * L;
  const int64_t* row = beams + (int64_t)b * WL;
  for (int t = threadIdx.x; t < WL; t += kThreads) s_tok[t] = row[t];
  __syncthreads();

  // owner[i][k] = smallest j whose first k+1 tokens equal beam i's.  Every pair (i, j < i) is
  // looked at by some thread: the length of the common prefix, then a minimum per position.
  for (int t = threadIdx.x; t < WL; t += kThreads) s_owner[t] = t / L;  // a beam matches itself
  __syncthreads();
  for (int pr = threadIdx.x; pr < W * W; pr += kThreads) {
    const int i = pr / W, j = pr - i * W;
    if (j >= i) continue;
    const int64_t* mine = s_tok + i * L;
    const int64_t* other = s_tok + j * L;
    int m = 0;
    while (m < L && other[m] == mine[m]) ++m;
    for (int k = 0; k < m; ++k) atomicMin(&s_owner[i * L + k], j);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < W; i += kThreads) {
    int n = 0;
    for (int k = 0; k < L; ++k) n += (s_owner[i * L + k] == i);
    s_nown[i] = (int16_t)n;
  }
  __syncthreads();

  for (int i = threadIdx.x; i < W; i += kThreads) {
    int s = 0;
    for (int j = 0; j < i; ++j) s += s_nown[j];
    s_start[i] = s;
  }
  __syncthreads();

  const int64_t base = (int64_t)b * WL;
  for (int t = threadIdx.x; t < WL; t += kThreads) {
    const int i = t / L, k = t - i * L;
    const int p = s_owner[t];
    const int slot = s_start[p] + k - (L - s_nown[p]);
    unpacker[base + t] = slot;
    if (prefix_tree) prefix_tree[base + t] = p;
    if (p == i) {
      sel_tok[base + slot] = s_tok[t];
      sel_idx[base + slot] = t;
    }
  }
  if (threadIdx.x == 0) counts[b] = s_start[W - 1] + s_nown[W - 1];
}

constexpr int kRowSlotsPad = 32;  // row_slots is zero-filled up to the next multiple of this

// ---------------------------------------------------------------------------------------------
// Per batch row: slot n of row b reads entry min(offset_b + n, total-1) of the batch-wide list.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void tree_fill_kernel(
    const int64_t* __restrict__ sel_tok, const int32_t* __restrict__ sel_idx, int B, int WL, int L,
    int32_t* __restrict__ counts, int64_t* __restrict__ packed_tokens,
    int64_t* __restrict__ packed_token_indices, int64_t* __restrict__ position_offsets,
    int32_t* __restrict__ row_start, int64_t* __restrict__ row_slots,
    int64_t* __restrict__ row_tokens) {
  __shared__ int s_red[3][kThreads / 64];
  const int b = blockIdx.x;
  int before = 0, total = 0, mx = 0;
  for (int r = threadIdx.x; r < B; r += kThreads) {
    const int c = counts[r];
    total += c;
    before += (r < b) ? c : 0;
    mx = c > mx ? c : mx;
  }
  for (int off = 32; off > 0; off >>= 1) {
    total += __shfl_xor(total, off);
    before += __shfl_xor(before, off);
    const int o = __shfl_xor(mx, off);
    mx = o > mx ? o : mx;
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
    s_red[0][wave] = total;
    s_red[1][wave] = before;
    s_red[2][wave] = mx;
  }
  __syncthreads();
  total = before = mx = 0;
  for (int w = 0; w < kThreads / 64; ++w) {
    total += s_red[0][w];
    before += s_red[1][w];
    mx = s_red[2][w] > mx ? s_red[2][w] : mx;
  }
  if (b == 0 && threadIdx.x == 0) {
    counts[B] = mx;
    counts[B + 1] = total;
    if (row_start != nullptr) row_start[B] = total;
  }
  // the slots that exist, row after row without the padding: where each one sits in (B, max_n)
  if (row_start != nullptr && threadIdx.x == 0) row_start[b] = before;
  if (row_slots != nullptr) {
    for (int n = threadIdx.x; n < counts[b]; n += kThreads) row_slots[before + n] = (int64_t)b * mx + n;
    // a caller may round the number of rows up to a multiple of kRowSlotsPad (slot 0 stands in)
    if (b == 0) {
      const int64_t cap = (int64_t)B * WL;
      int64_t end = ((int64_t)total + kRowSlotsPad - 1) / kRowSlotsPad * kRowSlotsPad;
      end = end < cap ? end : cap;
      for (int64_t n = total + threadIdx.x; n < end; n += kThreads) row_slots[n] = 0;
    }
  }
  // and their tokens in the same order (what the embedding lookup of the packed rows needs)
  if (row_tokens != nullptr) {
    for (int n = threadIdx.x; n < counts[b]; n += kThreads) row_tokens[before + n] = sel_tok[(int64_t)b * WL + n];
    if (b == 0) {
      const int64_t cap = (int64_t)B * WL;
      int64_t end = ((int64_t)total + kRowSlotsPad - 1) / kRowSlotsPad * kRowSlotsPad;
      end = end < cap ? end : cap;
      for (int64_t n = total + threadIdx.x; n < end; n += kThreads) row_tokens[n] = 0;
    }
  }
  for (int n = threadIdx.x; n < mx; n += kThreads) {
    int g = before + n;
    g = g < total - 1 ? g : total - 1;
    int r = b, lo = before;  // row r covers [lo, lo+counts[r])
    while (g >= lo + counts[r]) {
      lo += counts[r];
      ++r;
    }
    const int64_t src = (int64_t)r * WL + (g - lo);
    const int64_t dst = (int64_t)b * mx + n;
    const int f = sel_idx[src];
    packed_tokens[dst] = sel_tok[src];
    packed_token_indices[dst] = f;
    position_offsets[dst] = f % L;
  }
}

// ---------------------------------------------------------------------------------------------
// One workgroup per (batch row, packed slot).  Left part: the key's padding flag; tree part:
// True at the packed slots of the source beam's positions 0..k.
// ---------------------------------------------------------------------------------------------
template <typename PM>
__global__ __launch_bounds__(kThreads) void tree_mask_kernel(
    const int64_t* __restrict__ unpacker, const int64_t* __restrict__ packed_token_indices,
    const int32_t* __restrict__ counts, const PM* __restrict__ padding_mask,
    int64_t pm_row_stride, int64_t prev, int B, int WL, int L, uint8_t* __restrict__ mask,
    int64_t pm_pad_value) {
  const int max_n = counts[B];
  const int n = blockIdx.x;
  const int b = blockIdx.y;
  if (n >= max_n) return;
  __shared__ int s_tgt[kMaxLength];
  const int f = (int)packed_token_indices[(int64_t)b * max_n + n];
  const int i = f / L, k = f - i * L;
  if (threadIdx.x <= k) s_tgt[threadIdx.x] = (int)unpacker[(int64_t)b * WL + i * L + threadIdx.x];
  __syncthreads();

  const int64_t row_len = prev + max_n;
  const int64_t row_off = ((int64_t)b * max_n + n) * row_len;
  uint8_t* out = mask + row_off;
  const PM* pm = padding_mask + (int64_t)b * pm_row_stride;

  auto value = [&](int64_t c) -> uint8_t {
    if (c < prev) return pm[c] != (PM)pm_pad_value;
    const int t = (int)(c - prev);
    uint8_t hit = 0;
    for (int kk = 0; kk <= k; ++kk) hit |= (s_tgt[kk] == t);
    return hit;
  };

  int64_t head = (16 - (row_off & 15)) & 15;
  head = head < row_len ? head : row_len;
  for (int64_t c = threadIdx.x; c < head; c += kThreads) out[c] = value(c);
  const int64_t nvec = (row_len - head) >> 4;
  for (int64_t v = threadIdx.x; v < nvec; v += kThreads) {
    const int64_t c0 = head + (v << 4);
    union {
      uint8_t b8[16];
      uint4 v4;
    } u;
#pragma unroll
    for (int e = 0; e < 16; ++e) u.b8[e] = value(c0 + e);
    *reinterpret_cast<uint4*>(out + c0) = u.v4;
  }
  for (int64_t c = head + (nvec << 4) + threadIdx.x; c < row_len; c += kThreads) out[c] = value(c);
}

template <typename PM>
__global__ __launch_bounds__(kThreads) void causal_mask_kernel(const PM* __restrict__ padding_mask,
                                                              int64_t pm_row_stride, int64_t kv_len,
                                                              int64_t query_len,
                                                              uint8_t* __restrict__ mask) {
  const int64_t i = blockIdx.x;
  const int b = blockIdx.y;
  const PM* pm = padding_mask + (int64_t)b * pm_row_stride;
  uint8_t* out = mask + ((int64_t)b * query_len + i) * kv_len;
  const int64_t last = kv_len - query_len + i;  // last key this query may attend to
  for (int64_t j = threadIdx.x; j < kv_len; j += kThreads) out[j] = (j <= last) && (pm[j] != 0);
}

}  // namespace

extern "C" int rd_causal_mask(const void* padding_mask, int pm_elem_bytes, int64_t pm_row_stride,
                              int batch, int64_t kv_len, int64_t query_len, uint8_t* mask,
                              void* stream) {
  RD_REQUIRE(batch > 0 && kv_len > 0 && query_len > 0 && query_len <= kv_len, RD_EINVAL,
             "rd_causal_mask: bad sizes (batch %d kv_len %lld query_len %lld)", batch,
             (long long)kv_len, (long long)query_len);
  RD_REQUIRE(batch <= 65535 && query_len <= 2147483647LL, RD_ELIMIT, "rd_causal_mask: too large");
  RD_REQUIRE(padding_mask && mask, RD_EINVAL, "rd_causal_mask: null pointer");
  RD_REQUIRE(pm_row_stride >= kv_len, RD_EINVAL, "rd_causal_mask: pm_row_stride < kv_len");
  RD_REQUIRE(pm_elem_bytes == 1 || pm_elem_bytes == 4 || pm_elem_bytes == 8, RD_EINVAL,
             "rd_causal_mask: pm_elem_bytes must be 1, 4 or 8 (got %d)", pm_elem_bytes);
  hipStream_t s = rd::as_stream(stream);
  const dim3 grid((unsigned)query_len, batch);
#define RD_LAUNCH_CM(T)                                                                     \
  do { rd::ScopedTiming rd_t("causal_mask_kernel", s); hipLaunchKernelGGL(causal_mask_kernel<T>, grid, dim3(kThreads), 0, s,                      \
                     reinterpret_cast<const T*>(padding_mask), pm_row_stride, kv_len, query_len, mask); } while (0)
  if (pm_elem_bytes == 1) RD_LAUNCH_CM(uint8_t);
  else if (pm_elem_bytes == 4) RD_LAUNCH_CM(int32_t);
  else RD_LAUNCH_CM(int64_t);
#undef RD_LAUNCH_CM
  return rd::check_launch("rd_causal_mask");
}

extern "C" size_t rd_tree_workspace_bytes(int batch, int width, int length) {
  if (batch <= 0 || width <= 0 || length <= 0) return 0;
  const size_t n = (size_t)batch * width * length;
  return rd::align_up(n * sizeof(int64_t), 256) + rd::align_up(n * sizeof(int32_t), 256);
}

extern "C" int rd_tree_build(const int64_t* beams, int batch, int width, int length,
                             int64_t* prefix_tree, int64_t* unpacker, int64_t* packed_tokens,
                             int64_t* packed_token_indices, int64_t* position_offsets,
                             int32_t* counts, int32_t* row_start, int64_t* row_slots,
                             int64_t* row_tokens, void* workspace, size_t workspace_bytes, void* stream) {
  RD_REQUIRE(batch > 0 && width > 0 && length > 0, RD_EINVAL,
             "rd_tree_build: batch/width/length must be positive (%d,%d,%d)", batch, width, length);
  RD_REQUIRE(width <= kMaxWidth && length <= kMaxLength && width * length <= kMaxTokens, RD_ELIMIT,
             "rd_tree_build: width %d (<=%d), length %d (<=%d), width*length (<=%d)", width,
             kMaxWidth, length, kMaxLength, kMaxTokens);
  RD_REQUIRE(batch <= 65535, RD_ELIMIT, "rd_tree_build: batch %d > 65535", batch);
  RD_REQUIRE(beams && unpacker && packed_tokens && packed_token_indices && position_offsets &&
                 counts && workspace,
             RD_EINVAL, "rd_tree_build: null pointer");
  RD_REQUIRE(workspace_bytes >= rd_tree_workspace_bytes(batch, width, length), RD_EWORKSPACE,
             "rd_tree_build: workspace %zu < %zu bytes", workspace_bytes,
             rd_tree_workspace_bytes(batch, width, length));
  RD_REQUIRE(((uintptr_t)workspace & 255) == 0, RD_EINVAL, "rd_tree_build: workspace not 256B aligned");
  const size_t n = (size_t)batch * width * length;
  int64_t* sel_tok = reinterpret_cast<int64_t*>(workspace);
  int32_t* sel_idx = reinterpret_cast<int32_t*>(reinterpret_cast<char*>(workspace) +
                                                rd::align_up(n * sizeof(int64_t), 256));
  hipStream_t s = rd::as_stream(stream);
  { rd::ScopedTiming rd_t("tree_rows_kernel", s); hipLaunchKernelGGL(tree_rows_kernel, dim3(batch), dim3(kThreads), 0, s, beams, width, length,
                     prefix_tree, unpacker, sel_tok, sel_idx, counts); }
  if (int e = rd::check_launch("rd_tree_build(rows)")) return e;
  { rd::ScopedTiming rd_t("tree_fill_kernel", s); hipLaunchKernelGGL(tree_fill_kernel, dim3(batch), dim3(kThreads), 0, s, sel_tok, sel_idx, batch,
                     width * length, length, counts, packed_tokens, packed_token_indices,
                     position_offsets, row_start, row_slots, row_tokens); }
  return rd::check_launch("rd_tree_build(fill)");
}

extern "C" int rd_tree_mask(const int64_t* unpacker, const int64_t* packed_token_indices,
                            const int32_t* counts, const void* padding_mask, int pm_elem_bytes,
                            int64_t pm_row_stride, int64_t pm_pad_value, int64_t prev, int batch,
                            int width, int length, uint8_t* mask, void* stream) {
  RD_REQUIRE(batch > 0 && width > 0 && length > 0 && prev >= 0, RD_EINVAL,
             "rd_tree_mask: bad sizes (batch %d width %d length %d prev %lld)", batch, width, length,
             (long long)prev);
  RD_REQUIRE(length <= kMaxLength && width * length <= kMaxTokens, RD_ELIMIT,
             "rd_tree_mask: length %d (<=%d), width*length (<=%d)", length, kMaxLength, kMaxTokens);
  RD_REQUIRE(batch <= 65535, RD_ELIMIT, "rd_tree_mask: batch %d > 65535", batch);
  RD_REQUIRE(unpacker && packed_token_indices && counts && mask, RD_EINVAL,
             "rd_tree_mask: null pointer");
  RD_REQUIRE(prev == 0 || padding_mask, RD_EINVAL, "rd_tree_mask: padding_mask is null, prev > 0");
  RD_REQUIRE(prev == 0 || pm_row_stride >= prev, RD_EINVAL,
             "rd_tree_mask: pm_row_stride %lld < prev %lld", (long long)pm_row_stride,
             (long long)prev);
  RD_REQUIRE(pm_elem_bytes == 1 || pm_elem_bytes == 4 || pm_elem_bytes == 8, RD_EINVAL,
             "rd_tree_mask: pm_elem_bytes must be 1, 4 or 8 (got %d)", pm_elem_bytes);
  hipStream_t s = rd::as_stream(stream);
  const dim3 grid(width * length, batch);
  const int WL = width * length;
#define RD_LAUNCH_MASK(T)                                                                       \
  do { rd::ScopedTiming rd_t("tree_mask_kernel", s); hipLaunchKernelGGL(tree_mask_kernel<T>, grid, dim3(kThreads), 0, s, unpacker,                  \
                     packed_token_indices, counts, reinterpret_cast<const T*>(padding_mask),    \
                     pm_row_stride, prev, batch, WL, length, mask, pm_pad_value); } while (0)
  if (pm_elem_bytes == 1) RD_LAUNCH_MASK(uint8_t);
  else if (pm_elem_bytes == 4) RD_LAUNCH_MASK(int32_t);
  else RD_LAUNCH_MASK(int64_t);
#undef RD_LAUNCH_MASK
  return rd::check_launch("rd_tree_mask");
}
