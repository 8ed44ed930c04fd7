// Draft beams -> prefix tree -> packed tokens -> tree attention mask (gfx950).
//
// Integer, byte and index work only.  One workgroup per batch row keeps the row's beams in LDS;
// nothing is reshaped into a matrix product.  Three kernels:
//   tree_rows_kernel   per row: owner of every prefix, unpacker, the row's own packed list
//   tree_fill_kernel   per row: batch-wide offsets, max over rows, spill-over fill of the padding
//   tree_mask_kernel   per chunk of whole output lines: bytes of the (batch, max_n, prev+max_n) mask
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
// The byte mask (batch, max_n, prev + max_n).  Left part of a row: the key's padding flag; tree
// part: True at the packed slots of the source beam's positions 0..k.
// A workgroup writes one CHUNK of a batch row's mask bytes: a range of whole 128-byte lines of the
// output, about kMaskRows mask rows long (16 KiB at most), whatever the row length -- so every line
// is written once, in full, by one workgroup (a workgroup per mask row wrote 2.7 kB rows that
// start and end in the middle of lines: 2.3x the traffic on short rows, 90 000 workgroups on a
// batch of 512).  Per chunk the row's padding flags are turned into bit words once (LDS), and the
// (k, target slots) of the chunk's rows are staged in LDS.
// ---------------------------------------------------------------------------------------------
constexpr int kMaskRows = 30;        // mask rows per chunk, about
constexpr int kMaskRowsLds = 34;     // rows a chunk can touch: kMaskRows + both partial ends + slack
constexpr int kMaskMaxChunk = 16384;
constexpr int kMaskLeftWords = 2048; // padding flags of at most 131072 keys

__host__ __device__ inline int64_t mask_chunk_bytes(int64_t row_len) {
  int64_t c = kMaskRows * row_len / 128 * 128;
  if (c < 128) c = kMaskRows * row_len;  // rows of a few bytes: whole lines are not worth keeping to
  return c > kMaskMaxChunk ? kMaskMaxChunk : c;
}

// eight bits -> eight bytes of 0 / 1, bit 0 in the lowest byte
__device__ inline uint64_t bits_to_bytes(uint32_t b) {
  const uint64_t spread = ((uint64_t)b * 0x0101010101010101ull) & 0x8040201008040201ull;
  return ((spread + 0x7f7f7f7f7f7f7f7full) >> 7) & 0x0101010101010101ull;
}

template <typename PM>
__global__ __launch_bounds__(kThreads) void tree_mask_kernel(
    const int64_t* __restrict__ unpacker, const int64_t* __restrict__ packed_token_indices,
    const int32_t* __restrict__ counts, const PM* __restrict__ padding_mask,
    int64_t pm_row_stride, int64_t prev, int B, int WL, int L, uint8_t* __restrict__ mask,
    int64_t pm_pad_value) {
  __shared__ uint64_t s_left[kMaskLeftWords];
  __shared__ int16_t s_tgt[kMaskRowsLds * kMaxLength];
  __shared__ int s_k[kMaskRowsLds];
  const int max_n = counts[B];
  const int b = blockIdx.y;
  const int64_t row_len = prev + max_n;
  const int64_t total = (int64_t)max_n * row_len;  // mask bytes of one batch row
  const int64_t chunk = mask_chunk_bytes(row_len);
  // chunks are cut at absolute 128-byte lines of the output
  const uintptr_t base_addr = reinterpret_cast<uintptr_t>(mask) + (uintptr_t)((int64_t)b * total);
  const int64_t lead = (int64_t)(base_addr & 127);  // bytes of this batch row's first line that belong to the row before
  int64_t lo = (int64_t)blockIdx.x * chunk - lead, hi = lo + chunk;  // relative to the batch row's first byte
  lo = lo < 0 ? 0 : lo;
  hi = hi > total ? total : hi;
  if (lo >= hi) return;
  const int q0 = (int)(lo / row_len), q1 = (int)((hi - 1) / row_len);  // first and last mask row touched
  // stage: k and the target slots of every row touched; the padding flags of the left part as bits
  for (int t = threadIdx.x; t < (q1 - q0 + 1) * L; t += kThreads) {
    const int r = t / L, kk = t - r * L;
    const int f = (int)packed_token_indices[(int64_t)b * max_n + q0 + r];
    const int i = f / L, k = f - i * L;
    if (kk == 0) s_k[r] = k;
    s_tgt[r * kMaxLength + kk] = kk <= k ? (int16_t)unpacker[(int64_t)b * WL + i * L + kk] : (int16_t)-1;
  }
  {
    const PM* pm = padding_mask + (int64_t)b * pm_row_stride;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nw = (int)((prev + 63) >> 6);
    // four words per wave and round: the loads of a round are in flight together
    constexpr int kWavesHere = kThreads / 64;
    for (int w0 = wave; w0 < nw; w0 += 4 * kWavesHere) {
      bool on[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t j = (int64_t)(w0 + u * kWavesHere) * 64 + lane;
        on[u] = j < prev && pm[j] != (PM)pm_pad_value;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const uint64_t word = __ballot(on[u]);
        if (lane == 0 && w0 + u * kWavesHere < nw) s_left[w0 + u * kWavesHere] = word;
      }
    }
  }
  __syncthreads();
  uint8_t* out = mask + (int64_t)b * total;
  const int nw_left = (int)((prev + 63) >> 6);
  // flags of columns c .. c+15 of staged row r as sixteen bits (columns past the row's end: junk)
  auto row_flags = [&](int r, int64_t c) -> uint32_t {
    uint32_t f = 0;
    if (c < prev) {
      const int w = (int)(c >> 6), sh = (int)(c & 63);
      uint64_t x = s_left[w] >> sh;
      if (sh > 48 && w + 1 < nw_left) x |= s_left[w + 1] << (64 - sh);
      f = (uint32_t)x & 0xffffu;  // (bits of columns >= prev are zero in the words)
    }
    if (c + 16 > prev) {
      const int16_t* tg = s_tgt + r * kMaxLength;
      const int k = s_k[r];
      for (int kk = 0; kk <= k; ++kk) {
        const int64_t d = prev + tg[kk] - c;
        if ((uint64_t)d < 16) f |= 1u << d;
      }
    }
    return f;
  };
  // sixteen consecutive mask bytes that begin at column c of staged row r, as bits; they may run on
  // into the following rows
  auto flags16 = [&](int r, int64_t c) -> uint32_t {
    uint32_t f = row_flags(r, c);
    int64_t have = row_len - c;  // bytes of f that belong to row r
    while (have < 16) {
      ++r;
      f = (f & ((1u << have) - 1u)) | (row_flags(r, 0) << have);
      have += row_len;
    }
    return f & 0xffffu;
  };
  // bytes in front of the first 16-byte boundary, whole 16-byte vectors, bytes behind the last one
  int64_t head = (16 - (int64_t)((base_addr + (uintptr_t)lo) & 15)) & 15;
  head = head < hi - lo ? head : hi - lo;
  const int64_t nvec = (hi - lo - head) >> 4;
  for (int64_t o = lo + threadIdx.x; o < lo + head; o += kThreads)
    out[o] = (uint8_t)(row_flags((int)(o / row_len) - q0, o % row_len) & 1u);
  // a thread's vectors are kThreads * 16 bytes apart: (row, column) of the first one by division,
  // of the others by stepping
  int r_next = 0;
  int64_t c_next = 0;
  if (threadIdx.x < nvec) {
    const int64_t o = lo + head + ((int64_t)threadIdx.x << 4);
    r_next = (int)(o / row_len);
    c_next = o - (int64_t)r_next * row_len;
    r_next -= q0;
  }
  for (int64_t v = threadIdx.x; v < nvec; v += kThreads) {
    const int64_t o = lo + head + (v << 4);
    const uint32_t f = flags16(r_next, c_next);
    c_next += kThreads * 16;
    while (c_next >= row_len) { c_next -= row_len; ++r_next; }
    union {
      uint64_t b64[2];
      uint4 v4;
    } u;
    u.b64[0] = bits_to_bytes(f & 0xffu);
    u.b64[1] = bits_to_bytes(f >> 8);
    *reinterpret_cast<uint4*>(out + o) = u.v4;
  }
  for (int64_t o = lo + head + (nvec << 4) + threadIdx.x; o < hi; o += kThreads)
    out[o] = (uint8_t)(row_flags((int)(o / row_len) - q0, o % row_len) & 1u);
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
  RD_REQUIRE(prev <= (int64_t)kMaskLeftWords * 64, RD_ELIMIT, "rd_tree_mask: prev %lld > %d", (long long)prev,
             kMaskLeftWords * 64);
  hipStream_t s = rd::as_stream(stream);
  const int WL = width * length;
  // chunks per batch row for the largest tree the buffers allow (the real size is on the device):
  // 64 KiB chunks of long rows, or about kMaskRows rows of short ones
  const int64_t cap_bytes = (int64_t)WL * (prev + WL);
  const int64_t chunks = cap_bytes / kMaskMaxChunk + WL / (kMaskRows - 2) + 4;  // (an upper bound for any tree size)
  RD_REQUIRE(chunks <= 2147483647LL, RD_ELIMIT, "rd_tree_mask: mask too large");
  const dim3 grid((unsigned)chunks, batch);
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
