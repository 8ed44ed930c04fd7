// Row movement kernels (gfx950): pure HBM traffic, 16-byte lanes, no arithmetic.
//   gather_rows_kernel   out[b,t,:] = src[b, index[b,t], :]          (unpack of hidden/logits)
//   kv_unpack_kernel     cache[.., prev+t, :] = cache[.., prev+index[b,t], :] in place, per slab
//   kv_compact_kernel    keep the accepted rows and re-right-align each row's live region in place
// A "slab" is one (layer, key|value, batch row, head) block of max_len rows of head_dim elements.
#include "rd_common.h"

namespace {

constexpr int kThreads = 256;

// (a plain vector type: arrays of HIP's uint4 class were placed in scratch memory by the compiler)
typedef unsigned int vec16 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(kThreads) void gather_rows_kernel(
    const char* __restrict__ src, int64_t src_batch_stride, int64_t row_bytes,
    const int64_t* __restrict__ index, int64_t index_batch_stride, int n_src,
    char* __restrict__ dst, int64_t dst_batch_stride, int64_t dst_row_stride, int vec_bytes,
    const int32_t* __restrict__ row_start) {
  const int t = blockIdx.x, b = blockIdx.y;
  const int64_t r = index[(int64_t)b * index_batch_stride + t];
  // packed source rows (row_start): batch row b owns rows [row_start[b], row_start[b + 1])
  const int64_t first = row_start ? row_start[b] : 0;
  const int64_t limit = row_start ? row_start[b + 1] - first : n_src;
  if (r < 0 || r >= limit || r >= n_src) return;  // a corrupt index must not leave the buffer
  const char* s = src + (row_start ? first * row_bytes : (int64_t)b * src_batch_stride) + r * row_bytes;
  char* d = dst + (int64_t)b * dst_batch_stride + (int64_t)t * dst_row_stride;
  if (vec_bytes == 16) {
    const int64_t n = row_bytes >> 4;
    for (int64_t i = threadIdx.x; i < n; i += kThreads)
      reinterpret_cast<vec16*>(d)[i] = reinterpret_cast<const vec16*>(s)[i];
  } else if (vec_bytes == 4) {
    const int64_t n = row_bytes >> 2;
    for (int64_t i = threadIdx.x; i < n; i += kThreads)
      reinterpret_cast<uint32_t*>(d)[i] = reinterpret_cast<const uint32_t*>(s)[i];
  } else {
    for (int64_t i = threadIdx.x; i < row_bytes; i += kThreads) d[i] = s[i];
  }
}

// Source rows [prev, prev+n_src) are staged in LDS column-chunk by column-chunk, then the T
// destination rows are written from LDS: the ranges overlap, so reads must precede writes.
__global__ __launch_bounds__(kThreads) void kv_unpack_kernel(
    char* __restrict__ cache, int B, int H, int64_t max_len, int64_t row_bytes, int64_t prev,
    const int64_t* __restrict__ index, int T, int n_src, int chunk_bytes) {
  extern __shared__ vec16 s_rows[];
  const int64_t slab = blockIdx.x;
  const int b = (int)((slab / H) % B);
  char* base = cache + slab * max_len * row_bytes + prev * row_bytes;
  const int64_t* idx = index + (int64_t)b * T;
  // one column chunk of the slab per workgroup (blockIdx.y): narrow chunks keep the LDS share
  // small, so that several workgroups are resident and their read and write phases overlap
  const int64_t c0 = (int64_t)blockIdx.y * chunk_bytes;
  const int cb = (int)((row_bytes - c0) < chunk_bytes ? (row_bytes - c0) : chunk_bytes);
  const int vpr = cb >> 4;  // 16-byte vectors per row in this chunk
  for (int v = threadIdx.x; v < n_src * vpr; v += kThreads) {
    const int r = v / vpr, c = v - r * vpr;
    s_rows[v] = *reinterpret_cast<const vec16*>(base + (int64_t)r * row_bytes + c0 + (c << 4));
  }
  __syncthreads();
  for (int v = threadIdx.x; v < T * vpr; v += kThreads) {
    const int t = v / vpr, c = v - t * vpr;
    const int64_t r = idx[t];
    if (r >= 0 && r < n_src)
      *reinterpret_cast<vec16*>(base + (int64_t)t * row_bytes + c0 + (c << 4)) = s_rows[r * vpr + c];
  }
}

// plan: see realign_plan_kernel.  Per slab: (1) stash the accepted rows, (2) move the live region
// [old_pads, prev) to [new_pads, new_pads+live) with a direction-aware chunked memmove, (3) write
// the accepted rows behind it.
constexpr int kUnroll = 4;

__global__ __launch_bounds__(kThreads) void kv_compact_kernel(
    char* __restrict__ cache, int B, int H, int64_t max_len, int64_t row_bytes,
    const int32_t* __restrict__ plan, int L) {
  // A plan is trusted only as far as it stays inside the slab.
  extern __shared__ vec16 s_acc[];  // L rows
  const int64_t slab = blockIdx.x;
  const int b = (int)((slab / H) % B);
  const int32_t* rp = plan + 4 + (int64_t)b * (4 + L);
  const int old_pads = rp[0], new_pads = rp[1], n_new = rp[2], live = rp[3];
  if (old_pads < 0 || new_pads < 0 || live < 0 || n_new < 0 || n_new > L ||
      (int64_t)old_pads + live > max_len || (int64_t)new_pads + live + n_new > max_len)
    return;
  char* base = cache + slab * max_len * row_bytes;
  const int vpr = (int)(row_bytes >> 4);

  for (int v = threadIdx.x; v < n_new * vpr; v += kThreads) {
    const int j = v / vpr, c = v - j * vpr;
    int64_t row = rp[4 + j];
    row = (row < 0 || row >= max_len) ? 0 : row;
    s_acc[v] = *reinterpret_cast<const vec16*>(base + row * row_bytes + (c << 4));
  }
  __syncthreads();  // accepted rows are safe in LDS before anything is overwritten

  const int64_t nvec = (int64_t)live * vpr;
  const vec16* src = reinterpret_cast<const vec16*>(base + (int64_t)old_pads * row_bytes);
  vec16* dst = reinterpret_cast<vec16*>(base + (int64_t)new_pads * row_bytes);
  constexpr int64_t kChunk = (int64_t)kThreads * kUnroll;
  if (new_pads != old_pads && nvec > 0) {
    const int64_t n_chunks = (nvec + kChunk - 1) / kChunk;
    for (int64_t it = 0; it < n_chunks; ++it) {
      // moving right: highest chunk first; moving left: lowest chunk first
      const int64_t ch = new_pads > old_pads ? n_chunks - 1 - it : it;
      // (loads past the end are clamped, not skipped: an element left unset on some path would
      // send the whole array through scratch memory, i.e. through HBM a second time)
      vec16 r[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int64_t i = ch * kChunk + (int64_t)u * kThreads + threadIdx.x;
        r[u] = src[i < nvec ? i : nvec - 1];
      }
      __syncthreads();  // the whole chunk is in registers before any of it is overwritten
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int64_t i = ch * kChunk + (int64_t)u * kThreads + threadIdx.x;
        if (i < nvec) dst[i] = r[u];
      }
    }
  }
  vec16* tail = reinterpret_cast<vec16*>(base + (int64_t)(new_pads + live) * row_bytes);
  for (int v = threadIdx.x; v < n_new * vpr; v += kThreads) tail[v] = s_acc[v];
}

// The re-alignment when no row moves (plans written for rows kept in place: old_pads == new_pads):
// only the accepted rows are copied behind the live ones.  Eight slabs per workgroup, 32 threads
// each: one slab per workgroup is 16 384 workgroups of which most threads have nothing to do.
constexpr int kAppendSlabs = 8, kAppendPer = 8;  // slabs per workgroup, vectors per thread

__global__ __launch_bounds__(kThreads) void kv_append_kernel(
    char* __restrict__ cache, int64_t slabs, int B, int H, int64_t max_len, int64_t row_bytes,
    const int32_t* __restrict__ plan, int L) {
  const int sub = threadIdx.x >> 5, lane = threadIdx.x & 31;
  const int64_t slab = (int64_t)blockIdx.x * kAppendSlabs + sub;
  const bool valid = slab < slabs;
  const int b = valid ? (int)((slab / H) % B) : 0;
  const int32_t* rp = plan + 4 + (int64_t)b * (4 + L);
  const int start = rp[1], live = rp[3];
  int n_new = rp[2];
  if (!valid || start < 0 || live < 0 || n_new < 0 || n_new > L || (int64_t)start + live + n_new > max_len) n_new = 0;
  char* base = cache + (valid ? slab : 0) * max_len * row_bytes;
  const int vpr = (int)(row_bytes >> 4);
  const int total = n_new * vpr;
  vec16 r[kAppendPer];
#pragma unroll
  for (int u = 0; u < kAppendPer; ++u) {
    // Every thread reads something, whether its vector is wanted or not (a read that is skipped on
    // some path would send the array through scratch memory); an unwanted one re-reads the first
    // vector of the first row.  The plan's row entry is picked without looking at n_new, so that
    // it is requested together with the plan's counts instead of after them (entries past n_new
    // may hold anything: they are read, never used).
    const int v = lane + 32 * u;
    int j = v / vpr;
    int c = v - j * vpr;
    j = j < L ? j : L - 1;
    const int32_t listed = rp[4 + j], first = rp[4];
    const bool want = v < total;
    int64_t row = want ? listed : first;
    c = want ? c : 0;
    row = (row < 0 || row >= max_len) ? 0 : row;
    r[u] = *reinterpret_cast<const vec16*>(base + row * row_bytes + (c << 4));
  }
  __syncthreads();  // source and destination rows of a slab overlap: every read precedes every write
  vec16* tail = reinterpret_cast<vec16*>(base + (int64_t)(start + live) * row_bytes);
#pragma unroll
  for (int u = 0; u < kAppendPer; ++u) {
    const int v = lane + 32 * u;
    if (v < total) tail[v] = r[u];
  }
}

// Plan that moves every row of the cache from where it physically is (token column c in cache row
// c - shift[b]) to the layout in which column and cache row agree; the shifts are cleared.
__global__ void materialize_plan_kernel(int32_t* __restrict__ shift, int B, int64_t length,
                                        int64_t max_len, int32_t* __restrict__ plan) {
  for (int b = threadIdx.x; b < B; b += blockDim.x) {
    const int64_t s = shift[b];
    int64_t p0 = s < 0 ? -s : 0;                 // first cache row whose column is not negative
    int64_t p1 = length - s;                     // cache row of column `length`
    p1 = p1 > max_len ? max_len : p1;
    if (p1 + s > max_len) p1 = max_len - s;
    const int64_t live = p1 > p0 ? p1 - p0 : 0;
    int32_t* rp = plan + 4 + (int64_t)b * 5;
    rp[0] = (int32_t)p0; rp[1] = (int32_t)(p0 + s); rp[2] = 0; rp[3] = (int32_t)live; rp[4] = 0;
    shift[b] = 0;
  }
  if (threadIdx.x == 0) { plan[0] = (int32_t)length; plan[1] = (int32_t)length; plan[2] = 1; plan[3] = 0; }
}

int check_cache_args(const char* who, const void* cache, int n_layers, int B, int H,
                     int64_t max_len, int64_t row_bytes) {
  RD_REQUIRE(cache, RD_EINVAL, "%s: null cache", who);
  RD_REQUIRE(n_layers > 0 && B > 0 && H > 0 && max_len > 0 && row_bytes > 0, RD_EINVAL,
             "%s: bad cache shape (layers %d batch %d heads %d max_len %lld row_bytes %lld)", who,
             n_layers, B, H, (long long)max_len, (long long)row_bytes);
  RD_REQUIRE(row_bytes % 16 == 0 && ((uintptr_t)cache % 16) == 0, RD_EINVAL,
             "%s: rows must be 16-byte multiples and the cache 16-byte aligned (row_bytes %lld)",
             who, (long long)row_bytes);
  RD_REQUIRE((int64_t)n_layers * 2 * B * H <= 2147483647LL, RD_ELIMIT, "%s: too many slabs", who);
  return RD_OK;
}

}  // namespace

extern "C" int rd_unpack_rows(const void* packed, int64_t packed_batch_stride_bytes,
                              int64_t row_bytes, const int64_t* index, int64_t index_batch_stride,
                              int batch, int n_out, int n_src, void* out,
                              int64_t out_batch_stride_bytes, int64_t out_row_stride_bytes,
                              const int32_t* row_start, void* stream) {
  RD_REQUIRE(batch > 0 && n_out > 0 && n_src > 0 && row_bytes > 0, RD_EINVAL,
             "rd_unpack_rows: bad sizes (batch %d n_out %d n_src %d row_bytes %lld)", batch, n_out,
             n_src, (long long)row_bytes);
  RD_REQUIRE(batch <= 65535, RD_ELIMIT, "rd_unpack_rows: batch %d > 65535", batch);
  RD_REQUIRE(packed && index && out, RD_EINVAL, "rd_unpack_rows: null pointer");
  RD_REQUIRE(index_batch_stride >= n_out, RD_EINVAL, "rd_unpack_rows: index_batch_stride < n_out");
  RD_REQUIRE(out_row_stride_bytes >= row_bytes, RD_EINVAL,
             "rd_unpack_rows: out_row_stride_bytes %lld < row_bytes %lld",
             (long long)out_row_stride_bytes, (long long)row_bytes);
  RD_REQUIRE(out_batch_stride_bytes >= (int64_t)(n_out - 1) * out_row_stride_bytes + row_bytes,
             RD_EINVAL, "rd_unpack_rows: out_batch_stride_bytes too small");
  RD_REQUIRE(row_start || packed_batch_stride_bytes >= (int64_t)n_src * row_bytes, RD_EINVAL,
             "rd_unpack_rows: packed_batch_stride_bytes too small");
  const uintptr_t all = (uintptr_t)packed | (uintptr_t)out | (uintptr_t)row_bytes |
                        (uintptr_t)(row_start ? 0 : packed_batch_stride_bytes) | (uintptr_t)out_batch_stride_bytes |
                        (uintptr_t)out_row_stride_bytes;
  const int vec = (all % 16 == 0) ? 16 : (all % 4 == 0 ? 4 : 1);
  { rd::ScopedTiming rd_t("gather_rows_kernel", rd::as_stream(stream)); hipLaunchKernelGGL(gather_rows_kernel, dim3(n_out, batch), dim3(kThreads), 0,
                     rd::as_stream(stream), reinterpret_cast<const char*>(packed),
                     packed_batch_stride_bytes, row_bytes, index, index_batch_stride, n_src,
                     reinterpret_cast<char*>(out), out_batch_stride_bytes, out_row_stride_bytes, vec, row_start); }
  return rd::check_launch("rd_unpack_rows");
}

extern "C" int rd_kv_unpack(void* cache, int n_layers, int batch, int n_heads, int64_t max_len,
                            int64_t row_bytes, int64_t prev, const int64_t* index, int n_out,
                            int n_src, void* stream) {
  if (int e = check_cache_args("rd_kv_unpack", cache, n_layers, batch, n_heads, max_len, row_bytes))
    return e;
  RD_REQUIRE(index && n_out > 0 && n_src > 0 && prev >= 0, RD_EINVAL,
             "rd_kv_unpack: bad arguments (n_out %d n_src %d prev %lld)", n_out, n_src,
             (long long)prev);
  RD_REQUIRE(prev + n_out <= max_len && prev + n_src <= max_len, RD_EINVAL,
             "rd_kv_unpack: prev %lld + max(n_out %d, n_src %d) exceeds max_len %lld",
             (long long)prev, n_out, n_src, (long long)max_len);
  constexpr int kLds = 64 * 1024;
  RD_REQUIRE((int64_t)n_src * 16 <= kLds, RD_ELIMIT, "rd_kv_unpack: n_src %d > %d", n_src, kLds / 16);
  // column chunk: one 128-byte line per row (whole 256-byte rows left too few workgroups resident:
  // 450 us against 352 us for the 7B cache at 1500 tokens; 64-byte pieces took 624 us)
  int64_t chunk = (int64_t)n_src * 128 <= kLds ? 128 : (kLds / n_src) / 16 * 16;
  if (chunk > row_bytes) chunk = row_bytes;
  const size_t lds = (size_t)n_src * chunk;
  const int64_t slabs = (int64_t)n_layers * 2 * batch * n_heads;
  const int col_chunks = (int)((row_bytes + chunk - 1) / chunk);
  RD_REQUIRE(col_chunks <= 65535, RD_ELIMIT, "rd_kv_unpack: row_bytes %lld needs %d column chunks", (long long)row_bytes, col_chunks);
  { rd::ScopedTiming rd_t("kv_unpack_kernel", rd::as_stream(stream)); hipLaunchKernelGGL(kv_unpack_kernel, dim3(slabs, col_chunks), dim3(kThreads), lds, rd::as_stream(stream),
                     reinterpret_cast<char*>(cache), batch, n_heads, max_len, row_bytes, prev, index,
                     n_out, n_src, (int)chunk); }
  return rd::check_launch("rd_kv_unpack");
}

extern "C" int rd_kv_compact(void* cache, int n_layers, int batch, int n_heads, int64_t max_len,
                             int64_t row_bytes, int64_t prev, int length, const int32_t* plan,
                             void* stream) {
  if (int e = check_cache_args("rd_kv_compact", cache, n_layers, batch, n_heads, max_len, row_bytes))
    return e;
  RD_REQUIRE(plan && length > 0, RD_EINVAL, "rd_kv_compact: null plan or length %d", length);
  RD_REQUIRE(prev >= 0 && prev + length <= max_len, RD_EINVAL,
             "rd_kv_compact: prev %lld + length %d exceeds max_len %lld", (long long)prev, length,
             (long long)max_len);
  const size_t lds = (size_t)length * row_bytes;
  RD_REQUIRE(lds <= 64 * 1024, RD_ELIMIT, "rd_kv_compact: length*row_bytes %zu > 65536", lds);
  const int64_t slabs = (int64_t)n_layers * 2 * batch * n_heads;
  { rd::ScopedTiming rd_t("kv_compact_kernel", rd::as_stream(stream)); hipLaunchKernelGGL(kv_compact_kernel, dim3(slabs), dim3(kThreads), lds, rd::as_stream(stream),
                     reinterpret_cast<char*>(cache), batch, n_heads, max_len, row_bytes, plan, length); }
  return rd::check_launch("rd_kv_compact");
}

extern "C" size_t rd_kv_materialize_plan_ints(int batch) { return batch > 0 ? 4 + (size_t)batch * 5 : 0; }

extern "C" int rd_kv_materialize(void* cache, int n_layers, int batch, int n_heads, int64_t max_len,
                                 int64_t row_bytes, int64_t length, int32_t* kv_row_shift,
                                 int32_t* plan, void* stream) {
  if (int e = check_cache_args("rd_kv_materialize", cache, n_layers, batch, n_heads, max_len, row_bytes))
    return e;
  RD_REQUIRE(kv_row_shift && plan && length >= 0 && length <= max_len, RD_EINVAL,
             "rd_kv_materialize: null pointer or length %lld outside [0, %lld]", (long long)length,
             (long long)max_len);
  RD_REQUIRE(row_bytes <= 64 * 1024, RD_ELIMIT, "rd_kv_materialize: row_bytes %lld > 65536", (long long)row_bytes);
  hipStream_t s = rd::as_stream(stream);
  hipLaunchKernelGGL(materialize_plan_kernel, dim3(1), dim3(kThreads), 0, s, kv_row_shift, batch, length, max_len, plan);
  if (int e = rd::check_launch("rd_kv_materialize(plan)")) return e;
  const int64_t slabs = (int64_t)n_layers * 2 * batch * n_heads;
  { rd::ScopedTiming rd_t("kv_compact_kernel", s); hipLaunchKernelGGL(kv_compact_kernel, dim3(slabs), dim3(kThreads), (size_t)row_bytes, s,
                     reinterpret_cast<char*>(cache), batch, n_heads, max_len, row_bytes, plan, 1); }
  return rd::check_launch("rd_kv_materialize");
}

extern "C" int rd_kv_append(void* cache, int n_layers, int batch, int n_heads, int64_t max_len,
                            int64_t row_bytes, int length, const int32_t* plan, void* stream) {
  if (int e = check_cache_args("rd_kv_append", cache, n_layers, batch, n_heads, max_len, row_bytes))
    return e;
  RD_REQUIRE(plan && length > 0, RD_EINVAL, "rd_kv_append: null plan or length %d", length);
  RD_REQUIRE((int64_t)length * (row_bytes >> 4) <= 32 * kAppendPer, RD_ELIMIT,
             "rd_kv_append: length %d x row_bytes %lld is more than %d bytes per slab", length,
             (long long)row_bytes, 32 * kAppendPer * 16);
  const int64_t slabs = (int64_t)n_layers * 2 * batch * n_heads;
  const int64_t grid = (slabs + kAppendSlabs - 1) / kAppendSlabs;
  { rd::ScopedTiming rd_t("kv_append_kernel", rd::as_stream(stream)); hipLaunchKernelGGL(kv_append_kernel, dim3((unsigned)grid), dim3(kThreads), 0, rd::as_stream(stream),
                     reinterpret_cast<char*>(cache), slabs, batch, n_heads, max_len, row_bytes, plan, length); }
  return rd::check_launch("rd_kv_append");
}
