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
//                         v_mfma_f32_32x32x16_bf16.  512 threads = 8 waves; a wave owns 32 query
//                         rows (with at most 128 rows per workgroup, two waves share a row block
//                         and split every tile's keys).  64-key K and V tiles travel global ->
//                         register ring -> LDS as they lie in memory and are shared by the waves;
//                         the V^T operand of the second product comes out of transposing LDS
//                         reads (ds_read_b64_tr_b16).  The
//                         loop is a software pipeline over 32-key units: while the vector ALU turns
//                         the scores of one unit into probabilities (online softmax in fp32, lazy
//                         rescale), the matrix pipeline already multiplies the next unit's keys.
//                         With the transposed products a query row lives in one lane pair, so the
//                         row maximum and sum need a single cross-lane exchange, and P^T is already
//                         laid out as the B operand of the second product.
//   attn_generic_kernel   any dtype, head_dim <= 256, one workgroup per (row, head, query); the
//                         correctness path for shapes the MFMA kernel does not cover.
// Work items come from the plan (attn_plan.h): (batch row, key range) chunks, longest first; rows
// whose keys are split over several items write fp32 partials, and the item that finishes last
// merges them (an arrival counter per (row, head, query tile); every launch counts on a slab of its
// own, taken from a ring of counters that is part of the library).
#include <hip/hip_bf16.h>
#include <hip/hip_ext.h>
#include <hip/hip_fp16.h>

#include <mutex>
#include <type_traits>

#include "attn_addr.h"
#include "attn_plan.h"
#include "rd_common.h"

namespace {

// tile sizes, wave layouts, loader roles and every index formula of the MFMA kernel (attn_addr.h)
using namespace rd::attn;

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
  // Packed query rows (or null): row t of batch row b is row row_start[b] + t of q and out (their
  // batch strides are unused) and exists only for t < row_start[b + 1] - row_start[b].  The mask
  // rows and the partials keep the padded (batch, n_q) layout.
  const int32_t* row_start;
  unsigned int* counters;  // arrival counters of this launch, [batch][heads][query tiles]; zero before and after
  int B, H, Hkv, n_q, kv_len, words, max_splits, D;
  float scale;  // softmax scale; the MFMA kernel works in log2 units (scale * log2 e)
  // Rotary embedding and cache append fused in (the ROPE instantiation of the MFMA kernel): q arrives
  // unrotated; k_new / v_new (token rows like q's, heads D apart, strides {batch, token}) are the new
  // keys and values, whose rotated / copied rows belong at key columns [new_col0, new_col0 + n_q) of
  // k and v; cos / sin (table_rows, D) and position_ids (batch, n_q) as for rd_rope_append.
  const void* k_new; int64_t kn_sb, kn_st;
  const void* v_new; int64_t vn_sb, vn_st;
  const void* cos; const void* sin; int64_t table_rows;
  const int64_t* position_ids; int64_t pos_sb;
  int new_col0;       // kv_len - n_q
  int64_t max_len;    // cache rows of a slab: a new row that a shift would put outside is dropped
};

__device__ inline float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Query rows of batch row b: their count and the element offsets of row 0 in q and out.
struct RowSpan { int n; int64_t q_off, o_off; int r0; };  // r0: first packed row, or -1 (padded layout)
__device__ inline RowSpan row_span(const AttnArgs& a, int b) {
  if (a.row_start == nullptr) return {a.n_q, (int64_t)b * a.q_sb, (int64_t)b * a.o_sb, -1};
  const int r0 = a.row_start[b], r1 = a.row_start[b + 1];
  const int n = r1 - r0;
  return {n < a.n_q ? n : a.n_q, (int64_t)r0 * a.q_ss, (int64_t)r0 * a.o_ss, r0};
}

// the same from `wide`, which holds entry min(lane, batch) of row_start in every lane (batch < 64:
// every entry is in some lane; otherwise the two entries are loaded)
__device__ inline RowSpan row_span(const AttnArgs& a, int b, int wide) {
  if (a.row_start == nullptr || a.B >= 64) return row_span(a, b);
  const int r0 = __builtin_amdgcn_readlane(wide, b), r1 = __builtin_amdgcn_readlane(wide, b + 1);
  const int n = r1 - r0;
  return {n < a.n_q ? n : a.n_q, (int64_t)r0 * a.q_ss, (int64_t)r0 * a.o_ss, r0};
}

// round to bf16 and back; products and sums of the rotation are rounded one by one, as the separate
// elementwise kernels of the reference's op chain round them (no fused multiply-add)
__device__ inline float bf16_round(float v) { return static_cast<float>(static_cast<__bf16>(v)); }
__device__ inline float rope_lo(float x1, float x2, float c, float s) {
#pragma clang fp contract(off)
  const float p = bf16_round(x1 * c), q = bf16_round(x2 * s);
  return p - q;
}
__device__ inline float rope_hi(float x1, float x2, float c, float s) {
#pragma clang fp contract(off)
  const float p = bf16_round(x2 * c), q = bf16_round(x1 * s);
  return p + q;
}

// ---------------------------------------------------------------------------------------------
// MFMA kernel
// ---------------------------------------------------------------------------------------------
constexpr int kMfmaThreads = kThreads;  // 512

template <int N, typename F, int I = 0>
__device__ __attribute__((always_inline)) inline void rd_static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    rd_static_for<N, F, I + 1>(static_cast<F&&>(f));
  }
}
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

template <int LAYOUT, bool ROPE>
__global__ __launch_bounds__(kMfmaThreads) void attn_mfma_kernel(AttnArgs a) {
  constexpr int kRowsPerWG = rows_per_wg(LAYOUT);
  constexpr bool kHasFull = LAYOUT != kSplit, kHasHalf = LAYOUT != kFull;
  __shared__ __attribute__((aligned(16))) char smem[kLdsBytes];

  // The item is requested together with the item count (one trip to memory instead of two; the
  // item array has a slot for every blockIdx.y), and every kernel argument is fetched up front:
  // fetched where first used, they cost one more wait each on the way to the first tile load.
  const int item = blockIdx.y;
  const int32_t* it = a.plan + RD_PLAN_HDR + 4 * a.B + RD_ITEM_INTS * item;
  const int n_items = a.plan[0];
  // Packed query rows: which rows belong to the item's batch row is an entry of row_start that could
  // only be asked for once the item is here -- one more trip to memory on the way to everything
  // else.  The lanes ask for all entries now (entry min(lane, batch); of the plan, which is at least
  // as long, where the rows are not packed: a load that always happens), and the item's two are
  // picked from them once it is known.
  const int wide_i = (int)(threadIdx.x & 63) < a.B ? (int)(threadIdx.x & 63) : a.B;
  const int wide = (a.row_start != nullptr ? a.row_start : a.plan)[wide_i];
  int b = it[0], lo = it[1], hi = it[2], split = it[3];
  int kv_shift = it[4];   // key column c of this row is cache row c - kv_shift
  int key_min = it[5];    // the keys some query of the row attends to lie in [key_min, key_end):
  int n_splits = it[6];
  int key_end = it[7];    // nothing outside that span is read
  asm volatile("" : "+s"(b), "+s"(lo), "+s"(hi), "+s"(split), "+s"(kv_shift), "+s"(key_min), "+s"(n_splits), "+s"(key_end));
  asm volatile("" ::"s"(a.q), "s"(a.q_sb), "s"(a.q_sh), "s"(a.q_ss), "s"(a.k), "s"(a.k_sb), "s"(a.k_sh), "s"(a.k_ss));
  asm volatile("" ::"s"(a.v), "s"(a.v_sb), "s"(a.v_sh), "s"(a.v_ss), "s"(a.bits), "s"(a.n_q), "s"(a.kv_len), "s"(a.words));
  if (item >= n_items) return;
  // query tiles of one (row, head, key range) are neighbours in dispatch order, so they run
  // together and the second read of the K/V tiles is served by the L2
  const int q_tiles = gridDim.x / a.H;
  const int h = blockIdx.x / q_tiles, q_tile = blockIdx.x - h * q_tiles;
  const int hk = h / (a.H / a.Hkv);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, and the compiler knows it
  const int g = lane >> 5, r = lane & 31;
  const WaveRole role = wave_role(LAYOUT, wave);
  const int row_wave = role.block;                     // row block of this wave
  const bool full = kHasFull && (!kHasHalf || role.part == 2);  // wave-uniform
  const int kp = full ? 0 : role.part;                 // key half of a half wave
  const __bf16* kbase = reinterpret_cast<const __bf16*>(a.k) + (int64_t)b * a.k_sb + (int64_t)hk * a.k_sh - (int64_t)kv_shift * a.k_ss;
  const __bf16* vbase = reinterpret_cast<const __bf16*>(a.v) + (int64_t)b * a.v_sb + (int64_t)hk * a.v_sh - (int64_t)kv_shift * a.v_ss;

  // Loader roles (attn_addr.h: loader_of): waves 0-3 stage the K tile, waves 4-7 the V tile, four
  // 16-byte chunks per thread and tile.
  const bool k_loader = wave < kWaves / 2;  // (== ld.k_loader, and wave-uniform for the compiler)
  const Loader ld = loader_of(tid);
  const int chunk = ld.chunk, lrow = ld.lrow;

  const int n_tiles = n_tiles_of(lo, hi);
  // Tiles in flight: a ring of kRing register stages between global memory and LDS; tile j
  // passes through slot j % kRing.  The mask words travel in a ring of their own.
  // Every step issues the same loads on every path (tile indices past the end are clamped to the
  // last tile, keys outside the row's span read as zeros): with loads under divergent or data-dependent
  // branches the compiler can no longer count which loads are still in flight and waits for all
  // of them at every use, which would cap the ring at one tile.
  static_assert(kRing == 2, "two named register stages");
  // the four 16-byte chunks a thread carries per tile, for ring slots 0 (a) and 1 (b); plain
  // variables: grouped in arrays or structs they are left in scratch memory
  bf16x8 a0, a1, a2, a3, b0, b1, b2, b3;
  uint64_t wring[kRing];
  // address of a 16-byte chunk = wave-uniform part (tile, i) + 32-bit lane part
  const char* base = reinterpret_cast<const char*>(k_loader ? kbase : vbase);
  const int64_t row_bytes = (k_loader ? a.k_ss : a.v_ss) * 2;
  const int key_step = ld.key_step, first_key = ld.first_key;  // this thread's keys within a tile: first_key + i * key_step
  // K and V come through a buffer descriptor over the cache rows of the keys that some query of the
  // row attends to (attn_addr.h: tile_chunk_offset): every step issues the same four loads whatever
  // the tile, and the lanes whose key lies outside that span -- left padding in front of it, tree
  // slots that do not exist and the end of the cache behind it -- get zeros without touching memory.
  // Non-temporal: every K and V row is read once per launch (twice when two query tiles or grouped
  // heads share it, back to back), so it should not push the L2's other lines out on its way
  // through.  In the decode step this alone takes the launch from 28.8 to 27.3 us at 600 keys per
  // row and from 85 to 70 us at 2500.
  const __amdgpu_buffer_rsrc_t tiles = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(base) + (int64_t)key_min * row_bytes, 0, (int)span_bytes(key_min, key_end, row_bytes), 0x00020000);
  const uint32_t lane_off = tile_chunk_offset(ld, 0, 0, 0, row_bytes);  // the thread's place in a tile
  const uint32_t step_bytes = (uint32_t)(key_step * row_bytes);
  constexpr int kNonTemporal = 2;
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  auto fetch_into = [&](bf16x8& c0, bf16x8& c1, bf16x8& c2, bf16x8& c3, int j) __attribute__((always_inline)) {
    const int key0 = tile_key0(lo, j, n_tiles);
    const uint32_t at = (uint32_t)((int64_t)(key0 - key_min) * row_bytes) + lane_off;  // (wraps below the span)
    const u32x4 w0 = __builtin_amdgcn_raw_buffer_load_b128(tiles, at, 0, kNonTemporal);
    const u32x4 w1 = __builtin_amdgcn_raw_buffer_load_b128(tiles, at + step_bytes, 0, kNonTemporal);
    const u32x4 w2 = __builtin_amdgcn_raw_buffer_load_b128(tiles, at + 2 * step_bytes, 0, kNonTemporal);
    const u32x4 w3 = __builtin_amdgcn_raw_buffer_load_b128(tiles, at + 3 * step_bytes, 0, kNonTemporal);
    c0 = __builtin_bit_cast(bf16x8, w0);
    c1 = __builtin_bit_cast(bf16x8, w1);
    c2 = __builtin_bit_cast(bf16x8, w2);
    c3 = __builtin_bit_cast(bf16x8, w3);
  };
  auto fetch_tile = [&](auto slot_c, int j) __attribute__((always_inline)) {
    if constexpr (decltype(slot_c)::value == 0) fetch_into(a0, a1, a2, a3, j); else fetch_into(b0, b1, b2, b3, j);
  };
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1 % kRing>;
  // What can be asked for with nothing but the work item is asked for now: a trip to memory takes
  // more than a microsecond at the start of a launch, and everything on the way to the first product
  // would otherwise queue up behind the item, the row's query rows and, with the rotation, the
  // positions and the table rows they select, one trip each.  First the positions (of the lane's
  // query row and of the new tokens whose keys this thread will rotate: eight bytes each, their
  // index clamped to the array instead of to the row's query count, which is not here yet), then
  // the first tiles.  Loads return in the order of their issue: the positions are back after one
  // trip, and the loads that depend on them go out while the tiles are still coming in.
  const int q_row = q_row_of(q_tile, kRowsPerWG, row_wave, r);
  // (ROPE) K tile j is requested in step j - 2 - kRing (the prologue for j < 2 + kRing), V tiles
  // later: t_first is the step whose barrier the new rows must have reached the cache by.  Where
  // that is the prologue itself (a short cache: its own tiles hold new rows), the rows are written
  // first, at the price of the trips saved here.
  const int first_new_tile = a.new_col0 > lo ? (a.new_col0 - lo) / kTile : 0;
  const int t_first = first_new_tile - 3 - kRing;
  const bool rows_first = ROPE && t_first < 0;  // (uniform over the workgroup)
  const int t_lo = new_rows_of_item(lo, hi, key_end, a.new_col0, 0).t_lo;  // (does not depend on the row's query count)
  int64_t q_pos = 0, pos_a[2] = {0, 0}, pos_b[2] = {0, 0};
  auto ask_positions = [&](int64_t (&pos)[2], int round) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int t = rope_k_token(t_lo + kNewRowsPerRound * round, tid, i);
      pos[i] = a.position_ids[(int64_t)b * a.pos_sb + (t < a.n_q ? t : a.n_q - 1)];
    }
  };
  if constexpr (ROPE) {
    q_pos = a.position_ids[(int64_t)b * a.pos_sb + (q_row < a.n_q ? q_row : a.n_q - 1)];
    ask_positions(pos_a, 0);
    ask_positions(pos_b, 1);  // (at most 256 new tokens: two rounds)
  }
  // Every thread issues the same eight loads here, on every path: the K loaders tiles 0 and 1, the V
  // loaders tile 0 twice (the second request rides on the first one's cache lines; the ring refills
  // that slot before anything reads it), and a workgroup that has to write new rows first asks too
  // and asks again later.  With a different number of loads on some path, every wait for an older
  // load below (the row's query rows, the positions) would have to be a wait for the path with the
  // fewest -- that is, for some or all of these tiles.
  // (Without the rotation the only older load is the one for the row's query rows: there the V
  // loaders skip the second request, and the K loaders' wait for those rows becomes a wait for their
  // first tile as well -- measured 0.35 us shorter per launch than with the extra requests.)
  fetch_tile(S0{}, 0);
  if constexpr (ROPE) fetch_tile(S1{}, k_loader ? 1 : 0);
  else if (k_loader) fetch_tile(S1{}, 1);
  const RowSpan rows = row_span(a, b, wide);
  if (q_tile * kRowsPerWG >= rows.n) return;  // (every thread of the workgroup: no barrier is skipped)
  const bool wave_active = q_tile * kRowsPerWG + row_wave * 32 < rows.n;
  const bool row_valid = q_row < rows.n;

  // ---- new cache rows and rotated queries (ROPE) ---------------------------------------------------
  // The new keys and values of this (batch row, kv head) go to their cache rows before anybody's
  // tile loads ask for them: the keys rotated by their positions, the values as they are -- what a
  // separate kernel did between the projection and this one (a launch, and a pass over q, k and v).
  // A workgroup writes the rows that its own tile loop may read (its item's share of the key
  // columns [new_col0, new_col0 + rows.n)); workgroups that share them (grouped heads) write the
  // same bytes.  Nobody else reads them in this launch.  The item that ends the row's key span
  // also writes what lies behind the span, so that rows nobody attends to reach the cache too.
  // A round covers 128 tokens: 1024 rotation tasks (a 16-byte chunk of the first half of a key and
  // its partner in the second half), two per thread, and 2048 copy tasks, four per thread.
  //
  // Order.  The first round's operands (the new keys and values, the table rows of their positions)
  // are requested once the row's query rows are known, behind the first tiles, and used after those
  // have been staged; a second round's (more than 128 tokens) go out then and are used under cover of
  // the ring's first loads.  The stores are not waited for in the prologue: the first tile that holds
  // new rows is requested many steps into the loop, and the step before that request waits for them
  // (t_sync), ahead of its barrier.
  const NewRows mine = new_rows_of_item(lo, hi, key_end, a.new_col0, rows.n);  // (uniform over the workgroup)
  const int t_hi = ROPE ? mine.t_hi : 0;
  const bool has_new = t_lo < t_hi;
  const bool second_round = t_lo + kNewRowsPerRound < t_hi;
  const int t_sync = has_new && !rows_first ? t_first : -1;  // the step whose barrier the rows need
  struct NewRows {
    bf16x8 x1[2], x2[2], vv[4], c1[2], c2[2], s1[2], s2[2];
    int kt[2], kc[2], vt[4], vc[4];  // token and chunk of every task; token -1: no task
  } nr;
  const __bf16* kn = nullptr; const __bf16* vn = nullptr;
  if constexpr (ROPE) {
    const int64_t new_off = rows.r0 >= 0 ? (int64_t)rows.r0 * a.kn_st : (int64_t)b * a.kn_sb;
    const int64_t newv_off = rows.r0 >= 0 ? (int64_t)rows.r0 * a.vn_st : (int64_t)b * a.vn_sb;
    kn = reinterpret_cast<const __bf16*>(a.k_new) + new_off + (int64_t)hk * kD;
    vn = reinterpret_cast<const __bf16*>(a.v_new) + newv_off + (int64_t)hk * kD;
  }
  auto table_row = [&](const void* table, int64_t pos) __attribute__((always_inline)) {
    pos = pos < 0 ? 0 : (pos >= a.table_rows ? a.table_rows - 1 : pos);  // never read outside the table
    return reinterpret_cast<const __bf16*>(table) + pos * kD;
  };
  auto new_rows_issue = [&](int round, const int64_t (&pos)[2]) __attribute__((always_inline)) {
    // every load reads a token that exists (the round's first one stands in where a thread has no
    // task): the loads are then unconditional and the compiler keeps them together
    const int t0 = t_lo + kNewRowsPerRound * round;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int t = rope_k_token(t0, tid, i);
      const bool on = t < t_hi && new_row_in_slab(a.new_col0, t, kv_shift, a.max_len);
      nr.kt[i] = on ? t : -1;
      nr.kc[i] = rope_k_chunk(tid, i);
      const int tl = on ? t : t0;
      nr.x1[i] = *reinterpret_cast<const bf16x8*>(kn + (int64_t)tl * a.kn_st + 8 * nr.kc[i]);
      nr.x2[i] = *reinterpret_cast<const bf16x8*>(kn + (int64_t)tl * a.kn_st + kD / 2 + 8 * nr.kc[i]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int t = rope_v_token(t0, tid, i);
      const bool on = t < t_hi && new_row_in_slab(a.new_col0, t, kv_shift, a.max_len);
      nr.vt[i] = on ? t : -1;
      nr.vc[i] = rope_v_chunk(tid, i);
      nr.vv[i] = *reinterpret_cast<const bf16x8*>(vn + (int64_t)(on ? t : t0) * a.vn_st + 8 * nr.vc[i]);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      // (the position of the thread's own token, or of the array's last one where it has no task)
      const __bf16* cos_row = table_row(a.cos, pos[i]) + 8 * nr.kc[i];
      const __bf16* sin_row = table_row(a.sin, pos[i]) + 8 * nr.kc[i];
      nr.c1[i] = *reinterpret_cast<const bf16x8*>(cos_row); nr.c2[i] = *reinterpret_cast<const bf16x8*>(cos_row + kD / 2);
      nr.s1[i] = *reinterpret_cast<const bf16x8*>(sin_row); nr.s2[i] = *reinterpret_cast<const bf16x8*>(sin_row + kD / 2);
    }
  };
  auto new_rows_finish = [&]() __attribute__((always_inline)) {
    __bf16* kw = const_cast<__bf16*>(kbase);
    __bf16* vw = const_cast<__bf16*>(vbase);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (nr.vt[i] >= 0)
        *reinterpret_cast<bf16x8*>(vw + ((int64_t)a.new_col0 + nr.vt[i]) * a.v_ss + 8 * nr.vc[i]) = nr.vv[i];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      bf16x8 o1, o2;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        o1[e] = static_cast<__bf16>(rope_lo((float)nr.x1[i][e], (float)nr.x2[i][e], (float)nr.c1[i][e], (float)nr.s1[i][e]));
        o2[e] = static_cast<__bf16>(rope_hi((float)nr.x1[i][e], (float)nr.x2[i][e], (float)nr.c2[i][e], (float)nr.s2[i][e]));
      }
      if (nr.kt[i] >= 0) {
        __bf16* dst = kw + ((int64_t)a.new_col0 + nr.kt[i]) * a.k_ss + 8 * nr.kc[i];
        *reinterpret_cast<bf16x8*>(dst) = o1;
        *reinterpret_cast<bf16x8*>(dst + kD / 2) = o2;
      }
    }
  };
  auto new_rows_wait = [&]() __attribute__((always_inline)) { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };

  // Q fragments: B operand of S^T = K Q^T; lane (r,g) holds Q[q_row][16*ks + 8*g .. +8)
  bf16x8 qf[8];
  // (ROPE) the table rows of the query's position: the lane holds dims 16*ks + 8*g + e, so the
  // partner of a first-half dim (ks < 4) sits in fragment ks + 4 of the same lane
  bf16x8 qc[8], qs[8];
  if constexpr (ROPE) {
    if (rows_first) {
      // a short cache: the new rows first, all of them, and a barrier before anybody's tile load
      if (has_new) {
        new_rows_issue(0, pos_a);
        new_rows_finish();
        if (second_round) {
          new_rows_issue(1, pos_b);
          new_rows_finish();
        }
      }
      new_rows_wait();
      __syncthreads();
      fetch_tile(S0{}, 0);
      fetch_tile(S1{}, k_loader ? 1 : 0);
    }
  }
  {
    const __bf16* qp = reinterpret_cast<const __bf16*>(a.q) + rows.q_off +
                       q_frag_offset(h, a.q_sh, row_valid ? q_row : 0, a.q_ss, g, 0);
    // (a lane whose row does not exist takes the batch row's first one: its results are never used,
    // and a load that always happens is one the compiler can keep in flight)
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qp + 16 * ks);
    if constexpr (ROPE) {
      if (has_new && !rows_first) new_rows_issue(0, pos_a);
      const __bf16* cos_row = table_row(a.cos, q_pos) + 8 * g;
      const __bf16* sin_row = table_row(a.sin, q_pos) + 8 * g;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        qc[ks] = *reinterpret_cast<const bf16x8*>(cos_row + 16 * ks);
        qs[ks] = *reinterpret_cast<const bf16x8*>(sin_row + 16 * ks);
      }
    }
  }
  auto rotate_q = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const bf16x8 x1 = qf[ks], x2 = qf[ks + 4];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        qf[ks][e] = static_cast<__bf16>(rope_lo((float)x1[e], (float)x2[e], (float)qc[ks][e], (float)qs[ks][e]));
        qf[ks + 4][e] = static_cast<__bf16>(rope_hi((float)x1[e], (float)x2[e], (float)qc[ks + 4][e], (float)qs[ks + 4][e]));
      }
    }
  };
  const uint64_t* brow = a.bits + mask_word_index(b, a.n_q, row_valid ? q_row : 0, a.words, 0);

  f32x16 o[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
  float m = -INFINITY, l = 0.f;  // m in log2 units (already scaled)
  const float scale_log2 = a.scale * 1.4426950408889634f;

  auto fetch_word = [&](auto slot_c, int j) __attribute__((always_inline)) {
    const int key0 = tile_key0(lo, j, n_tiles);
    // nothing may touch the loaded value here: an operation on it would make the wave wait for
    // this load, and with it for every tile load issued before it, at this point of every step
    wring[decltype(slot_c)::value] = brow[key0 >> 6];
  };
  auto stage_k_from = [&](bf16x8 c0, bf16x8 c1, bf16x8 c2, bf16x8 c3, int j) __attribute__((always_inline)) {
    char* dst = smem + lds_k_stage(ld, j, 0);
    *reinterpret_cast<bf16x8*>(dst) = c0;
    *reinterpret_cast<bf16x8*>(dst + (lds_k_stage(ld, 0, 1) - lds_k_stage(ld, 0, 0))) = c1;
    *reinterpret_cast<bf16x8*>(dst + (lds_k_stage(ld, 0, 2) - lds_k_stage(ld, 0, 0))) = c2;
    *reinterpret_cast<bf16x8*>(dst + (lds_k_stage(ld, 0, 3) - lds_k_stage(ld, 0, 0))) = c3;
  };
  auto stage_k = [&](auto slot_c, int j) __attribute__((always_inline)) {
    if constexpr (decltype(slot_c)::value == 0) stage_k_from(a0, a1, a2, a3, j); else stage_k_from(b0, b1, b2, b3, j);
  };
  auto stage_v_from = [&](bf16x8 c0, bf16x8 c1, bf16x8 c2, bf16x8 c3, int j) __attribute__((always_inline)) {
    char* dst = smem + lds_v_stage(ld, j, 0);
    *reinterpret_cast<bf16x8*>(dst) = c0;
    *reinterpret_cast<bf16x8*>(dst + (lds_v_stage(ld, 0, 1) - lds_v_stage(ld, 0, 0))) = c1;
    *reinterpret_cast<bf16x8*>(dst + (lds_v_stage(ld, 0, 2) - lds_v_stage(ld, 0, 0))) = c2;
    *reinterpret_cast<bf16x8*>(dst + (lds_v_stage(ld, 0, 3) - lds_v_stage(ld, 0, 0))) = c3;
  };
  auto stage_v = [&](auto slot_c, int j) __attribute__((always_inline)) {
    if constexpr (decltype(slot_c)::value == 0) stage_v_from(a0, a1, a2, a3, j); else stage_v_from(b0, b1, b2, b3, j);
  };

  // S^T of one unit: 32 keys x 32 queries; accumulator i is key 8*(i/4) + 4*g + i%4 of the unit.
  // A wave walks through one or two units per tile: both 32-key halves (a full wave) or its own.
  static_assert(kRing % 2 == 0, "the score registers alternate between two sets per unit");
  f32x16 s_reg[2];
  // (lds_k_frag is linear in its arguments: the lane's place in the tile's buffer plus the wave-uniform
  // place of the unit's fragment)
  auto k_lane = [&](int tile) __attribute__((always_inline)) { return smem + lds_k_frag(tile, 0, r, g, 0); };
  auto k_frag = [&](const char* sk, int key_off, int ks) __attribute__((always_inline)) {
    return *reinterpret_cast<const bf16x8*>(sk + lds_k_frag(0, key_off, 0, 0, ks));
  };

  // ---- prologue: K of tiles 0 and 1 and V of tile 0 into LDS, the ring filled behind them --------
  // K runs one tile further ahead than V (K(t+1) is multiplied during step t); both roles keep
  // the tile that step t stages in ring slot (t + 1) % kRing, so that one piece of code, with
  // the same registers, serves both.
  const int ahead = k_loader ? 2 : 1;
  if (k_loader) {  // (requested at the kernel's entry)
    stage_k(S0{}, 0);
    stage_k(S1{}, 1);
  } else {
    stage_v(S0{}, 0);
  }
  if constexpr (ROPE) {
    if (has_new && !rows_first) {
      new_rows_finish();
      if (second_round) new_rows_issue(1, pos_b);
    }
  }
  // The ring is filled in the order in which the steps refill it (mask word, then tile, slot by
  // slot): the loads in flight at the top of the first step are then the same as at the top of
  // every later one, and the compiler's count of them stays exact around the loop.  The mask word
  // of tile j sits in wring[j % kRing] from two steps before its tile until the tile's last unit;
  // it is never copied to another variable (a copy right after the load would be a wait for it).
  rd_static_for<kRing>([&](auto j) __attribute__((always_inline)) {
    constexpr int J = decltype(j)::value;
    fetch_word(std::integral_constant<int, J>{}, J);
    fetch_tile(std::integral_constant<int, (J + 1) % kRing>{}, ahead + J);
  });
  if constexpr (ROPE) {
    // under cover of the ring's first loads: the queries are rotated, a second round of new rows finished
    rotate_q();
    if (has_new && !rows_first && second_round) new_rows_finish();
  }
  __syncthreads();
  // The scores of a unit are masked, and their row maximum taken, as soon as they exist: in the
  // step before the one that turns them into probabilities, under that step's second product
  // (the matrix pipeline is busy there and the vector ALU is not).  tmax: that maximum, in log2
  // units, of the unit whose scores wait in the score registers; here for the first unit.
  // Rows past n_q take an all-ones word: their results are never used.
  auto unit_bits = [&](uint64_t word, int key_off) __attribute__((always_inline)) {  // the unit's 32 keys
    return row_valid ? (uint32_t)(word >> key_off) : ~0u;
  };
  auto masked = [&](float score, uint32_t w, int i) __attribute__((always_inline)) {
    // accumulator i is key 8*(i/4) + 4*g + i%4 of the unit; w: the unit's bits shifted down by 4*g
    return ((w >> (8 * (i >> 2) + (i & 3))) & 1u) ? score : -INFINITY;
  };
  float tmax = -INFINITY;
  if (wave_active) {
#pragma unroll
    for (int i = 0; i < 16; ++i) s_reg[0][i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
      s_reg[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_frag(k_lane(0), kp * 32, ks), qf[ks], s_reg[0], 0, 0, 0);
    const uint32_t w = unit_bits(wring[0], kp * 32) >> (4 * g);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s_reg[0][i] = masked(s_reg[0][i], w, i);
      tmax = fmaxf(tmax, s_reg[0][i]);
    }
    tmax = pair_max(tmax) * scale_log2;
  }

  // ---- one unit per step -----------------------------------------------------------------------
  // A step holds S of its unit in registers.  It multiplies the next unit's K by Q on the matrix
  // pipeline while the vector ALU turns S into P (two scores per MFMA, in source order), then adds
  // V^T P^T; the last step of a tile stages the tiles that later steps need in between.
  // j_c: t % kRing; cur_c: which score register set holds this unit's S; last_c: the tile's last
  // step (staging, fetches and barrier belong to it); run: this wave has a unit in this step
  // (wave-uniform); key_off: the unit's keys within the tile; next_t, next_off: tile and key offset
  // of the unit whose scores this step forms for the wave's next turn.
  auto unit_step = [&](auto j_c, auto cur_c, auto last_c, int t, bool run, int key_off, int next_t,
                       int next_off) __attribute__((always_inline)) {
    constexpr int J = decltype(j_c)::value;
    constexpr int CUR = decltype(cur_c)::value;
    constexpr bool kLast = decltype(last_c)::value;
    f32x16& s_cur = s_reg[CUR];
    f32x16& s_next = s_reg[CUR ^ 1];
    const bool busy = wave_active && run;
    bf16x8 pf[2];  // P^T of the unit, the B operand of the second product
    if (kLast) {
      // This tile's mask word is done with (its last unit was masked in the step before): the word
      // of tile t+kRing takes its slot.  Requested ahead of this step's tile, so that the step that
      // uses it waits for no tile it has not staged.
      fetch_word(std::integral_constant<int, J>{}, t + kRing);
    }
    if (busy) {
      // lazy rescale (the unit's scores were masked and their maximum taken in the wave's previous step)
      // The running maximum only has to bound the exponents, not equal the true maximum: it is
      // raised (and O, l rescaled) only when a unit exceeds it by more than kSlack, so most units
      // skip the 64-register rescale.  p <= 2^kSlack stays far inside bf16/fp32 range.
      constexpr float kSlack = 8.f;
      // (rows without a key so far have m = tmax = -inf: nothing to raise, nothing to rescale)
      const bool raise = tmax > m + kSlack;
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
      // S(next unit) = K Q^T  ||  P = exp2(S * scale - m).  After the last unit the product reads
      // a stale buffer; its result is never used.
      const char* sk = k_lane(next_t);
      float psum = 0.f;
      constexpr int kDepth = 4;  // K fragments in flight from LDS (a read takes longer than two MFMAs)
      bf16x8 ka[kDepth];
#pragma unroll
      for (int d = 0; d < kDepth; ++d) ka[d] = k_frag(sk, next_off, d);
#pragma unroll
      for (int i = 0; i < 16; ++i) s_next[i] = 0.f;
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        s_next = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[q % kDepth], qf[q], s_next, 0, 0, 0);
        if (q + kDepth < 8) ka[q % kDepth] = k_frag(sk, next_off, q + kDepth);
        const int i = 2 * q;
        const float p0 = fast_exp2(fmaf(s_cur[i], scale_log2, -m_use));
        const float p1 = fast_exp2(fmaf(s_cur[i + 1], scale_log2, -m_use));
        psum += p0 + p1;
        const f32x2 pp = {p0, p1};
        const bf16x2 pb = __builtin_convertvector(pp, bf16x2);
        pf[i >> 3][i & 7] = pb[0];
        pf[i >> 3][(i & 7) + 1] = pb[1];
        // the order written here is the order wanted: the vector work of two scores runs while the
        // matrix pipeline works through the MFMA in front of it
        __builtin_amdgcn_sched_barrier(0);
      }
      l += psum;
      // P is used only after the staging branches below: pin it here, or its computation is sunk
      // behind them and out from under the MFMAs
      asm volatile("" : "+v"(pf[0]), "+v"(pf[1]));
    }
    // the first V fragments are requested before the staging code, so that they have arrived when
    // the second product starts
    constexpr int kVDepth = 4;
    bf16x8 va[kVDepth];
    // (lds_v_frag is linear: the lane's own place in the tile's buffer plus the wave-uniform place
    // of the fragment's keys and dims; a fragment is two transposing reads of four keys each)
    typedef __attribute__((address_space(3))) bf16x4 lds_bf16x4;
    typedef __attribute__((address_space(3))) char lds_char;
    lds_char* sv = (lds_char*)smem + lds_v_frag(t, key_off, lane, 0, 0);
    auto v_frag = [&](int c) __attribute__((always_inline)) {
      const bf16x4 first = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
          (lds_bf16x4*)(sv + (lds_v_frag(0, 0, 0, c, 0) - lds_v_frag(0, 0, 0, 0, 0))));
      const bf16x4 second = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
          (lds_bf16x4*)(sv + (lds_v_frag(0, 0, 0, c, 1) - lds_v_frag(0, 0, 0, 0, 0))));
      return __builtin_shufflevector(first, second, 0, 1, 2, 3, 4, 5, 6, 7);
    };
    if (busy) {
#pragma unroll
      for (int c = 0; c < kVDepth; ++c) va[c] = v_frag(c);
    }
    if (kLast) {
      // stage and fetch before the second product: the LDS writes and the V transposes run under it
      using Slot = std::integral_constant<int, (J + 1) % kRing>;
      if (k_loader) stage_k(Slot{}, t + 2); else stage_v(Slot{}, t + 1);
      fetch_tile(Slot{}, t + ahead + kRing);
    }
    if (busy) {
      // O^T += V^T P^T ; k-slot j of lane group g is key 16*tt + 4*g + (j%4) + 8*(j/4) of the unit.
      // Behind each MFMA, two scores of the NEXT unit (complete since the first product above) are
      // folded into that unit's row maximum.  Its mask word has been in the ring since the step
      // before (requested before that step's tile: using it waits for no tile that this step has
      // not already staged).
      uint64_t next_word = wring[(J + 1) % kRing];  // the next unit lies in the next tile ...
      if constexpr (!kLast) next_word = next_t == t ? wring[J] : next_word;  // ... or is this tile's other half
      const uint32_t next_bits = unit_bits(next_word, next_off);
      float next_max = -INFINITY;
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        o[c >> 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[c % kVDepth], pf[c & 1], o[c >> 1], 0, 0, 0);
        if (c + kVDepth < 8) va[c % kVDepth] = v_frag(c + kVDepth);
        next_max = fmaxf(next_max, fmaxf(s_next[2 * c], s_next[2 * c + 1]));
        __builtin_amdgcn_sched_barrier(0);
      }
      // Most units lie in front of the tree, where every key is attended.  The others (the tree's
      // tiles, a tile with left padding) are masked now and their maximum is taken again.
      if (!__all(next_bits == ~0u)) {
        const uint32_t wn = next_bits >> (4 * g);
        next_max = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          s_next[i] = masked(s_next[i], wn, i);
          next_max = fmaxf(next_max, s_next[i]);
        }
      }
      tmax = pair_max(next_max) * scale_log2;
    }
    if (kLast) {
      if constexpr (ROPE) {
        if (t == t_sync) new_rows_wait();  // (uniform) the next step may request a tile with new rows
      }
      __syncthreads();
    }
  };
  // Whole rounds of the ring first, then the odd tile.  A round that could skip its second step
  // would leave two possible sets of loads in flight at the top of the loop, and every wait in
  // the first step would then have to be a wait for all of them.
  // One tile.  A full wave takes both units of the tile, in score sets 0 and 1.  A half wave takes
  // its unit (keys kp*32..) and alternates between the score sets from tile to tile, which is one
  // unit per tile of the two-tile ring round: its turn is the first step of even tiles and the
  // second step of odd ones.  In a layout that has both kinds, both run the same two steps per
  // tile, a half wave idling through the step that is not its turn (wave-uniform branches): two
  // separate loops in one kernel keep the registers of both alive and spill.
  using Yes = std::true_type;
  using No = std::false_type;
  using One = std::integral_constant<int, 1>;
  auto tile_step = [&](auto j, int t) __attribute__((always_inline)) {
    constexpr int J = decltype(j)::value;
    if constexpr (kHasFull && kHasHalf) {
      const int off = kp * 32;  // kp is 0 for a full wave
      unit_step(j, S0{}, No{}, t, full || J == 0, off, full ? t : t + 1, full ? 32 : off);
      unit_step(j, One{}, Yes{}, t, full || J == 1, full ? 32 : off, t + 1, full ? 0 : off);
    } else if constexpr (kHasFull) {
      unit_step(j, S0{}, No{}, t, true, 0, t, 32);
      unit_step(j, One{}, Yes{}, t, true, 32, t + 1, 0);
    } else {
      unit_step(j, std::integral_constant<int, J & 1>{}, Yes{}, t, true, kp * 32, t + 1, kp * 32);
    }
  };
  // Whole rounds of the ring first, then the odd tile.  A round that could skip its second step
  // would leave two possible sets of loads in flight at the top of the loop, and every wait in
  // the first step would then have to be a wait for all of them.
  int t0 = 0;
  for (; t0 + kRing <= n_tiles; t0 += kRing) {
    rd_static_for<kRing>([&](auto j) __attribute__((always_inline)) { tile_step(j, t0 + decltype(j)::value); });
  }
  if (t0 < n_tiles) tile_step(S0{}, t0);

  l = pair_sum(l);
  // accumulator i of block db is d = 32*db + 8*(i/4) + 4*g + i%4
  static_assert(kMergeFloats * 4 <= kLdsBytes, "merge buffer");
  if (kHasHalf) {
    // Merge of the two key parts of every row block through LDS (the tile buffers are free: every
    // wave has passed the loop's last barrier).  The two waves of a pair exchange halves: each hands
    // over the two accumulator blocks it does not keep and its (m, l), and merges the partner's
    // part of the two blocks it keeps -- half the LDS traffic per wave of handing everything to one
    // wave, and both waves normalise and store.  Both evaluate the same expressions on the same
    // operands in the same order (part 0's term first), so they agree on m and l to the bit.
    auto x_o = [&](int acc) __attribute__((always_inline)) -> float& {
      return *reinterpret_cast<float*>(smem + lds_merge_o(role.pair, acc, lane));
    };
    auto x_ml = [&](int part, int which) __attribute__((always_inline)) -> float& {
      return *reinterpret_cast<float*>(smem + lds_merge_ml(role.pair, part, which, lane));
    };
    auto hand_over = [&](auto first_c) __attribute__((always_inline)) {  // the blocks this wave does not keep
      constexpr int kFirst = decltype(first_c)::value;
#pragma unroll
      for (int db = kFirst; db < kFirst + 2; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) x_o(16 * db + i) = o[db][i];
    };
    auto take_over = [&](auto first_c, float a0, float a1) __attribute__((always_inline)) {  // the blocks it keeps
      constexpr int kFirst = decltype(first_c)::value;
#pragma unroll
      for (int db = kFirst; db < kFirst + 2; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float theirs = x_o(16 * db + i);
          // (part 0's term first, whoever computes it)
          o[db][i] = kFirst == 0 ? a0 * o[db][i] + a1 * theirs : a0 * theirs + a1 * o[db][i];
        }
    };
    const bool half = !full && wave_active;  // (wave-uniform)
    if (half) {
      if (kp == 0) hand_over(std::integral_constant<int, 2>{}); else hand_over(std::integral_constant<int, 0>{});
      x_ml(kp, 0) = m;
      x_ml(kp, 1) = l;
    }
    __syncthreads();
    if (half) {
      const float m0 = kp == 0 ? m : x_ml(0, 0), l0 = kp == 0 ? l : x_ml(0, 1);
      const float m1 = kp == 1 ? m : x_ml(1, 0), l1 = kp == 1 ? l : x_ml(1, 1);
      const float m_new = fmaxf(m0, m1);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      const float a0 = fast_exp2(m0 - m_safe), a1 = fast_exp2(m1 - m_safe);  // exp2(-inf) = 0
      {
#pragma clang fp contract(off)
        l = a0 * l0 + a1 * l1;
      }
      if (kp == 0) take_over(std::integral_constant<int, 0>{}, a0, a1); else take_over(std::integral_constant<int, 2>{}, a0, a1);
      m = m_new;
    }
  }
  const bool writer = wave_active && row_valid;
  // What a wave writes: the accumulator blocks it keeps (attn_addr.h: first_block_kept,
  // blocks_kept), named at compile time in each of the three cases (a block index that is only
  // known at run time would put the accumulators into scratch memory).
  using B0 = std::integral_constant<int, 0>;
  using B1 = std::integral_constant<int, 1>;
  using B2 = std::integral_constant<int, 2>;
  using B3 = std::integral_constant<int, 3>;
#define RD_FOR_KEPT_BLOCKS(body)                                         \
  do {                                                                   \
    if (full || !kHasHalf) { body(B0{}); body(B1{}); body(B2{}); body(B3{}); } \
    else if (kp == 0) { body(B0{}); body(B1{}); }                        \
    else { body(B2{}); body(B3{}); }                                     \
  } while (0)
  if (n_splits == 1) {
    // The rows leave through LDS (attn_addr.h: lds_out_stage): in the accumulators a lane holds
    // four dims of one row, and stored from there an instruction would touch 32 rows with 16 bytes
    // each -- 32 requests to the L2 where, read back along the rows, two or four whole rows go out.
    // Each wave uses a region of its own and needs no barrier for it (the tile buffers are free:
    // every wave has passed the loop's last barrier; where accumulators were merged through LDS, the
    // merge buffers must have been read first).
    if constexpr (kHasHalf) __syncthreads();
    if (!wave_active) return;  // (wave-uniform)
    const bool live = l > 0.f;
    const float inv = live ? 1.f / l : 0.f;
    char* const mine = smem + lds_out_stage(wave, r, g, 0, 0);
    auto stage_block = [&](auto db_c) __attribute__((always_inline)) {
      constexpr int db = decltype(db_c)::value;
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        // (a row without any attended key gets zeros, whatever its accumulators picked up)
        bf16x4 w = {static_cast<__bf16>(live ? o[db][4 * i4 + 0] * inv : 0.f), static_cast<__bf16>(live ? o[db][4 * i4 + 1] * inv : 0.f),
                    static_cast<__bf16>(live ? o[db][4 * i4 + 2] * inv : 0.f), static_cast<__bf16>(live ? o[db][4 * i4 + 3] * inv : 0.f)};
        *reinterpret_cast<bf16x4*>(mine + lds_out_stage(0, 0, 0, db, i4)) = w;
      }
    };
    RD_FOR_KEPT_BLOCKS(stage_block);
    // (the wave reads what its own lanes wrote: its LDS instructions execute in program order)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __bf16* const orow = reinterpret_cast<__bf16*>(a.out) + rows.o_off;
    auto store_rows = [&](auto first_c, auto blocks_c) __attribute__((always_inline)) {
      constexpr int kFirst = decltype(first_c)::value, kBlocks = decltype(blocks_c)::value;
#pragma unroll
      for (int pass = 0; pass < out_passes(kBlocks); ++pass) {
        const int row = out_piece_row(kBlocks, pass, lane), dim = out_piece_dim(kFirst, kBlocks, pass, lane);
        const bf16x4 w = *reinterpret_cast<const bf16x4*>(smem + lds_out_piece(wave, row, dim));
        const int q = q_row_of(q_tile, kRowsPerWG, row_wave, row);
        if (q < rows.n) *reinterpret_cast<bf16x4*>(orow + out_row_offset(h, a.o_sh, q, a.o_ss, dim)) = w;
      }
    };
    using Two = std::integral_constant<int, 2>;
    using Four = std::integral_constant<int, 4>;
    if (full || !kHasHalf) store_rows(B0{}, Four{});
    else if (kp == 0) store_rows(B0{}, Two{});
    else store_rows(B2{}, Two{});
    return;
  }
  // The keys of this batch row are split over n_splits work items: each leaves (m, l, O) of its
  // key range as fp32 partials, counts itself in, and the last one to arrive merges the partials
  // of all of them (m in log2 units).  Nobody returns before the count: the barriers below are
  // reached by every wave of the workgroup.
  // The partials cross from one XCD to another, whose L2s do not see each other's lines.  They are
  // therefore stored and loaded with device-scope accesses (the sc1 bit: the store goes through
  // this XCD's L2 to memory, the load does not take a line another XCD may have changed from its
  // own L2), 16 bytes at a time.  A release fence before the count and an acquire fence behind it
  // would do the same for ordinary accesses, but each works on the whole L2 of its XCD while the
  // other workgroups stream through it: rows split four ways ran 8-19 % longer that way.
  if (writer) {
    float* po = a.part_o + partial_row(b, a.H, h, a.max_splits, split, a.n_q, q_row) * kD + 4 * g;
    auto store_partial = [&](auto db_c) __attribute__((always_inline)) {
      constexpr int db = decltype(db_c)::value;
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const f32x4 w = {o[db][4 * i4 + 0], o[db][4 * i4 + 1], o[db][4 * i4 + 2], o[db][4 * i4 + 3]};
        float* const dst = po + 32 * db + 8 * i4;  // (a local: an asm operand cannot name a captured variable here)
        asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(dst), "v"(w) : "memory");
      }
    };
    RD_FOR_KEPT_BLOCKS(store_partial);
    if (g == 0 && (full || kp == 0)) {  // (both waves of a pair hold the same m and l)
      float* pm = a.part_ml + partial_row(b, a.H, h, a.max_splits, split, a.n_q, q_row) * 2;
      const f32x2 ml = {m, l};
      asm volatile("global_store_dwordx2 %0, %1, off sc1" ::"v"(pm), "v"(ml) : "memory");
    }
  }
  // Every wave waits until its stores have arrived, the barrier collects the waves, and one lane
  // counts the item in: whoever reads n_splits - 1 there knows that the partials of all the others
  // are in memory.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  int* s_last = reinterpret_cast<int*>(smem);  // (the tile buffers are free by now)
  unsigned int* counter = a.counters + counter_index(b, a.H, h, q_tiles, q_tile);
  if (wave == 0) {
    int last = 0;
    if (lane == 0) last = atomicAdd(counter, 1u) == (unsigned int)(n_splits - 1);
    last = __builtin_amdgcn_readfirstlane(last);
    if (lane == 0) *s_last = last;
  }
  __syncthreads();
  if (*s_last == 0) return;
  // 16 row groups x 32 lanes of four dims; eight rows per pass and thread, so that the loads of
  // a pass (two per row and split) are in flight together: the merge is bound by their latency
  const int q_end = (q_tile + 1) * kRowsPerWG < rows.n ? (q_tile + 1) * kRowsPerWG : rows.n;
  constexpr int kGroups = kMfmaThreads / 32, kPass = 8;
  const int rg = tid >> 5, dq = (tid & 31) * 4;
  for (int q0 = q_tile * kRowsPerWG + rg; q0 < q_end; q0 += kGroups * kPass) {
    float mx[kPass], ls[kPass];
    f32x4 acc[kPass];
#pragma unroll
    for (int j = 0; j < kPass; ++j) {
      mx[j] = -INFINITY; ls[j] = 0.f; acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    for (int s = 0; s < n_splits; ++s) {
      f32x2 ml[kPass];
      f32x4 po[kPass];
#pragma unroll
      for (int j = 0; j < kPass; ++j) {
        const int q = q0 + kGroups * j < q_end ? q0 + kGroups * j : q_end - 1;  // clamped: loads stay unconditional
        const int64_t row = partial_row(b, a.H, h, a.max_splits, s, a.n_q, q);
        asm volatile("global_load_dwordx2 %0, %1, off sc1" : "=v"(ml[j]) : "v"(a.part_ml + row * 2) : "memory");
        asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(po[j]) : "v"(a.part_o + row * kD + dq) : "memory");
      }
      // (the compiler does not count these loads: one wait for all of them, and every destination
      // register is an operand of that wait, so that none of them can be copied, spilled or read
      // between its load and the wait)
      static_assert(kPass == 8, "the wait below names eight register pairs and eight quads");
      asm volatile("s_waitcnt vmcnt(0)"
                   : "+v"(ml[0]), "+v"(ml[1]), "+v"(ml[2]), "+v"(ml[3]), "+v"(ml[4]), "+v"(ml[5]), "+v"(ml[6]), "+v"(ml[7]),
                     "+v"(po[0]), "+v"(po[1]), "+v"(po[2]), "+v"(po[3]), "+v"(po[4]), "+v"(po[5]), "+v"(po[6]), "+v"(po[7])
                   :
                   : "memory");
#pragma unroll
      for (int j = 0; j < kPass; ++j) {
        const float m_new = fmaxf(mx[j], ml[j][0]);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float a1 = fast_exp2(mx[j] - m_safe), a2 = fast_exp2(ml[j][0] - m_safe);  // exp2(-inf) = 0
        ls[j] = a1 * ls[j] + a2 * ml[j][1];
        acc[j] = a1 * acc[j] + a2 * po[j];
        mx[j] = m_new;
      }
    }
#pragma unroll
    for (int j = 0; j < kPass; ++j) {
      const int q = q0 + kGroups * j;
      if (q < q_end) {
        const bool live = ls[j] > 0.f;
        const float inv = live ? 1.f / ls[j] : 0.f;
        __bf16* op = reinterpret_cast<__bf16*>(a.out) + rows.o_off + out_offset(h, a.o_sh, q, a.o_ss, 0, 0, 0) + dq;
        bf16x4 w = {static_cast<__bf16>(live ? acc[j][0] * inv : 0.f), static_cast<__bf16>(live ? acc[j][1] * inv : 0.f),
                    static_cast<__bf16>(live ? acc[j][2] * inv : 0.f), static_cast<__bf16>(live ? acc[j][3] * inv : 0.f)};
        *reinterpret_cast<bf16x4*>(op) = w;
      }
    }
  }
  // zero again: for the launch that gets this part of the ring next, and for this one's replay by a graph
  if (tid == 0) *counter = 0u;
#undef RD_FOR_KEPT_BLOCKS
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
  const RowSpan rows = row_span(a, b);
  if (q >= rows.n) return;
  const T* qp = reinterpret_cast<const T*>(a.q) + rows.q_off + (int64_t)h * a.q_sh + (int64_t)q * a.q_ss;
  const int kv_shift = a.plan[RD_PLAN_HDR + 4 * b + 3];
  const T* kb = reinterpret_cast<const T*>(a.k) + (int64_t)b * a.k_sb + (int64_t)hk * a.k_sh - (int64_t)kv_shift * a.k_ss;
  const T* vb = reinterpret_cast<const T*>(a.v) + (int64_t)b * a.v_sb + (int64_t)hk * a.v_sh - (int64_t)kv_shift * a.v_ss;
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
    T* op = reinterpret_cast<T*>(a.out) + rows.o_off + (int64_t)h * a.o_sh + (int64_t)q * a.o_ss;
    st<T>(op + tid, l > 0.f ? acc / l : 0.f);
  }
}

}  // namespace

// Arrival counters of split rows.  Zero when the library is loaded; the item that merges a row puts
// the row's counter back to zero.  Every launch takes the next slab of the ring, so two launches
// that are in flight together (on two streams, on one plan or not) count on different counters
// unless a whole ring's worth of launches (2^18 counters) was enqueued between them.
constexpr int kArrivalRing = 1 << 18;
static __device__ unsigned int attn_arrivals[kArrivalRing];

namespace {

constexpr int kMaxDevices = 64;
// `n` counters of the current device's ring; nullptr with a message on failure
unsigned int* arrival_slab(const char* who, size_t n, int* error) {
  static std::mutex mu;
  static unsigned int* base[kMaxDevices] = {nullptr};
  static size_t next[kMaxDevices] = {0};
  if (n > (size_t)kArrivalRing) {
    *error = rd::fail(RD_ELIMIT, "%s: batch x heads x query tiles = %zu arrival counters (at most %d)", who, n, kArrivalRing);
    return nullptr;
  }
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    *error = rd::fail(RD_ELAUNCH, "%s: no current device (or an ordinal above %d)", who, kMaxDevices - 1);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (base[dev] == nullptr) {
    // (the array's name is a host-side stand-in: its address on this GPU is asked for once)
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(attn_arrivals));
    if (e != hipSuccess || p == nullptr) {
      *error = rd::fail(RD_ELAUNCH, "%s: hipGetSymbolAddress: %s", who, hipGetErrorString(e));
      return nullptr;
    }
    base[dev] = reinterpret_cast<unsigned int*>(p);
  }
  if (next[dev] + n > (size_t)kArrivalRing) next[dev] = 0;
  unsigned int* slab = base[dev] + next[dev];
  next[dev] += n;
  return slab;
}

bool mfma_eligible(const AttnArgs& a, int dtype) {
  auto al = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
  auto m8 = [](int64_t s) { return (s % 8) == 0; };
  // (the tile loads address a row's keys with 32-bit byte offsets)
  if (a.k_ss <= 0 || a.v_ss <= 0 || !span_fits(a.kv_len, a.k_ss * 2) || !span_fits(a.kv_len, a.v_ss * 2)) return false;
  return dtype == RD_BF16 && a.D == kD && a.H <= rd::kAttnMaxHeads && al(a.q) && al(a.k) && al(a.v) && ((uintptr_t)a.out & 7) == 0 &&
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

namespace {

// The new keys and values of a fused call (null: the cache already holds them).
struct RopeInputs {
  const void* k_new; const int64_t* k_new_strides;
  const void* v_new; const int64_t* v_new_strides;
  const void* cos; const void* sin; int64_t table_rows;
  const int64_t* position_ids; int64_t pos_batch_stride;
  int64_t max_len;
};

int verify_attention(const char* who, const void* q, const int64_t* q_strides, const void* k,
                     const int64_t* k_strides, const void* v, const int64_t* v_strides, void* out,
                     const int64_t* o_strides, int dtype, int batch, int n_heads, int n_kv_heads, int n_q,
                     int kv_len, int head_dim, float scale, const uint64_t* bits, const int32_t* plan,
                     void* workspace, size_t workspace_bytes, int force_generic, const int32_t* row_start,
                     const RopeInputs* rope, void* stream) {
  RD_REQUIRE(batch > 0 && n_heads > 0 && n_kv_heads > 0 && n_q > 0 && kv_len > 0 && head_dim > 0,
             RD_EINVAL, "%s: bad sizes (batch %d heads %d kv_heads %d n_q %d kv %d D %d)", who,
             batch, n_heads, n_kv_heads, n_q, kv_len, head_dim);
  RD_REQUIRE(n_heads % n_kv_heads == 0, RD_EINVAL, "%s: heads %d not a multiple of kv heads %d", who,
             n_heads, n_kv_heads);
  RD_REQUIRE(head_dim <= 256, RD_ELIMIT, "%s: head_dim %d > 256", who, head_dim);
  RD_REQUIRE(batch <= 65535 && n_heads <= 65535, RD_ELIMIT, "%s: batch/heads > 65535", who);
  // what the MFMA kernel's launch would need of the ring of arrival counters (asked of every bf16
  // call of its head size, before any pointer is looked at)
  RD_REQUIRE(dtype != RD_BF16 || head_dim != kD || n_heads > rd::kAttnMaxHeads || force_generic ||
                 rd::attn_counter_ints(batch, n_heads, n_q) <= (size_t)kArrivalRing,
             RD_ELIMIT, "%s: batch x heads x query tiles = %zu arrival counters (at most %d)", who,
             rd::attn_counter_ints(batch, n_heads, n_q), kArrivalRing);
  RD_REQUIRE(q && k && v && out && bits && plan && q_strides && k_strides && v_strides && o_strides,
             RD_EINVAL, "%s: null pointer", who);
  RD_REQUIRE(dtype == RD_BF16 || dtype == RD_F16 || dtype == RD_F32, RD_EINVAL, "%s: unknown dtype %d", who, dtype);
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
  a.row_start = row_start;
  a.counters = nullptr;
  a.k_new = a.v_new = a.cos = a.sin = nullptr;
  a.kn_sb = a.kn_st = a.vn_sb = a.vn_st = a.table_rows = a.pos_sb = a.max_len = 0;
  a.position_ids = nullptr; a.new_col0 = kv_len;
  hipStream_t s = rd::as_stream(stream);

  const bool mfma = !force_generic && mfma_eligible(a, dtype);
  if (rope != nullptr) {
    auto al = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
    RD_REQUIRE(mfma && n_q <= rows_per_wg(kFull), RD_ELIMIT, "%s: only bf16, head_dim %d, n_q <= %d, 16-byte aligned "
               "operands (use rd_rope_append and rd_verify_attention)", who, kD, rows_per_wg(kFull));
    RD_REQUIRE(rope->k_new && rope->v_new && rope->cos && rope->sin && rope->position_ids && rope->k_new_strides &&
                   rope->v_new_strides, RD_EINVAL, "%s: null pointer", who);
    RD_REQUIRE(al(rope->k_new) && al(rope->v_new) && al(rope->cos) && al(rope->sin), RD_EINVAL,
               "%s: pointers must be 16-byte aligned", who);
    RD_REQUIRE(rope->table_rows > 0, RD_EINVAL, "%s: empty cos/sin table", who);
    RD_REQUIRE(kv_len >= n_q && kv_len <= rope->max_len, RD_EINVAL, "%s: kv_len %d must lie in [n_q %d, max_len %lld]",
               who, kv_len, n_q, (long long)rope->max_len);
    for (const int64_t* st : {rope->k_new_strides, rope->v_new_strides})
      RD_REQUIRE(st[0] % 8 == 0 && st[1] % 8 == 0 && st[0] >= 0 && st[1] >= (int64_t)n_kv_heads * kD, RD_EINVAL,
                 "%s: token and batch strides of the new keys and values must be multiples of 8 elements, "
                 "tokens at least kv_heads * head_dim apart", who);
    a.k_new = rope->k_new; a.kn_sb = rope->k_new_strides[0]; a.kn_st = rope->k_new_strides[1];
    a.v_new = rope->v_new; a.vn_sb = rope->v_new_strides[0]; a.vn_st = rope->v_new_strides[1];
    a.cos = rope->cos; a.sin = rope->sin; a.table_rows = rope->table_rows;
    a.position_ids = rope->position_ids; a.pos_sb = rope->pos_batch_stride;
    a.new_col0 = kv_len - n_q;
    a.max_len = rope->max_len;
  }

  if (mfma) {
    const size_t need = rd_attention_workspace_bytes(batch, n_heads, n_q, kv_len, head_dim);
    RD_REQUIRE(workspace && workspace_bytes >= need, RD_EWORKSPACE, "%s: workspace %zu < %zu bytes", who,
               workspace_bytes, need);
    RD_REQUIRE(((uintptr_t)workspace & 255) == 0, RD_EINVAL, "%s: workspace not 256B aligned", who);
    const size_t slots = (size_t)batch * n_heads * a.max_splits;
    a.part_o = reinterpret_cast<float*>(workspace);
    a.part_ml = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) +
                                         rd::align_up(slots * n_q * head_dim * sizeof(float), 256));
    const int max_items = batch * a.max_splits;
    const int layout = layout_for(n_q);
    const int q_tiles = (n_q + rows_per_wg(layout) - 1) / rows_per_wg(layout);
    RD_REQUIRE(max_items <= 65535 && (int64_t)q_tiles * n_heads <= 2147483647LL, RD_ELIMIT, "%s: grid too large", who);
    int slab_error = RD_OK;
    a.counters = arrival_slab(who, rd::attn_counter_ints(batch, n_heads, n_q), &slab_error);
    if (a.counters == nullptr) return slab_error;
    {
      // when timed, the events carry the kernel's own begin and end (what a kernel trace reports)
      hipEvent_t t0, t1;
      rd::timing_events("attn_mfma_kernel", &t0, &t1);
      const dim3 grid(n_heads * q_tiles, max_items), block(kMfmaThreads);
      auto launch = [&](auto layout_c) {
        constexpr int L = decltype(layout_c)::value;
        if (rope) hipExtLaunchKernelGGL((attn_mfma_kernel<L, true>), grid, block, 0, s, t0, t1, 0, a);
        else hipExtLaunchKernelGGL((attn_mfma_kernel<L, false>), grid, block, 0, s, t0, t1, 0, a);
      };
      switch (layout) {
        case kSplit: launch(std::integral_constant<int, kSplit>{}); break;
        case kMix5: launch(std::integral_constant<int, kMix5>{}); break;
        case kMix6: launch(std::integral_constant<int, kMix6>{}); break;
        default: launch(std::integral_constant<int, kFull>{}); break;
      }
    }
    return rd::check_launch(who);
  }
  const dim3 grid(n_q, n_heads, batch);
  switch (dtype) {
    case RD_BF16: { rd::ScopedTiming rd_t("attn_generic_kernel", s); hipLaunchKernelGGL(attn_generic_kernel<__hip_bfloat16>, grid, dim3(kGenThreads), 0, s, a); } break;
    case RD_F16: { rd::ScopedTiming rd_t("attn_generic_kernel", s); hipLaunchKernelGGL(attn_generic_kernel<__half>, grid, dim3(kGenThreads), 0, s, a); } break;
    default: { rd::ScopedTiming rd_t("attn_generic_kernel", s); hipLaunchKernelGGL(attn_generic_kernel<float>, grid, dim3(kGenThreads), 0, s, a); } break;
  }
  return rd::check_launch(who);
}

}  // namespace

extern "C" int rd_verify_attention(const void* q, const int64_t* q_strides, const void* k,
                                   const int64_t* k_strides, const void* v,
                                   const int64_t* v_strides, void* out, const int64_t* o_strides,
                                   int dtype, int batch, int n_heads, int n_kv_heads, int n_q,
                                   int kv_len, int head_dim, float scale, const uint64_t* bits,
                                   const int32_t* plan, void* workspace, size_t workspace_bytes,
                                   int force_generic, const int32_t* row_start, void* stream) {
  return verify_attention("rd_verify_attention", q, q_strides, k, k_strides, v, v_strides, out, o_strides, dtype,
                          batch, n_heads, n_kv_heads, n_q, kv_len, head_dim, scale, bits, plan, workspace,
                          workspace_bytes, force_generic, row_start, nullptr, stream);
}

extern "C" int rd_rope_verify_attention_eligible(int dtype, int n_heads, int head_dim, int n_q) {
  return dtype == RD_BF16 && head_dim == kD && n_heads <= rd::kAttnMaxHeads && n_q > 0 && n_q <= rows_per_wg(kFull);
}

extern "C" int rd_rope_verify_attention(const void* q, const int64_t* q_strides, const void* k_new,
                                        const int64_t* k_new_strides, const void* v_new,
                                        const int64_t* v_new_strides, const void* cos, const void* sin,
                                        int64_t table_rows, const int64_t* position_ids,
                                        int64_t pos_batch_stride, void* k_cache, void* v_cache,
                                        const int64_t* cache_strides, int64_t max_len, void* out,
                                        const int64_t* o_strides, int dtype, int batch, int n_heads,
                                        int n_kv_heads, int n_q, int kv_len, int head_dim, float scale,
                                        const uint64_t* bits, const int32_t* plan, void* workspace,
                                        size_t workspace_bytes, const int32_t* row_start, void* stream) {
  const RopeInputs rope{k_new, k_new_strides, v_new, v_new_strides, cos, sin, table_rows, position_ids,
                        pos_batch_stride, max_len};
  return verify_attention("rd_rope_verify_attention", q, q_strides, k_cache, cache_strides, v_cache, cache_strides,
                          out, o_strides, dtype, batch, n_heads, n_kv_heads, n_q, kv_len, head_dim, scale, bits,
                          plan, workspace, workspace_bytes, 0, row_start, &rope, stream);
}
