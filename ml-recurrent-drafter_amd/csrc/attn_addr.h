// Index arithmetic of attn_mfma_kernel: which wave owns which query rows and keys, which thread
// loads which 16-byte chunk of a K or V tile, where tiles, fragments and partial results live in
// LDS and in the workspace.  Plain integer functions that compile for the device and for the host:
// the kernel computes its addresses with them, and a host program can walk over every (workgroup,
// thread, tile) of a launch and hold every address against the extent of the tensor it falls into
// before the kernel ever runs on a GPU.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define RD_HD __host__ __device__ inline __attribute__((always_inline))
#else
#define RD_HD inline
#endif

namespace rd {
namespace attn {

constexpr int kD = 128;                    // head_dim of the MFMA kernel
constexpr int kTile = 64;                  // keys per tile
constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;      // 512
constexpr int kKBuffers = 3;               // K tiles in LDS: K(t+1) is multiplied while K(t+2) is staged
constexpr int kVBuffers = 2;               // V tiles in LDS: V(t) is multiplied while V(t+1) is staged
constexpr int kRing = 2;                   // register stages of tiles on their way from memory
constexpr int kKsStride = kD + 8;          // bf16 elements; 272-byte rows spread 16 lanes over all banks
constexpr int kVtStride = kTile + 8;       // bf16 elements; 144-byte rows: 16-byte aligned, conflict-free
constexpr int kKBytes = kKBuffers * kTile * kKsStride * 2;
constexpr int kVBytes = kVBuffers * kD * kVtStride * 2;
constexpr int kLdsBytes = kKBytes + kVBytes;

// How the 8 waves of a workgroup share its query rows (blocks of 32) and the 64 keys of a tile.
// A wave is either FULL (it takes both 32-key units of every tile for its row block) or a HALF (it
// takes one unit; two halves share a row block, each with its own running maximum, sum and
// accumulators, merged through LDS at the end).  Wave w runs on SIMD w % 4, so the layouts spread
// the units of a tile evenly over the SIMDs:
//   kSplit  <= 128 rows  4 blocks, all halves (w, w+4)                      2 units per SIMD
//   kMix5   <= 160 rows  blocks 0,1 full (w0,w1); 2,3,4 halves (w2+w6, w3+w7, w4+w5)   3,3,2,2
//   kMix6   <= 192 rows  blocks 0-3 full (w0-w3); 4,5 halves (w4+w5, w6+w7)            3 each
//   kFull   <= 256 rows  8 blocks, all full                                 4 units per SIMD
// Without halves, a workgroup with few rows would leave waves idle and let the others serialise
// their MFMA and softmax phases alone on their SIMDs.
enum Layout { kSplit = 0, kMix5 = 1, kMix6 = 2, kFull = 3 };
constexpr int rows_per_wg(int layout) { return layout == kSplit ? 128 : layout == kMix5 ? 160 : layout == kMix6 ? 192 : 256; }
constexpr int layout_for(int n_q) { return n_q <= 128 ? kSplit : n_q <= 160 ? kMix5 : n_q <= 192 ? kMix6 : kFull; }
struct WaveRole { int block, part, pair; };  // part: 0/1 = that half of the keys, 2 = full; pair: merge slot of a half
RD_HD WaveRole wave_role(int layout, int w) {
  switch (layout) {
    case kSplit: return {w & 3, w >> 2, w & 3};
    case kMix5: {
      if (w < 2) return {w, 2, 0};
      if (w == 2 || w == 6) return {2, w == 6, 0};
      if (w == 3 || w == 7) return {3, w == 7, 1};
      return {4, w == 5, 2};
    }
    case kMix6: return w < 4 ? WaveRole{w, 2, 0} : WaveRole{4 + ((w - 4) >> 1), (w - 4) & 1, (w - 4) >> 1};
    default: return {w, 2, 0};
  }
}

// ---- tile loads ------------------------------------------------------------------------------
// Threads [0,256) stage K rows (keys lrow + 16*i), threads [256,512) stage V transposed (keys
// 4*lrow + i); four 16-byte chunks each per tile.  The V threads map lanes to (chunk, key quad) so
// that the 16 lanes of one LDS write cycle hit 16 different bank pairs: lane bits 0-1 and 4-5
// select the chunk, bits 2-3 and 6-7 the key quad.
struct Loader {
  bool k_loader;
  int chunk;      // 16-byte column chunk of a row (0..15)
  int lrow;       // 0..15
  int key_step;   // this thread's keys within a tile: first_key + i * key_step, i = 0..3
  int first_key;
};
RD_HD Loader loader_of(int tid) {
  Loader ld;
  ld.k_loader = tid < kThreads / 2;
  const int lt = tid & 255;
  ld.chunk = ld.k_loader ? (lt & 15) : ((lt & 3) | (((lt >> 4) & 3) << 2));
  ld.lrow = ld.k_loader ? (lt >> 4) : (((lt >> 2) & 3) | ((lt >> 6) << 2));
  ld.key_step = ld.k_loader ? 16 : 1;
  ld.first_key = ld.k_loader ? ld.lrow : 4 * ld.lrow;
  return ld;
}
RD_HD int n_tiles_of(int lo, int hi) { return (hi - lo + kTile - 1) / kTile; }
// first key of tile j of an item; tile indices past the end repeat the last tile (the loads of the
// pipeline's tail are issued like all the others and never used)
RD_HD int tile_key0(int lo, int j, int n_tiles) { return lo + (j < n_tiles ? j : n_tiles - 1) * kTile; }
// a tile that leaves the span [key_min, key_end) of the keys somebody attends to
RD_HD bool tile_leaves_span(int key0, int key_min, int key_end) { return key0 + kTile > key_end || key0 < key_min; }
// the key whose cache row stands in for `key`: keys in front of the row's first attended key (left
// padding) re-read that key, keys behind its last attended key (tree slots that do not exist, the
// end of the cache) re-read that one
RD_HD int key_in_span(int key, int key_min, int key_end) { return key < key_end ? (key > key_min ? key : key_min) : key_end - 1; }
// key column read by chunk i (0..3) of a loader thread for the tile at key0
RD_HD int tile_chunk_key(const Loader& ld, int key0, int i, int key_min, int key_end) {
  const int key = key0 + ld.first_key + i * ld.key_step;
  return tile_leaves_span(key0, key_min, key_end) ? key_in_span(key, key_min, key_end) : key;
}

// ---- LDS -------------------------------------------------------------------------------------
// byte offsets from the start of the workgroup's LDS; K buffers first, then the V^T buffers
RD_HD int lds_k_stage(const Loader& ld, int j, int i) {  // chunk i of the K tile j
  return ((j % kKBuffers) * kTile * kKsStride + (ld.lrow + 16 * i) * kKsStride + 8 * ld.chunk) * 2;
}
// V^T rows hold the keys of every 16-key group in the order [0-3, 8-11, 4-7, 12-15]: the eight
// keys that one lane feeds to a 16-key MFMA step are then 16 contiguous bytes.
RD_HD int vt_col(int lrow) { return 16 * (lrow >> 2) + 4 * (((lrow & 1) << 1) | ((lrow >> 1) & 1)); }
RD_HD int lds_v_stage(const Loader& ld, int j, int e) {  // the four keys of element e (0..7) of the thread's chunk
  return kKBytes + ((j % kVBuffers) * kD * kVtStride + (8 * ld.chunk + e) * kVtStride + vt_col(ld.lrow)) * 2;
}
// K fragment ks (0..7) of lane (r, g) for the unit at key_off (0 or 32) of tile j: 8 elements
RD_HD int lds_k_frag(int j, int key_off, int r, int g, int ks) {
  return ((j % kKBuffers) * kTile * kKsStride + (key_off + r) * kKsStride + 16 * ks + 8 * g) * 2;
}
// V^T fragment c (0..7) of lane (r, g) for the unit at key_off of tile j: 8 elements
RD_HD int lds_v_frag(int j, int key_off, int r, int g, int c) {
  return kKBytes + ((j % kVBuffers) * kD * kVtStride + (32 * (c >> 1) + r) * kVtStride + 16 * (c & 1) + key_off + 8 * g) * 2;
}
// merge of the two key halves of a row block after the loop: [pair][64 accumulators][lane] floats,
// then [pair][2][lane]
constexpr int kMergeFloats = (kWaves / 2) * (64 * 64 + 2 * 64);
RD_HD int lds_merge_o(int pair, int acc, int lane) { return ((pair * 64 + acc) * 64 + lane) * 4; }
RD_HD int lds_merge_ml(int pair, int which, int lane) { return ((kWaves / 2) * 64 * 64 + (pair * 2 + which) * 64 + lane) * 4; }

// ---- query rows, outputs, mask words ---------------------------------------------------------
RD_HD int q_row_of(int q_tile, int rows_per_workgroup, int row_block, int r) { return q_tile * rows_per_workgroup + row_block * 32 + r; }
// element offset of Q fragment ks of lane (r, g) from the first row of the batch row
RD_HD int64_t q_frag_offset(int h, int64_t q_sh, int q_row, int64_t q_ss, int g, int ks) {
  return (int64_t)h * q_sh + (int64_t)q_row * q_ss + 8 * g + 16 * ks;
}
// element offset of the four outputs (block db, group i4) of lane (r, g): d = 32*db + 8*i4 + 4*g ..
RD_HD int64_t out_offset(int h, int64_t o_sh, int q_row, int64_t o_ss, int g, int db, int i4) {
  return (int64_t)h * o_sh + (int64_t)q_row * o_ss + 4 * g + 32 * db + 8 * i4;
}
RD_HD int64_t mask_word_index(int b, int n_q, int q_row, int words, int key0) {
  return ((int64_t)b * n_q + q_row) * words + (key0 >> 6);
}

// ---- partial results of split rows and their arrival counters --------------------------------
RD_HD int64_t partial_row(int b, int H, int h, int max_splits, int split, int n_q, int q_row) {
  return ((((int64_t)b * H + h) * max_splits) + split) * n_q + q_row;
}
RD_HD int64_t counter_index(int b, int max_heads, int h, int q_tiles, int q_tile) {
  return ((int64_t)b * max_heads + h) * q_tiles + q_tile;
}


// ---- new cache rows of the fused rotation + append (the ROPE instantiation) --------------------
// The item [lo, hi) of a row whose new tokens sit at key columns [new_col0, new_col0 + rows_n)
// writes the tokens [t_lo, t_hi) of them: its own share of those columns, and, if it ends the
// row's key span, everything behind the span too (rows nobody attends to reach the cache as well).
struct NewRows { int t_lo, t_hi; };
RD_HD NewRows new_rows_of_item(int lo, int hi, int key_end, int new_col0, int rows_n) {
  const bool writes = hi > new_col0 || hi >= key_end;
  NewRows nr;
  nr.t_lo = lo > new_col0 ? lo - new_col0 : 0;
  nr.t_hi = !writes ? 0 : (hi >= key_end || hi - new_col0 > rows_n ? rows_n : hi - new_col0);
  return nr;
}
// A round covers 128 tokens from t0 on: 1024 rotation tasks (a 16-byte chunk of the first half of
// a key and its partner in the second half), two per thread, and 2048 copy tasks (a 16-byte chunk
// of a value row), four per thread.
constexpr int kNewRowsPerRound = 128;
RD_HD int rope_k_token(int t0, int tid, int i) { return t0 + ((tid + kThreads * i) >> 3); }
RD_HD int rope_k_chunk(int tid, int i) { return (tid + kThreads * i) & 7; }
RD_HD int rope_v_token(int t0, int tid, int i) { return t0 + ((tid + kThreads * i) >> 4); }
RD_HD int rope_v_chunk(int tid, int i) { return (tid + kThreads * i) & 15; }
// cache row of new token t (a shift that would leave the slab is not followed: the row is dropped)
RD_HD int64_t new_cache_row(int new_col0, int t, int kv_shift) { return (int64_t)new_col0 + t - kv_shift; }
RD_HD bool new_row_in_slab(int new_col0, int t, int kv_shift, int64_t max_len) {
  const int64_t row = new_cache_row(new_col0, t, kv_shift);
  return row >= 0 && row < max_len;
}

}  // namespace attn
}  // namespace rd
