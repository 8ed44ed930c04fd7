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
// V tiles lie in LDS as they lie in memory, one key per row; the V^T fragments of the second product
// come out of transposing reads (ds_read_b64_tr_b16).  320-byte rows: the four keys and 32 dims
// that the 32 lanes of one read cycle touch fall into 64 different banks.
constexpr int kVsStride = kD + 32;         // bf16 elements
constexpr int kKBytes = kKBuffers * kTile * kKsStride * 2;
constexpr int kVBytes = kVBuffers * kTile * kVsStride * 2;
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
// Threads [0,256) stage the K tile, threads [256,512) the V tile, both the same way: a thread
// carries the 16-byte chunk `chunk` of the rows lrow + 16*i, i = 0..3 (16 lanes per 256-byte row).
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
  ld.chunk = lt & 15;
  ld.lrow = lt >> 4;
  ld.key_step = 16;
  ld.first_key = ld.lrow;
  return ld;
}
RD_HD int n_tiles_of(int lo, int hi) { return (hi - lo + kTile - 1) / kTile; }
// first key of tile j of an item; tile indices past the end repeat the last tile (the loads of the
// pipeline's tail are issued like all the others and never used)
RD_HD int tile_key0(int lo, int j, int n_tiles) { return lo + (j < n_tiles ? j : n_tiles - 1) * kTile; }
// K and V are read through a buffer descriptor that covers exactly the cache rows of the span
// [key_min, key_end) of keys that some query of the batch row attends to: it begins at the row of
// key_min and holds span_bytes.  A tile may begin up to 63 keys below the span or end behind it; a
// lane whose key lies outside gets zeros from the hardware's range check and asks nothing of the
// memory (the probabilities of those keys are zero, and zero times zero is zero, where zero times
// whatever lay in the cache could be NaN).
// key column read by chunk i (0..3) of a loader thread for the tile at key0
RD_HD int tile_chunk_key(const Loader& ld, int key0, int i) { return key0 + ld.first_key + i * ld.key_step; }
RD_HD uint32_t span_bytes(int key_min, int key_end, int64_t row_bytes) { return (uint32_t)((int64_t)(key_end - key_min) * row_bytes); }
// byte offset of that chunk from the descriptor's base, as the 32-bit number the load instruction
// takes: below the span it wraps around to the top of the range
RD_HD uint32_t tile_chunk_offset(const Loader& ld, int key0, int i, int key_min, int64_t row_bytes) {
  return (uint32_t)((int64_t)(tile_chunk_key(ld, key0, i) - key_min) * row_bytes + 16 * ld.chunk);
}
// the range check of a 16-byte load (no swizzle, no stride in the descriptor)
RD_HD bool chunk_in_range(uint32_t offset, uint32_t records) { return (uint64_t)offset + 16 <= records; }
// what the host checks before a launch: every span fits the 32-bit offsets with room for the
// wrap-around of the 63 rows below it
RD_HD bool span_fits(int64_t kv_len, int64_t row_bytes) { return (kv_len + 2 * kTile) * row_bytes < ((int64_t)1 << 31); }

// ---- LDS -------------------------------------------------------------------------------------
// byte offsets from the start of the workgroup's LDS; K buffers first, then the V buffers
RD_HD int lds_k_stage(const Loader& ld, int j, int i) {  // chunk i of the K tile j
  return ((j % kKBuffers) * kTile * kKsStride + (ld.lrow + 16 * i) * kKsStride + 8 * ld.chunk) * 2;
}
RD_HD int lds_v_stage(const Loader& ld, int j, int i) {  // chunk i of the V tile j
  return kKBytes + ((j % kVBuffers) * kTile * kVsStride + (ld.lrow + 16 * i) * kVsStride + 8 * ld.chunk) * 2;
}
// K fragment ks (0..7) of lane (r, g) for the unit at key_off (0 or 32) of tile j: 8 elements
RD_HD int lds_k_frag(int j, int key_off, int r, int g, int ks) {
  return ((j % kKBuffers) * kTile * kKsStride + (key_off + r) * kKsStride + 16 * ks + 8 * g) * 2;
}
// V^T fragment c (0..7: dims 32 * (c / 2) .., keys 16 * (c % 2) .. of the unit) for the unit at
// key_off of tile j.  The lane (r = lane % 32, g = lane / 32) needs, as k-slot s = 0..7 of the
// MFMA's A operand, V[key_off + 16 * (c % 2) + 4 * g + s % 4 + 8 * (s / 4)][32 * (c / 2) + r]: the
// keys that its P^T operand holds in the same slots.  Two transposing reads deliver them, `half`
// = s / 4 each four slots.  A transposing read works on groups of 16 lanes: lane i of a group
// receives, as element e, element i % 4 of the 8 bytes that lane i / 4 + 4 * e of the group points
// at.  So the lane's OWN address is that of four dims of one key: key ((lane % 16) / 4) of the
// four, dims 4 * (lane % 4) .. of the group's sixteen (lanes 16-31 and 48-63: the upper sixteen
// dims of the 32).
RD_HD int lds_v_frag(int j, int key_off, int lane, int c, int half) {
  const int g = lane >> 5;
  const int key = key_off + 16 * (c & 1) + 4 * g + 8 * half + ((lane & 15) >> 2);
  const int dim = 32 * (c >> 1) + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  return kKBytes + ((j % kVBuffers) * kTile * kVsStride + key * kVsStride + dim) * 2;
}
// Merge of the two key halves of a row block after the loop.  Each wave of the pair ends up with
// one half of the head dimension: the wave with key part 0 keeps dims 0-63 (accumulator blocks 0,
// 1) and hands its blocks 2, 3 over, part 1 keeps dims 64-127 and hands blocks 0, 1 over; both
// leave their (m, l).  [pair][64 accumulators][lane] floats (accumulator 16 * block + i, written by
// the wave that does NOT keep that block), then [pair][key part][m | l][lane].
constexpr int kMergeFloats = (kWaves / 2) * (64 * 64 + 4 * 64);
RD_HD int lds_merge_o(int pair, int acc, int lane) { return ((pair * 64 + acc) * 64 + lane) * 4; }
RD_HD int lds_merge_ml(int pair, int part, int which, int lane) {
  return ((kWaves / 2) * 64 * 64 + ((pair * 2 + part) * 2 + which) * 64 + lane) * 4;
}
// accumulator blocks (32 dims each) that a wave normalises and stores: all four for a full wave,
// two for a half wave
RD_HD int first_block_kept(int part) { return part == 1 ? 2 : 0; }
RD_HD int blocks_kept(int part) { return part == 2 ? 4 : 2; }

// ---- results on their way out: a wave's rows through LDS --------------------------------------
// In the accumulators a lane holds four neighbouring dims of ONE query row, so a store instruction
// of the wave would touch 32 rows with 16 bytes each.  The wave therefore puts its normalised rows
// (32 rows x the dims it keeps, bf16) into a region of its own and reads them back along the rows:
// a store instruction then covers whole rows (256 bytes of a full wave's row, 128 of a half wave's).
// Rows lie 264 bytes apart: the 32 lanes of a half wave, writing 8 bytes each at that stride, hit
// 64 different banks.
constexpr int kOutRowBytes = kD * 2 + 8;
constexpr int kOutWaveBytes = 32 * kOutRowBytes;
// where lane (r, g) puts the four outputs (block db, group i4): dims 32*db + 8*i4 + 4*g ..
RD_HD int lds_out_stage(int wave, int r, int g, int db, int i4) {
  return wave * kOutWaveBytes + r * kOutRowBytes + (32 * db + 8 * i4 + 4 * g) * 2;
}
// The way back: piece = 8 bytes = four dims.  A wave that keeps `blocks` accumulator blocks from
// block `first` on has 8 * blocks pieces per row and takes 64 of them per pass, lane by lane along
// the rows: 32 * 8 * blocks / 64 passes.
RD_HD int out_passes(int blocks) { return 32 * 8 * blocks / 64; }
RD_HD int out_piece_row(int blocks, int pass, int lane) { return (pass * 64 + lane) / (8 * blocks); }
RD_HD int out_piece_dim(int first, int blocks, int pass, int lane) { return 32 * first + 4 * ((pass * 64 + lane) % (8 * blocks)); }
RD_HD int lds_out_piece(int wave, int row, int dim) { return wave * kOutWaveBytes + row * kOutRowBytes + dim * 2; }

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
// element offset of dim `dim` of a query row
RD_HD int64_t out_row_offset(int h, int64_t o_sh, int q_row, int64_t o_ss, int dim) {
  return (int64_t)h * o_sh + (int64_t)q_row * o_ss + dim;
}
RD_HD int64_t mask_word_index(int b, int n_q, int q_row, int words, int key0) {
  return ((int64_t)b * n_q + q_row) * words + (key0 >> 6);
}

// ---- partial results of split rows and their arrival counters --------------------------------
RD_HD int64_t partial_row(int b, int H, int h, int max_splits, int split, int n_q, int q_row) {
  return ((((int64_t)b * H + h) * max_splits) + split) * n_q + q_row;
}
RD_HD int64_t counter_index(int b, int n_heads, int h, int q_tiles, int q_tile) {
  return ((int64_t)b * n_heads + h) * q_tiles + q_tile;
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
