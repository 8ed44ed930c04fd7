// Layout of the attention plan shared by the planning and the attention kernels.
//
// plan (int32):
//   [0] n_items  [1] n_q  [2] kv_len  [3] words per mask row  [4] max_splits  [5] chunk  [6..7] 0
//   per batch row b, 4 ints at RD_PLAN_HDR + 4*b:  {kv_begin, n_splits, first_item, kv_shift}
//     (kv_shift: key column c of this row lives in cache row c - kv_shift; 0 unless the cache is
//      kept in place when the token ids are re-aligned)
//   items, RD_ITEM_INTS ints each at RD_PLAN_HDR + 4*batch, longest first:
//     {b, kv_lo, kv_hi, split, kv_shift, key_min, n_splits, key_end}: everything the attention kernel
//     needs for its first loads comes with this one record.  [key_min, key_end) spans the keys that
//     some query of the row attends to; the items of a row cover [key_min rounded down to a tile
//     boundary, key_end), and the keys of the first and last tile outside the span (left padding,
//     tree slots that do not exist: masked for every query) are never read from memory
//   scratch: first and last attended key of every (b, q) row (two arrays of batch * n_q)
// The plan is read-only for the attention kernels: the arrival counters of split rows live in a
// device array of the library (verify_attention.hip), a fresh slab of it for every launch.
//
// Nothing here needs the HIP runtime: the sizes and the arithmetic that decides how a row's keys
// are cut into work items compile for the device and for the host alike, so that a host program
// can form the plan of any launch and check it.
#pragma once

#include <stddef.h>
#include <stdint.h>

#include "attn_addr.h"

#define RD_PLAN_HDR 8
#define RD_ITEM_INTS 8

namespace rd {

constexpr int kAttnChunk = 512;       // target keys per work item
constexpr int kAttnSortLimit = 2048;  // more items than this are dispatched unsorted

constexpr int kAttnMaxHeads = 128;    // heads the MFMA kernel takes
constexpr int kAttnRowsPerTile = 256; // query rows of the largest workgroup layout

inline int attn_max_splits(int kv_len) { return (kv_len + kAttnChunk - 1) / kAttnChunk; }
inline int attn_max_q_tiles(int n_q) { return (n_q + kAttnRowsPerTile - 1) / kAttnRowsPerTile; }
inline size_t attn_plan_ints(int batch, int n_q, int kv_len) {
  return RD_PLAN_HDR + 4 * (size_t)batch + RD_ITEM_INTS * (size_t)batch * attn_max_splits(kv_len) + 2 * (size_t)batch * n_q;
}
// arrival counters of one launch: one per (batch row, head, query tile)
inline size_t attn_counter_ints(int batch, int n_heads, int n_q) {
  return (size_t)batch * n_heads * attn_max_q_tiles(n_q);
}

// ---- how a row's keys become work items ------------------------------------------------------
// A row's items cover [plan_begin(key_min), key_end): from the tile that holds its first attended
// key to its last attended key.
RD_HD int plan_begin(int key_min) { return (key_min / 64) * 64; }
// keys per item of a row of `live` keys cut into `splits` items: equal shares, whole tiles
RD_HD int plan_per(int live, int splits) {
  const int per = (live + splits - 1) / splits;
  return (per + 63) / 64 * 64;
}
// Items of a row of `live` keys at `chunk` keys per item.  An item may run an eighth over the
// chunk: a row a little longer than it stays whole (cutting off a short remainder would cost it
// the partials and the merge, and would send the remainders into a second round of items behind
// the first).  The share of an item is rounded up to whole tiles, which can cover the row with
// fewer items than first counted: the count returned is the number of items that hold keys, so
// that no item is ever empty.
RD_HD int plan_splits(int live, int chunk, int max_splits) {
  int splits = (live + chunk - 1 - chunk / 8) / chunk;
  splits = splits < 1 ? 1 : (splits > max_splits ? max_splits : splits);
  const int per = plan_per(live, splits);
  const int needed = (live + per - 1) / per;
  return needed < 1 ? 1 : needed;
}
// key range [lo, hi) of item s of a row's `splits` items
RD_HD void plan_extent(int begin, int end, int splits, int s, int* lo, int* hi) {
  const int per = plan_per(end - begin, splits);
  int l = begin + s * per, h = l + per;
  *lo = l < end ? l : end;
  *hi = h < end ? h : end;
}
// Keys per work item, first guess: one compute unit's even share of all (row, head) work, in whole
// tiles, but never below min_chunk.  Equal rows on a machine with batch * heads == compute units
// are then not split at all (no partials to merge).
RD_HD int plan_share(long long total_keys, int n_heads, int n_cu, int min_chunk) {
  long long share = (total_keys * n_heads + n_cu - 1) / n_cu;
  share = (share + 63) / 64 * 64;
  return (int)(share > min_chunk ? share : min_chunk);
}
// the item sizes tried for ragged rows: share * (1 .. 2.5) in eighths (smaller ones only split more)
constexpr int kPlanCandidates = 13;
RD_HD int plan_candidate(int share, int c) { return (int)((long long)share * (8 + c) / 8) / 64 * 64; }

}  // namespace rd
