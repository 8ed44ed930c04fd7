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
//   arrival counters, one per (b, head, query tile), zero between launches: the work items of a
//   split row count themselves in, and the last one to arrive merges the partials of all
#pragma once

#include "rd_common.h"

#define RD_PLAN_HDR 8
#define RD_ITEM_INTS 8

namespace rd {

constexpr int kAttnChunk = 512;       // target keys per work item
constexpr int kAttnSortLimit = 2048;  // more items than this are dispatched unsorted

constexpr int kAttnMaxHeads = 128;    // heads the arrival counters are laid out for
constexpr int kAttnRowsPerTile = 256; // query rows of the largest workgroup layout

inline int attn_max_splits(int kv_len) { return (kv_len + kAttnChunk - 1) / kAttnChunk; }
inline int attn_max_q_tiles(int n_q) { return (n_q + kAttnRowsPerTile - 1) / kAttnRowsPerTile; }
inline size_t attn_counter_offset(int batch, int n_q, int kv_len) {
  return RD_PLAN_HDR + 4 * (size_t)batch + RD_ITEM_INTS * (size_t)batch * attn_max_splits(kv_len) + 2 * (size_t)batch * n_q;
}
inline size_t attn_counter_ints(int batch, int n_q) {
  return (size_t)batch * kAttnMaxHeads * attn_max_q_tiles(n_q);
}

}  // namespace rd
