// Host-side walk over every memory address of an attn_mfma_kernel launch (test infrastructure).
//
// The kernel forms its addresses with the integer functions of csrc/attn_addr.h and cuts rows into
// work items with those of csrc/attn_plan.h; this program calls the same functions for every
// (work item, head, query tile, thread, tile) of a launch and holds each address against the
// extent of the tensor it falls into: Q and the output, the K/V cache rows of the span of attended
// keys, the mask words, the partial results and arrival counters of split rows, the new cache rows
// of the fused rotation, and every LDS offset.  What it restates from the kernel is only the ORDER
// of the accesses (which tiles a work item walks over, which rows a wave owns), not their arithmetic.
//
// Built by tests/test_attn_addresses_cpu.py with g++; no GPU, no HIP runtime.
#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <set>
#include <string>
#include <vector>

#include "attn_plan.h"

using namespace rd::attn;

extern "C" {

struct Launch {
  int B, H, Hkv, n_q, kv_len;
  int n_heads_for_plan;  // the head count the plan was made for (sizes the items)
  int n_cu;
  int64_t q_sb, q_sh, q_ss, q_elems;  // *_elems: elements of the allocation behind the pointer
  int64_t k_sb, k_sh, k_ss;           // K and V views share one geometry (two slabs of one cache)
  int64_t slab_rows;                  // cache rows of one (batch row, kv head) slab
  int64_t kv_elems;
  int64_t o_sb, o_sh, o_ss, o_elems;
  const int32_t* row_start;  // B + 1 entries, or null (padded query layout)
  const int32_t* key_min;    // per batch row: the span of keys that some query attends to
  const int32_t* key_end;
  const int32_t* kv_shift;   // per batch row (null: zeros)
  int forced_chunk;          // > 0: only this item size; 0: the share and every candidate of the search
  // the fused rotation + append (rope != 0)
  int rope;
  int64_t kn_sb, kn_st, kn_elems;  // new keys/values: batch and token strides, allocation
  int64_t pos_sb, pos_elems;
  int64_t max_len;
  int64_t table_rows;
};

struct Stats {
  long long items, workgroups, tile_loads, q_loads, stores, partial_rows, new_rows, chunks_tried;
};

}  // extern "C"

namespace {

struct Failure {
  char msg[512];
  bool failed = false;
  void set(const char* fmt, ...) {
    if (failed) return;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(msg, sizeof msg, fmt, ap);
    va_end(ap);
    failed = true;
  }
};

#define CHECK(cond, ...)            \
  do {                              \
    if (!(cond)) {                  \
      f.set(__VA_ARGS__);           \
      return;                       \
    }                               \
  } while (0)

struct Item { int b, lo, hi, split, n_splits; };

size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// LDS: every staging write and fragment read inside its region and aligned, the staging writes of
// a tile disjoint, and every fragment read delivers the elements the MFMA operand layout asks for.
// The staging is modelled by what it writes: element (key, dim) of the tile is tagged key * 128 + dim
// at the place its loader thread puts it; the fragment reads are then emulated on that model -- for
// V with the lane exchange of the transposing read (lane i of a group of 16 receives, as element e,
// element i % 4 of the 8 bytes that lane i / 4 + 4 * e of its group points at).
void check_lds(Failure& f) {
  for (int j = 0; j < 12; ++j) {
    std::vector<int> k_tag(kKBytes / 2, -1), v_tag(kVBytes / 2, -1);
    for (int tid = 0; tid < kThreads; ++tid) {
      const Loader ld = loader_of(tid);
      CHECK(ld.k_loader == (tid / 64 < kWaves / 2), "loader role of thread %d", tid);
      CHECK(ld.chunk >= 0 && ld.chunk < 16 && ld.lrow >= 0 && ld.lrow < 16, "loader lane map of thread %d", tid);
      for (int i = 0; i < 4; ++i) {
        const int key = ld.first_key + i * ld.key_step;  // the tile row this chunk was loaded from
        CHECK(key >= 0 && key < kTile, "loader thread %d chunk %d: key %d of the tile", tid, i, key);
        const int off = ld.k_loader ? lds_k_stage(ld, j, i) : lds_v_stage(ld, j, i);
        const int lo = ld.k_loader ? 0 : kKBytes, hi = ld.k_loader ? kKBytes : kLdsBytes;
        CHECK(off >= lo && off + 16 <= hi && off % 16 == 0, "stage offset %d (thread %d tile %d chunk %d)", off, tid, j, i);
        std::vector<int>& tag = ld.k_loader ? k_tag : v_tag;
        for (int x = 0; x < 8; ++x) {
          int& t = tag[(off - lo) / 2 + x];
          CHECK(t == -1, "stage writes overlap at byte %d", off + 2 * x);
          t = key * kD + 8 * ld.chunk + x;
        }
      }
    }
    for (int key_off = 0; key_off <= 32; key_off += 32)
      for (int c = 0; c < 8; ++c) {
        for (int lane = 0; lane < 64; ++lane) {
          const int r = lane & 31, g = lane >> 5;
          // K fragment ks = c: B^T operand of S^T = K Q^T: lane (r, g) holds K[key_off + r][16 c + 8 g ..]
          const int ko = lds_k_frag(j, key_off, r, g, c);
          CHECK(ko >= 0 && ko + 16 <= kKBytes && ko % 16 == 0, "K fragment offset %d", ko);
          for (int x = 0; x < 8; ++x)
            CHECK(k_tag[ko / 2 + x] == (key_off + r) * kD + 16 * c + 8 * g + x, "K fragment %d of lane %d: element %d is %d", c, lane, x, k_tag[ko / 2 + x]);
        }
        // V^T fragment c: two transposing reads; k-slot s of lane (r, g) must be
        // V[key_off + 16 (c % 2) + 4 g + s % 4 + 8 (s / 4)][32 (c / 2) + r]
        for (int half = 0; half < 2; ++half)
          for (int lane = 0; lane < 64; ++lane) {
            const int own = lds_v_frag(j, key_off, lane, c, half);
            CHECK(own >= kKBytes && own + 8 <= kLdsBytes && own % 8 == 0, "V fragment offset %d (lane %d)", own, lane);
            const int r = lane & 31, g = lane >> 5, i = lane & 15, group = lane & ~15;
            for (int e = 0; e < 4; ++e) {
              const int src = lds_v_frag(j, key_off, group + (i >> 2) + 4 * e, c, half);
              const int got = v_tag[(src - kKBytes) / 2 + (i & 3)];
              const int s_slot = 4 * half + e;
              const int want = (key_off + 16 * (c & 1) + 4 * g + (s_slot & 3) + 8 * (s_slot >> 2)) * kD + 32 * (c >> 1) + r;
              CHECK(got == want, "V fragment %d half %d of lane %d: slot %d holds element %d, the operand wants %d", c, half, lane, s_slot, got, want);
            }
          }
      }
  }
  for (int pair = 0; pair < kWaves / 2; ++pair)
    for (int lane = 0; lane < 64; ++lane) {
      for (int acc = 0; acc < 64; ++acc) {
        const int off = lds_merge_o(pair, acc, lane);
        CHECK(off >= 0 && off + 4 <= kLdsBytes && off + 4 <= lds_merge_ml(0, 0, 0, 0), "merge accumulator offset %d", off);
      }
      for (int part = 0; part < 2; ++part)
        for (int which = 0; which < 2; ++which) {
          const int off = lds_merge_ml(pair, part, which, lane);
          CHECK(off >= lds_merge_o(kWaves / 2 - 1, 63, 63) + 4 && off + 4 <= kLdsBytes && off + 4 <= kMergeFloats * 4, "merge (m, l) offset %d", off);
        }
    }
  // Results through LDS: every wave puts the accumulator blocks it keeps into its own region (tagged
  // here row * 128 + dim) and reads them back along the rows; every piece it reads must hold the
  // four dims the store then writes, and no two waves may share a byte.
  for (int layout = kSplit; layout <= kFull; ++layout) {
    std::vector<int> tag(kLdsBytes / 2, -1), owner(kLdsBytes / 2, -1);
    for (int w = 0; w < kWaves; ++w) {
      const WaveRole role = wave_role(layout, w);
      const int first = first_block_kept(role.part), blocks = blocks_kept(role.part);
      for (int lane = 0; lane < 64; ++lane) {
        const int r = lane & 31, g = lane >> 5;
        for (int db = first; db < first + blocks; ++db)
          for (int i4 = 0; i4 < 4; ++i4) {
            const int off = lds_out_stage(w, r, g, db, i4);
            CHECK(off >= 0 && off + 8 <= kLdsBytes && off % 8 == 0, "output stage offset %d (layout %d wave %d lane %d)", off, layout, w, lane);
            for (int x = 0; x < 4; ++x) {
              CHECK(tag[off / 2 + x] == -1, "output stage writes overlap at byte %d (layout %d wave %d)", off + 2 * x, layout, w);
              tag[off / 2 + x] = r * kD + 32 * db + 8 * i4 + 4 * g + x;  // accumulator 4*i4 + x of block db
              owner[off / 2 + x] = w;
            }
          }
      }
    }
    for (int w = 0; w < kWaves; ++w) {
      const WaveRole role = wave_role(layout, w);
      const int first = first_block_kept(role.part), blocks = blocks_kept(role.part);
      std::vector<int> seen(32 * kD, 0);
      CHECK(out_passes(blocks) * 64 == 32 * 8 * blocks, "output passes of a wave that keeps %d blocks", blocks);
      for (int pass = 0; pass < out_passes(blocks); ++pass)
        for (int lane = 0; lane < 64; ++lane) {
          const int row = out_piece_row(blocks, pass, lane), dim = out_piece_dim(first, blocks, pass, lane);
          CHECK(row >= 0 && row < 32 && dim >= 32 * first && dim + 4 <= 32 * (first + blocks) && dim % 4 == 0, "output piece (row %d, dim %d) of pass %d lane %d", row, dim, pass, lane);
          const int off = lds_out_piece(w, row, dim);
          CHECK(off >= 0 && off + 8 <= kLdsBytes && off % 8 == 0, "output piece offset %d", off);
          for (int x = 0; x < 4; ++x) {
            CHECK(owner[off / 2 + x] == w && tag[off / 2 + x] == row * kD + dim + x, "layout %d wave %d reads (row %d, dim %d) and finds %d of wave %d", layout, w, row, dim + x, tag[off / 2 + x], owner[off / 2 + x]);
            seen[row * kD + dim + x]++;
          }
        }
      for (int row = 0; row < 32; ++row)
        for (int d = 0; d < kD; ++d)
          CHECK(seen[row * kD + d] == (d >= 32 * first && d < 32 * (first + blocks) ? 1 : 0), "layout %d wave %d: (row %d, dim %d) goes out %d times", layout, w, row, d, seen[row * kD + d]);
    }
  }
  // the two waves of a pair hand over disjoint accumulator blocks and keep the other two: every
  // block of the head dimension is kept by exactly one of them
  for (int part = 0; part < 2; ++part) {
    CHECK(blocks_kept(part) == 2 && first_block_kept(part) == 2 * part, "blocks kept by key part %d", part);
  }
  CHECK(blocks_kept(2) == 4 && first_block_kept(2) == 0, "blocks kept by a full wave");
  // every layout gives every row block either one full wave or two halves with distinct key parts,
  // and halves of different blocks distinct merge slots
  for (int layout = kSplit; layout <= kFull; ++layout) {
    const int blocks = rows_per_wg(layout) / 32;
    std::vector<int> full(blocks, 0), half0(blocks, 0), half1(blocks, 0);
    std::set<int> pairs;
    for (int w = 0; w < kWaves; ++w) {
      const WaveRole role = wave_role(layout, w);
      CHECK(role.block >= 0 && role.block < blocks, "layout %d wave %d: row block %d", layout, w, role.block);
      CHECK(role.part >= 0 && role.part <= 2 && role.pair >= 0 && role.pair < kWaves / 2, "layout %d wave %d role", layout, w);
      if (role.part == 2) full[role.block]++;
      else (role.part ? half1 : half0)[role.block]++;
    }
    for (int blk = 0; blk < blocks; ++blk) {
      const bool as_full = full[blk] == 1 && half0[blk] == 0 && half1[blk] == 0;
      const bool as_halves = full[blk] == 0 && half0[blk] == 1 && half1[blk] == 1;
      CHECK(as_full || as_halves, "layout %d: row block %d has %d full waves and %d + %d halves", layout, blk, full[blk], half0[blk], half1[blk]);
    }
    for (int w = 0; w < kWaves; ++w) {
      const WaveRole a = wave_role(layout, w);
      if (a.part == 2) continue;
      for (int v = 0; v < kWaves; ++v) {
        const WaveRole b = wave_role(layout, v);
        if (b.part == 2 || v == w) continue;
        CHECK((a.pair == b.pair) == (a.block == b.block), "layout %d: waves %d and %d share a merge slot or a block but not both", layout, w, v);
      }
    }
  }
}

void check_items(const Launch& L, const std::vector<Item>& items, int chunk, int max_splits, Failure& f, Stats& st) {
  const int words = (L.kv_len + 63) / 64;
  const int layout = layout_for(L.n_q);
  const int rows_wg = rows_per_wg(layout);
  const int q_tiles = (L.n_q + rows_wg - 1) / rows_wg;
  const long long slots = (long long)L.B * L.H * max_splits;
  const size_t part_o_bytes = align_up((size_t)slots * L.n_q * kD * sizeof(float), 256);
  const size_t part_ml_bytes = align_up((size_t)slots * L.n_q * 2 * sizeof(float), 256);
  const size_t plan_ints = rd::attn_plan_ints(L.B, L.n_q, L.kv_len);
  // every lane reads entry min(lane, B) of row_start, or of the plan where the rows are not packed
  CHECK(plan_ints >= (size_t)(L.B < 63 ? L.B : 63) + 1, "the plan is shorter than the %d entries read in place of row_start", (L.B < 63 ? L.B : 63) + 1);
  CHECK((int)items.size() <= L.B * max_splits, "chunk %d: %zu items, the plan holds %d", chunk, items.size(), L.B * max_splits);
  CHECK(RD_PLAN_HDR + 4 * (size_t)L.B + RD_ITEM_INTS * (size_t)L.B * max_splits <= plan_ints, "item slots beyond the plan");
  CHECK(q_tiles <= rd::attn_max_q_tiles(L.n_q) || L.n_q <= 256, "query tiles %d beyond the counters' %d", q_tiles, rd::attn_max_q_tiles(L.n_q));
  CHECK(L.H <= rd::kAttnMaxHeads, "heads %d", L.H);
  CHECK(span_fits(L.kv_len, L.k_ss * 2), "keys %d x %lld bytes per cache row do not fit the 32-bit offsets of the tile loads", L.kv_len, (long long)L.k_ss * 2);
  for (const Item& it : items) {
    ++st.items;
    const int b = it.b, lo = it.lo, hi = it.hi;
    const int key_min = L.key_min[b], key_end = L.key_end[b];
    const int kv_shift = L.kv_shift ? L.kv_shift[b] : 0;
    const int n_tiles = n_tiles_of(lo, hi);
    CHECK(n_tiles >= 1, "chunk %d: empty item [%d, %d) of row %d", chunk, lo, hi, b);
    CHECK(lo % kTile == 0 && lo >= 0 && hi <= L.kv_len && hi <= key_end, "chunk %d: item [%d, %d) of row %d (kv_len %d, key_end %d)", chunk, lo, hi, b, L.kv_len, key_end);
    int rows_n = L.n_q;
    int64_t q_off = (int64_t)b * L.q_sb, o_off = (int64_t)b * L.o_sb;
    int r0 = -1;
    if (L.row_start) {
      r0 = L.row_start[b];
      const int n = L.row_start[b + 1] - r0;
      rows_n = n < L.n_q ? n : L.n_q;
      q_off = (int64_t)r0 * L.q_ss;
      o_off = (int64_t)r0 * L.o_ss;
    }
    const NewRows nr = new_rows_of_item(lo, hi, key_end, L.kv_len - L.n_q, rows_n);
    for (int h = 0; h < L.H; ++h) {
      const int hk = h / (L.H / L.Hkv);
      for (int q_tile = 0; q_tile < q_tiles; ++q_tile) {
        if (q_tile * rows_wg >= rows_n) continue;  // the workgroup returns
        ++st.workgroups;
        const int64_t cidx = counter_index(b, L.H, h, q_tiles, q_tile);
        CHECK(cidx >= 0 && (size_t)cidx < rd::attn_counter_ints(L.B, L.H, L.n_q), "counter index %lld of %zu", (long long)cidx, rd::attn_counter_ints(L.B, L.H, L.n_q));
        std::vector<int> covered((size_t)rows_wg * (kD / 4), 0);  // pieces of four dims of the tile's rows
        for (int tid = 0; tid < kThreads; ++tid) {
          const int wave = tid >> 6, lane = tid & 63, g = lane >> 5, r = lane & 31;
          const WaveRole role = wave_role(layout, wave);
          const int q_row = q_row_of(q_tile, rows_wg, role.block, r);
          const bool row_valid = q_row < rows_n;
          const bool wave_active = q_tile * rows_wg + role.block * 32 < rows_n;
          // Q fragments and mask words (rows past the count read row 0 of the batch row)
          const int q_use = row_valid ? q_row : 0;
          for (int ks = 0; ks < 8; ++ks) {
              const int64_t off = q_off + q_frag_offset(h, L.q_sh, q_use, L.q_ss, g, ks);
              CHECK(off >= 0 && off + 8 <= L.q_elems, "Q element %lld of %lld (row %d head %d query %d)", (long long)off, (long long)L.q_elems, b, h, q_row);
              ++st.q_loads;
            }
          // the tiles an item walks over: the prologue and the ring request tiles 0 .. n_tiles - 1 and,
          // past the end, repeats of the last one; the mask word travels with its tile
          const Loader ld = loader_of(tid);
          for (int j = 0; j < n_tiles + 2 + kRing; ++j) {
            const int key0 = tile_key0(lo, j, n_tiles);
            const int64_t w = mask_word_index(b, L.n_q, q_use, words, key0);
            CHECK(w >= 0 && w < (int64_t)L.B * L.n_q * words && (key0 >> 6) < words, "mask word %lld (row %d query %d key0 %d)", (long long)w, b, q_use, key0);
            // K and V through the descriptor over the span's cache rows: a lane is served exactly if
            // its key lies in the span, and then reads inside the slab
            const int64_t row_bytes = L.k_ss * 2;
            const uint32_t records = span_bytes(key_min, key_end, row_bytes);
            for (int i = 0; i < 4; ++i) {
              const int key = tile_chunk_key(ld, key0, i);
              const uint32_t at = tile_chunk_offset(ld, key0, i, key_min, row_bytes);
              // (the kernel forms the same number from three 32-bit parts: the tile's place relative to
              // the span, which wraps around below it, the thread's place in a tile, the chunk's step)
              const uint32_t in_parts = (uint32_t)((int64_t)(key0 - key_min) * row_bytes) + tile_chunk_offset(ld, 0, 0, 0, row_bytes) +
                                        (uint32_t)i * (uint32_t)(ld.key_step * row_bytes);
              CHECK(in_parts == at, "tile load offset of key %d: %u in parts, %u whole", key, in_parts, at);
              const bool served = chunk_in_range(at, records);
              CHECK(served == (key >= key_min && key < key_end), "tile load of key %d (span [%d, %d) of row %d, item [%d, %d) tile %d thread %d): offset %u of %u bytes is %s", key, key_min, key_end, b, lo, hi, j, tid, at, records, served ? "served" : "refused");
              if (!served) continue;
              CHECK((int64_t)at == (int64_t)(key - key_min) * row_bytes + 16 * ld.chunk, "tile load offset %u of key %d", at, key);
              const int64_t row = (int64_t)key - kv_shift;
              CHECK(row >= 0 && row < L.slab_rows, "cache row %lld of %lld (row %d key %d shift %d)", (long long)row, (long long)L.slab_rows, b, key, kv_shift);
              const int64_t off = (int64_t)b * L.k_sb + (int64_t)hk * L.k_sh + row * L.k_ss + 8 * ld.chunk;
              CHECK(off >= 0 && off + 8 <= L.kv_elems, "K/V element %lld of %lld", (long long)off, (long long)L.kv_elems);
              ++st.tile_loads;
            }
          }
          // results.  A row with all its keys in one item: every active wave sends out the rows of its
          // block along the rows, whatever rows its lanes computed
          if (it.n_splits == 1 && wave_active) {
            const int first = first_block_kept(role.part), blocks = blocks_kept(role.part);
            for (int pass = 0; pass < out_passes(blocks); ++pass) {
              const int row = out_piece_row(blocks, pass, lane), dim = out_piece_dim(first, blocks, pass, lane);
              const int q = q_row_of(q_tile, rows_wg, role.block, row);
              if (q >= rows_n) continue;
              const int64_t off = o_off + out_row_offset(h, L.o_sh, q, L.o_ss, dim);
              CHECK(off >= 0 && off + 4 <= L.o_elems, "output element %lld of %lld (row %d head %d query %d)", (long long)off, (long long)L.o_elems, b, h, q);
              CHECK(q >= q_tile * rows_wg && q < (q_tile + 1) * rows_wg, "query %d outside tile %d", q, q_tile);
              covered[(size_t)(q - q_tile * rows_wg) * (kD / 4) + dim / 4]++;
              ++st.stores;
            }
          }
          const bool writer = wave_active && row_valid;  // split rows: every wave leaves the accumulator blocks it keeps as partials
          if (writer) {
            if (it.n_splits > 1) {
              const int64_t row = partial_row(b, L.H, h, max_splits, it.split, L.n_q, q_row);
              CHECK(row >= 0 && row < slots * L.n_q, "partial row %lld of %lld", (long long)row, slots * L.n_q);
              CHECK((size_t)(row * kD + 4 * g + 32 * 3 + 8 * 3 + 4) * sizeof(float) <= part_o_bytes, "partial O beyond the workspace");
              CHECK((size_t)(row * 2 + 2) * sizeof(float) <= part_ml_bytes, "partial (m, l) beyond the workspace");
              ++st.partial_rows;
            }
          }
          // the merge of a split row, by whichever item arrives last: rows q0 + 16 * j of the tile
          if (it.n_splits > 1) {
            const int q_end = (q_tile + 1) * rows_wg < rows_n ? (q_tile + 1) * rows_wg : rows_n;
            const int rg = tid >> 5, dq = (tid & 31) * 4;
            for (int q0 = q_tile * rows_wg + rg; q0 < q_end; q0 += 16 * 8)
              for (int s = 0; s < it.n_splits; ++s)
                for (int j = 0; j < 8; ++j) {
                  const int q = q0 + 16 * j < q_end ? q0 + 16 * j : q_end - 1;
                  const int64_t row = partial_row(b, L.H, h, max_splits, s, L.n_q, q);
                  CHECK(row >= 0 && row < slots * L.n_q && q >= 0, "merge reads partial row %lld of %lld", (long long)row, slots * L.n_q);
                  CHECK((size_t)(row * kD + dq + 4) * sizeof(float) <= part_o_bytes, "merge reads beyond the workspace");
                  if (q0 + 16 * j < q_end) {
                    const int64_t off = o_off + out_offset(h, L.o_sh, q0 + 16 * j, L.o_ss, 0, 0, 0) + dq;
                    CHECK(off >= 0 && off + 4 <= L.o_elems, "merged output element %lld of %lld", (long long)off, (long long)L.o_elems);
                  }
                }
          }
          // the positions are asked for before the row's query count is known, by every thread: of
          // its query row and of the tokens of two rounds of new rows, clamped to the array
          if (L.rope) {
            CHECK(nr.t_lo == new_rows_of_item(lo, hi, key_end, L.kv_len - L.n_q, 0).t_lo, "the first new token depends on the row count");
            CHECK(nr.t_hi - nr.t_lo <= 2 * kNewRowsPerRound, "%d new tokens in one item: more than two rounds", nr.t_hi - nr.t_lo);
            const int64_t qp = (int64_t)b * L.pos_sb + (q_row < L.n_q ? q_row : L.n_q - 1);
            CHECK(qp >= 0 && qp < L.pos_elems, "position id %lld of %lld (query row %d)", (long long)qp, (long long)L.pos_elems, q_row);
            for (int round = 0; round < 2; ++round)
              for (int i = 0; i < 2; ++i) {
                const int t = rope_k_token(nr.t_lo + kNewRowsPerRound * round, tid, i);
                const int64_t pos = (int64_t)b * L.pos_sb + (t < L.n_q ? t : L.n_q - 1);
                CHECK(t >= 0 && pos >= 0 && pos < L.pos_elems, "position id %lld of %lld (token %d)", (long long)pos, (long long)L.pos_elems, t);
              }
          }
          // new cache rows of the fused rotation
          if (L.rope && nr.t_lo < nr.t_hi) {
            const int new_col0 = L.kv_len - L.n_q;
            const int64_t new_off = r0 >= 0 ? (int64_t)r0 * L.kn_st : (int64_t)b * L.kn_sb;
            for (int round = 0; nr.t_lo + kNewRowsPerRound * round < nr.t_hi; ++round) {
              const int t0 = nr.t_lo + kNewRowsPerRound * round;
              for (int i = 0; i < 6; ++i) {
                const bool is_k = i < 2;
                const int t = is_k ? rope_k_token(t0, tid, i) : rope_v_token(t0, tid, i - 2);
                const int c = is_k ? rope_k_chunk(tid, i) : rope_v_chunk(tid, i - 2);
                const bool on = t < nr.t_hi && new_row_in_slab(new_col0, t, kv_shift, L.max_len);
                const int tl = on ? t : t0;  // (a thread without a task reads the round's first token)
                CHECK(tl >= 0 && tl < rows_n, "new token %d of %d (row %d)", tl, rows_n, b);
                const int64_t src = new_off + (int64_t)hk * kD + (int64_t)tl * L.kn_st + 8 * c + (is_k ? kD / 2 : 0);
                CHECK(src >= 0 && src + 8 <= L.kn_elems, "new key/value element %lld of %lld", (long long)src, (long long)L.kn_elems);
                if (on) {
                  const int64_t row = new_cache_row(new_col0, t, kv_shift);
                  CHECK(row >= 0 && row < L.slab_rows && row < L.max_len, "new cache row %lld of %lld", (long long)row, (long long)L.slab_rows);
                  const int64_t off = (int64_t)b * L.k_sb + (int64_t)hk * L.k_sh + row * L.k_ss + 8 * c + (is_k ? kD / 2 : 0);
                  CHECK(off >= 0 && off + 8 <= L.kv_elems, "new cache element %lld of %lld", (long long)off, (long long)L.kv_elems);
                  ++st.new_rows;
                }
              }
            }
          }
        }
        // a row that is not split goes out whole, every piece once, and no row past the count
        if (it.n_splits == 1)
          for (int row = 0; row < rows_wg; ++row)
            for (int piece = 0; piece < kD / 4; ++piece) {
              const int want = q_tile * rows_wg + row < rows_n ? 1 : 0;
              CHECK(covered[(size_t)row * (kD / 4) + piece] == want, "row %d head %d query %d dims %d..: stored %d times", b, h, q_tile * rows_wg + row, 4 * piece, covered[(size_t)row * (kD / 4) + piece]);
            }
      }
    }
  }
}

// the items of every row at `chunk` keys per item, in row order (the order of dispatch does not
// change any address)
void build_items(const Launch& L, int chunk, int max_splits, std::vector<Item>& items, Failure& f) {
  items.clear();
  for (int b = 0; b < L.B; ++b) {
    const int begin = rd::plan_begin(L.key_min[b]), end = L.key_end[b];
    CHECK(end > L.key_min[b] && L.key_min[b] >= 0 && end <= L.kv_len, "span [%d, %d) of row %d", L.key_min[b], end, b);
    const int live = end - begin;
    const int splits = rd::plan_splits(live, chunk, max_splits);
    CHECK(splits >= 1 && splits <= max_splits, "chunk %d: %d splits of %d keys (at most %d)", chunk, splits, live, max_splits);
    int expect = begin;
    for (int s = 0; s < splits; ++s) {
      int lo, hi;
      rd::plan_extent(begin, end, splits, s, &lo, &hi);
      CHECK(lo == expect && hi > lo, "chunk %d: item %d of row %d is [%d, %d), expected to begin at %d and hold keys", chunk, s, b, lo, hi, expect);
      expect = hi;
      items.push_back({b, lo, hi, s, splits});
    }
    CHECK(expect == end, "chunk %d: the items of row %d end at %d, its span at %d", chunk, b, expect, end);
  }
}

}  // namespace

extern "C" int attn_check_lds(char* msg, int msg_len) {
  Failure f;
  check_lds(f);
  if (f.failed) snprintf(msg, msg_len, "%s", f.msg);
  return f.failed ? 1 : 0;
}

extern "C" int attn_check_launch(const Launch* launch, Stats* stats, char* msg, int msg_len) {
  const Launch& L = *launch;
  Failure f;
  Stats st;
  memset(&st, 0, sizeof st);
  const int max_splits = rd::attn_max_splits(L.kv_len);
  std::set<int> chunks;
  if (L.forced_chunk > 0) {
    chunks.insert(L.forced_chunk);
  } else {
    long long total = 0;
    for (int b = 0; b < L.B; ++b) total += L.key_end[b] - rd::plan_begin(L.key_min[b]);
    const int share = rd::plan_share(total, L.n_heads_for_plan, L.n_cu, rd::kAttnChunk);
    chunks.insert(share);
    for (int c = 0; c < rd::kPlanCandidates; ++c) chunks.insert(rd::plan_candidate(share, c));
  }
  std::vector<Item> items;
  for (int chunk : chunks) {
    ++st.chunks_tried;
    build_items(L, chunk, max_splits, items, f);
    if (!f.failed) check_items(L, items, chunk, max_splits, f, st);
    if (f.failed) break;
  }
  if (stats) *stats = st;
  if (f.failed) snprintf(msg, msg_len, "%s", f.msg);
  return f.failed ? 1 : 0;
}

// Plan arithmetic alone, over a sweep: every item non-empty, the items of a row tile its span.
extern "C" int attn_check_plan_sweep(int live_max, char* msg, int msg_len) {
  Failure f;
  for (int live = 1; live <= live_max && !f.failed; live += (live < 1300 ? 1 : 7)) {
    const int kv_len = live + 5;
    const int max_splits = rd::attn_max_splits(kv_len);
    for (int chunk = rd::kAttnChunk; chunk <= 4096 && !f.failed; chunk += 64) {
      const int splits = rd::plan_splits(live, chunk, max_splits);
      if (splits < 1 || splits > max_splits) { f.set("live %d chunk %d: %d splits (max %d)", live, chunk, splits, max_splits); break; }
      int expect = 0;
      for (int s = 0; s < splits; ++s) {
        int lo, hi;
        rd::plan_extent(0, live, splits, s, &lo, &hi);
        if (lo != expect || hi <= lo || lo % 64 != 0) { f.set("live %d chunk %d: item %d of %d is [%d, %d)", live, chunk, s, splits, lo, hi); break; }
        // an item is never longer than the chunk plus an eighth, rounded up to whole tiles
        if (splits > 1 && hi - lo > (chunk + chunk / 8 + 63) / 64 * 64) { f.set("live %d chunk %d: item of %d keys", live, chunk, hi - lo); break; }
        expect = hi;
      }
      if (!f.failed && expect != live) f.set("live %d chunk %d: items end at %d", live, chunk, expect);
    }
  }
  if (f.failed) snprintf(msg, msg_len, "%s", f.msg);
  return f.failed ? 1 : 0;
}
