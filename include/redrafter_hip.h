/*
 * redrafter_hip.h -- C ABI of libredrafter_hip.so: the per-step speculative-decoding hot path of
 * Recurrent Drafting (ReDrafter) as hand-written HIP kernels for gfx950 (MI355X).
 *
 * The upstream reference is pure Python on PyTorch and has no FFI of its own; each entry point
 * below replaces one chain of torch ops, cited as <file>:<lines> of the reference repository.
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer unless the comment says "host".  The caller owns all
 *     memory (inputs, outputs, workspaces); nothing here allocates or frees, except where a
 *     function's comment says otherwise.
 *   - `stream` is a hipStream_t passed as void*; all work is enqueued on it and the call returns
 *     without synchronising.  NULL is the default stream.
 *   - Token ids and indices are int64 (the reference asserts torch.long).  Shapes are row-major
 *     and contiguous unless explicit element strides are taken.
 *   - Return value: 0 on success, a negative RD_E* code otherwise; rd_last_error() then returns a
 *     thread-local message.  Arguments are validated on the host BEFORE any launch, so a failed
 *     call enqueues nothing.  No C++ exception crosses this boundary.
 *   - Data-dependent output sizes (packed tree length, new sequence length) are written to small
 *     device arrays; the caller reads them back when it needs the shapes on the host, where the
 *     reference calls int(...) / .item().
 */
#ifndef REDRAFTER_HIP_H_
#define REDRAFTER_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RD_OK 0
#define RD_EINVAL (-1)    /* bad argument / shape / alignment            */
#define RD_ELIMIT (-2)    /* shape beyond a compiled-in kernel limit      */
#define RD_EWORKSPACE (-3) /* workspace too small                         */
#define RD_ELAUNCH (-4)   /* HIP reported an error at launch              */

typedef enum { RD_BF16 = 0, RD_F16 = 1, RD_F32 = 2 } rd_dtype;

#define RD_API __attribute__((visibility("default")))

/* Version of this interface: changes whenever an entry point's arguments, the layout of a buffer
 * that crosses it (the attention plan, the realignment plan) or a workspace size changes.  A caller
 * compiled against this header compares rd_version() with RD_ABI_VERSION before its first call, so
 * that a stale build of the library is refused instead of being called with other arguments. */
#define RD_ABI_VERSION 106
RD_API int rd_version(void);
/* Message of the last failed call on this thread ("" if none). */
RD_API const char* rd_last_error(void);

/* Optional measurement aid, off by default.  rd_timing_enable(1) creates a pool of HIP events
 * (the one place this library allocates) and makes every entry point bracket each of its kernel
 * launches with two events on the launch stream; rd_timing_collect waits for them and writes one
 * text line per kernel, "<kernel> <launches> <total_ms>", into a HOST buffer, then resets the
 * pool.  rd_timing_enable(0) stops recording.  rd_timing_select("kernel_name") restricts the
 * recording to one kernel (the events of every launch cost a few percent of a decode step);
 * NULL or "" selects all again.  rd_timing_sample(n) times every n-th of the launches that qualify
 * (counted from the call and from every rd_timing_enable; n = 1 times all): the two events of a
 * launch keep the GPU idle for about 11 us, which for a kernel launched 32 times per decode step
 * is 2.4 % of the step. */
RD_API int rd_timing_enable(int on);
RD_API int rd_timing_select(const char* kernel);
RD_API int rd_timing_sample(int every);
/* Average event-to-event time of an EMPTY kernel timed the same way, in microseconds: the fixed
 * part (dispatch and completion signalling) that the figures of rd_timing_collect include and a
 * kernel trace does not.  Synchronises the stream. */
RD_API int rd_timing_null_kernel_us(int launches, void* stream, float* avg_us);
RD_API int rd_timing_collect(char* out, size_t out_bytes);

/* ------------------------------------------------------------------------------------------
 * Draft beams -> prefix tree -> packed tokens.
 * Replaces tree_attention._dedup_prefix (tree_attention.py:14-38), _get_unpacker (:125-188),
 * _pack_beams (:41-122) and position_offsets (:335).
 *
 * Limits: width <= 1024, length <= 64, width*length <= 4096.
 * counts (int32, batch+2): [0,batch) tokens selected per row, [batch] = max over rows (max_n),
 * [batch+1] = total over rows.
 * packed_tokens / packed_token_indices / position_offsets have capacity batch*width*length and are
 * written as a contiguous (batch, max_n) array; slots past a row's own count hold the following
 * rows' entries, clamped to the batch's last entry, exactly as the reference's gather does.
 * prefix_tree may be NULL.
 * row_start (int32, batch+1) and row_slots (int64, capacity batch*width*length), both optional:
 * the slots that exist, listed row after row without the padding -- row_start[b] = number of
 * slots of the rows before b (row_start[batch] = total), row_slots[row_start[b] + t] = b*max_n + t
 * for t < counts[b]; the entries from total up to the next multiple of 32 (or the capacity) are 0,
 * so that a caller may round its row count up.  row_tokens (int64, same capacity, optional): the
 * token of each of those slots in the same order, zeros in the rounding entries.  (No counterpart
 * in the reference, which runs the model on the padding too.)
 * ------------------------------------------------------------------------------------------ */
RD_API size_t rd_tree_workspace_bytes(int batch, int width, int length);
RD_API int rd_tree_build(const int64_t* beams, int batch, int width, int length,
                  int64_t* prefix_tree, int64_t* unpacker,
                  int64_t* packed_tokens, int64_t* packed_token_indices,
                  int64_t* position_offsets, int32_t* counts, int32_t* row_start,
                  int64_t* row_slots, int64_t* row_tokens, void* workspace, size_t workspace_bytes,
                  void* stream);

/* ------------------------------------------------------------------------------------------
 * Tree attention mask, rows of the packed tokens only.
 * Replaces tree_attention._get_causal_mask_of_packed_beams (tree_attention.py:191-250),
 * _get_causal_mask (:253-298), attention.causal_mask on the extended padding mask
 * (attention.py:12-55) and the final row slice (tree_attention.py:337).
 *
 * padding_mask: (batch, prev) of pm_elem_bytes-wide integers (1, 4 or 8), row stride
 * pm_row_stride elements; an element equal to pm_pad_value is padding, any other a real token
 * (0 for a 0/1 mask; the pad token id when the token ids themselves are handed in, which saves
 * the caller the comparison).  May be NULL when prev == 0.
 * mask: capacity batch*width*length*(prev+width*length) bytes, written as a contiguous
 * (batch, max_n, prev+max_n) array of 0/1 bytes with max_n = counts[batch].
 * ------------------------------------------------------------------------------------------ */
RD_API int rd_tree_mask(const int64_t* unpacker, const int64_t* packed_token_indices,
                 const int32_t* counts, const void* padding_mask, int pm_elem_bytes,
                 int64_t pm_row_stride, int64_t pm_pad_value, int64_t prev, int batch, int width,
                 int length,
                 uint8_t* mask, void* stream);

/* ------------------------------------------------------------------------------------------
 * Row gather: out[b, t, :] = packed[b, index[b, t], :], t in [0, n_out).
 * Replaces tree_attention.unpack (tree_attention.py:341-387) for hidden states and logits, and
 * _select_one_per_row gathers (recurrent_drafting.py:37-40) when n_out == 1.
 * Rows are row_bytes long; strides are in bytes (packed, out) / elements (index); output row t of
 * batch row b starts at out + b*out_batch_stride_bytes + t*out_row_stride_bytes.  An index outside
 * [0, n_src) leaves its output row untouched.
 * row_start (batch + 1 int32 on the device, or NULL): with it `packed` holds only the rows that
 * exist, batch row after batch row (rd_tree_build's row_start): row r of batch row b is row
 * row_start[b] + r of packed, packed_batch_stride_bytes is not used, and an index at or beyond the
 * batch row's count row_start[b+1] - row_start[b] leaves its output row untouched.
 * ------------------------------------------------------------------------------------------ */
RD_API int rd_unpack_rows(const void* packed, int64_t packed_batch_stride_bytes, int64_t row_bytes,
                          const int64_t* index, int64_t index_batch_stride, int batch, int n_out,
                          int n_src, void* out, int64_t out_batch_stride_bytes,
                          int64_t out_row_stride_bytes, const int32_t* row_start, void* stream);

/* ------------------------------------------------------------------------------------------
 * First maximal index of every row of a (rows, vocab) matrix; NaN counts as the largest value.
 * Replaces torch.argmax(logits_by_llm, dim=-1) (recurrent_drafting.py:52, :425).
 * row_stride in elements.  out_index (rows int64 on the device, or NULL): with it the result of
 * row r goes to out[out_index[r]] instead of out[r] -- the argmax of packed rows written straight
 * to their (batch, slot) places; elements of out that no row names are left as they are.
 * ------------------------------------------------------------------------------------------ */
RD_API int rd_argmax_rows(const void* x, int dtype, int64_t rows, int64_t vocab, int64_t row_stride,
                          int64_t* out, const int64_t* out_index, void* stream);

/* ------------------------------------------------------------------------------------------
 * Greedy acceptance.  Replaces _greedy_choose_from_candidates (recurrent_drafting.py:468-496) and
 * the token half of _greedy_prepare_next_input (:261-263).
 *
 * beams (batch,width,length): drafted tokens, position 0 is the LLM's own token.
 * llm_tokens: the LLM's argmax per candidate position.  With unpacker == NULL it is laid out
 * (batch,width,length) with row stride llm_row_stride; otherwise it is indexed per PACKED slot,
 * llm_tokens[b*llm_row_stride + unpacker[b,i,k]], which skips the unpack of the logits.
 * Outputs (batch,): n_tokens_in_seq, seq_in_beam (first beam with the longest match), and
 * optionally next_token = llm[b, seq, n] and last_slot = the index of that position (packed slot
 * when unpacker is given, else seq*length+n) for gathering the drafter context.
 * ------------------------------------------------------------------------------------------ */
RD_API int rd_accept_greedy(const int64_t* beams, const int64_t* llm_tokens, int64_t llm_row_stride,
                            const int64_t* unpacker, int batch, int width, int length,
                            int64_t* n_tokens_in_seq, int64_t* seq_in_beam, int64_t* next_token,
                            int64_t* last_slot, void* stream);

/* Leading pad run per row.  Replaces _count_left_paddings (recurrent_drafting.py:387-388). */
RD_API int rd_count_left_paddings(const int64_t* input_ids, int64_t ids_row_stride, int64_t prev,
                                  int batch, int64_t pad_token_id, int32_t* pads, void* stream);
/* rd_position_ids: position_ids[b, t] = (prev - leading pads of row b) + position_offsets[b, t],
 * contiguous (batch, n) int64: the position rule of the verification forward
 * (recurrent_drafting.py:449-458) with the pad count folded in. */
RD_API int rd_position_ids(const int64_t* input_ids, int64_t ids_row_stride, int64_t prev,
                           int batch, int64_t pad_token_id, const int64_t* position_offsets,
                           int64_t offsets_row_stride, int n, int64_t* position_ids,
                           void* stream);

/* ------------------------------------------------------------------------------------------
 * Token ids after acceptance, right-aligned and left-padded, plus the per-row plan that
 * rd_kv_compact follows.  Replaces the integer half of _update_kv_cache_and_input_ids
 * (recurrent_drafting.py:163-171, :211-226).
 *
 * plan: rd_realign_plan_ints(batch, length) int32: [0] = new length M (max over rows), [1] = prev,
 * [2] = length, [3] = 0, then per row {old_pads, new_pads, n_new, live_len, src_row[length]} where
 * src_row[j] is the cache row holding accepted token j: prev + seq*length + j when unpacker is
 * NULL (cache already unpacked by rd_kv_unpack), prev + unpacker[b,seq,j] otherwise.
 * new_ids: capacity batch*(prev+length), written as a contiguous (batch, M) array.
 * kv_row_shift (batch int32 on the device, read and written, or NULL): with it the cache is not
 * re-aligned.  Token column c of row b is taken to live in cache row c - kv_row_shift[b]; the plan
 * is written in cache rows with old_pads == new_pads (rd_kv_compact then only appends the accepted
 * rows behind the live ones) and kv_row_shift[b] grows by new_pads - old_pads.  The reference moves
 * the whole live cache on every step (recurrent_drafting.py:200-209); the same array is handed to
 * rd_rope_append and rd_attn_prepare, and rd_kv_materialize moves the rows once when the
 * reference's layout is wanted.
 * left_pads (batch int32 on the device, or NULL): the leading pad run of every row of input_ids when
 * the caller has it already (rd_tree_attn_prepare and rd_count_left_paddings write it); saves the
 * launch that counts them.
 * step_out (2 int32 on the device, or NULL): receives the new length M and the number of accepted
 * tokens summed over the rows (what the reference's loop reports as avg_num_accepted * batch,
 * recurrent_drafting.py:691-697), so that a caller can fetch both with whatever else it reads.
 * ------------------------------------------------------------------------------------------ */
RD_API size_t rd_realign_plan_ints(int batch, int length);
RD_API int rd_realign_plan(const int64_t* input_ids, int64_t ids_row_stride, int64_t prev,
                           const int64_t* n_tokens_in_seq, const int64_t* seq_in_beam,
                           const int64_t* beams, const int64_t* unpacker, int batch, int width,
                           int length, int64_t pad_token_id, int32_t* plan, int64_t* new_ids,
                           int32_t* kv_row_shift, const int32_t* left_pads, int32_t* step_out,
                           void* stream);

/* ------------------------------------------------------------------------------------------
 * KV cache, shape (n_layers, 2, batch, n_heads, max_len, head_dim), rows of row_bytes bytes.
 *
 * rd_kv_unpack: cache[..., prev+t, :] = cache[..., prev+index[b,t], :] for t in [0, n_out), all
 * reads before any write.  Replaces Cache.unpack (kv_cache.py:58-98).  n_src = number of packed
 * rows present at [prev, prev+n_src).
 *
 * rd_kv_compact: in place, per (layer, k|v, row, head): live rows [old_pads, prev) move to
 * [new_pads, ...) and the accepted rows src_row[0..n_new) follow them.  Replaces the cache half of
 * _update_kv_cache_and_input_ids (recurrent_drafting.py:174-209).  Rows outside [new_pads, M) keep
 * stale data (the reference leaves other stale data there).
 * ------------------------------------------------------------------------------------------ */
RD_API int rd_kv_unpack(void* cache, int n_layers, int batch, int n_heads, int64_t max_len,
                        int64_t row_bytes, int64_t prev, const int64_t* index, int n_out, int n_src,
                        void* stream);
/* rd_kv_append: rd_kv_compact for plans in which no row moves (old_pads == new_pads for every row,
 * as rd_realign_plan writes them when it is given kv_row_shift): only the accepted rows are copied
 * behind the live ones.  length * row_bytes <= 4096. */
RD_API int rd_kv_append(void* cache, int n_layers, int batch, int n_heads, int64_t max_len,
                        int64_t row_bytes, int length, const int32_t* plan, void* stream);
/* rd_kv_materialize: undoes kv_row_shift (see rd_realign_plan): every row's cache rows move to
 * the place where column and cache row agree (columns [0, length)), and the shifts are cleared.
 * plan: rd_kv_materialize_plan_ints(batch) int32 of workspace.  No counterpart in the reference,
 * which keeps that layout at all times. */
RD_API size_t rd_kv_materialize_plan_ints(int batch);
RD_API int rd_kv_materialize(void* cache, int n_layers, int batch, int n_heads, int64_t max_len,
                             int64_t row_bytes, int64_t length, int32_t* kv_row_shift,
                             int32_t* plan, void* stream);
RD_API int rd_kv_compact(void* cache, int n_layers, int batch, int n_heads, int64_t max_len,
                         int64_t row_bytes, int64_t prev, int length, const int32_t* plan,
                         void* stream);

/* ------------------------------------------------------------------------------------------
 * Elementwise chains of the decoder layer around the projections, one pass each.
 *
 * rd_add_rms_norm: h = x + delta when delta is given (the "hidden_states += ..." of
 * modeling_llama.py:196, :198; h is written to h_out, which may be x), else h = x;
 * y = weight * cast(h * rsqrt(mean(h^2) + eps)) with float32 statistics (LlamaRMSNorm.forward,
 * modeling_llama.py:27-32).  Rows of `cols` contiguous elements, row strides in elements.
 *
 * rd_silu_mul: y = silu(gate) * up (LlamaMLP.forward, modeling_llama.py:84-85, for
 * hidden_act "silu"); gate and up are row-strided views, e.g. the halves of one fused projection.
 * ------------------------------------------------------------------------------------------ */
RD_API int rd_add_rms_norm(const void* x, int64_t x_row_stride, const void* delta,
                           int64_t delta_row_stride, const void* weight, void* y,
                           int64_t y_row_stride, void* h_out, int64_t h_row_stride, int dtype,
                           int64_t rows, int cols, float eps, void* stream);
RD_API int rd_silu_mul(const void* gate, const void* up, int64_t in_row_stride, void* y,
                       int64_t y_row_stride, int dtype, int64_t rows, int cols, void* stream);
/* The elementwise steps between the GEMMs of the drafter head, one launch each.
 * mode 0: y = x + silu(z), ResBlock.forward (modeling_drafter.py:38-39);
 * mode 1: y = silu(x + z), the recurrent state update (modeling_drafter.py:192-197).
 * y2 (optional) receives the same values, e.g. the state's half of the [context, state] tensor
 * that upstream builds with torch.cat (modeling_drafter.py:199).  (rows, cols) with element row
 * strides, cols contiguous; every intermediate is rounded to dtype as the separate torch kernels
 * round it. */
RD_API int rd_silu_add(const void* x, int64_t x_row_stride, const void* z, int64_t z_row_stride,
                       void* y, int64_t y_row_stride, void* y2, int64_t y2_row_stride, int mode,
                       int dtype, int64_t rows, int cols, void* stream);

/* ------------------------------------------------------------------------------------------
 * Rotary position embedding of the new queries and keys, fused with the in-place append of the
 * new keys and values to one layer's cache slabs.  Replaces apply_rotary_pos_emb
 * (modeling_llama.py:87-110) and the two View.cat calls (modeling_llama.py:148-159,
 * kv_cache.py:24-32).
 *
 * q (batch, n_new, n_heads, head_dim), k and v (batch, n_new, n_kv_heads, head_dim): head_dim
 * contiguous, heads head_dim apart, *_strides = {batch, token} element strides.  cos/sin: tables
 * (table_rows, head_dim) in the same dtype, row p = the angles of position p (halves repeated,
 * NeoX layout).  position_ids (batch, n_new) int64, clamped to the table.  q_out: same layout as q
 * (may be q itself).  k_cache / v_cache: (batch, n_kv_heads, max_len, head_dim) slabs with element
 * strides cache_strides = {batch, head, row}; rows [row0, row0 + n_new) are written.
 * Every product and the sum are rounded to dtype, as the separate torch kernels round them.
 *
 * row_start (batch + 1 int32 on the device, or NULL): packed token rows.  The reference runs the
 * model on (batch, n_new) slots of which a row's trailing ones are padding whose results nobody
 * reads (tree_attention.py:70-122 fills them with other rows' tokens).  With row_start, token t of
 * batch row b is row row_start[b] + t of q, k, v and q_out (token stride; the batch strides are
 * unused) and exists only for t < row_start[b+1] - row_start[b]; position_ids stay (batch, n_new);
 * the cache rows of the slots that do not exist are not written.
 * kv_row_shift (batch int32 on the device, or NULL): token t of row b goes to cache row
 * row0 + t - kv_row_shift[b] (see rd_realign_plan); a row outside [0, max_len) is not written.
 * ------------------------------------------------------------------------------------------ */
RD_API int rd_rope_append(const void* q, const int64_t* q_strides, const void* k,
                          const int64_t* k_strides, const void* v, const int64_t* v_strides,
                          int dtype, int batch, int n_new, int n_heads, int n_kv_heads,
                          int head_dim, const void* cos, const void* sin, int64_t table_rows,
                          const int64_t* position_ids, int64_t pos_batch_stride, void* q_out,
                          const int64_t* q_out_strides, void* k_cache, void* v_cache,
                          const int64_t* cache_strides, int64_t row0, int64_t max_len,
                          const int32_t* row_start, const int32_t* kv_row_shift, void* stream);

/* ------------------------------------------------------------------------------------------
 * Verification attention.
 *
 * rd_attn_prepare: once per LLM forward (where the reference builds the additive bias,
 * modeling_llama.py:228 / attention.py:75-88).  Compresses the bool mask (batch, n_q, kv_len),
 * given as 0/1 bytes with element strides mask_stride_b / mask_stride_q (keys contiguous), into
 * bits: rd_attn_bits_words() uint64, one word per (row, 64 keys); and writes the work plan
 * (rd_attn_plan_ints() int32): per batch row the first key any query attends to and the split of
 * its keys into work items; n_heads (query heads of the attention that will use the plan) sizes
 * the items to one compute unit's share of the whole call.  fix_empty_rows != 0 turns a row that attends to nothing into a row
 * that attends to everything, which is what attention.set_sdpa_fully_masked_rows
 * (attention.py:58-72) does and what a finite-minimum additive bias amounts to.
 * Limits: batch <= 2048 (rd_tree_attn_prepare: 1024), batch * ceil(kv_len / 512) <= 32768.
 *
 * rd_verify_attention: out = softmax(q k^T * scale, masked) v per (batch row, head).  Replaces
 * repeat_interleave + F.scaled_dot_product_attention(attn_mask=bias) (modeling_llama.py:161-169).
 * q (batch, n_heads, n_q, head_dim), k/v (batch, n_kv_heads, kv_len, head_dim) and out
 * (batch, n_heads, n_q, head_dim) are addressed through HOST arrays of three element strides
 * {batch, head, sequence}; the last dimension is contiguous.  k and v are normally the strided
 * views View.cat returns (kv_cache.py:24-31).  bf16 with head_dim 128 runs on the MFMA kernel
 * (needs 16-byte aligned q/k/v, strides that are multiples of 8 elements, and the workspace);
 * everything else (more than 128 heads included), or force_generic != 0, runs on the generic
 * kernel (head_dim <= 256).  The plan and the bits are only read, so any number of calls, on any
 * streams, may share them.  Rows whose keys are split over several work items are merged by the
 * item that finishes last; the arrival counters for that are the library's (a ring of 2^18 per
 * GPU, of which every call takes batch * n_heads * ceil(n_q / rows per work group) for itself,
 * RD_ELIMIT beyond the ring) and leaves at zero, so calls that are in flight together do not meet
 * on a counter; each call needs a workspace of its own while it runs.  The first MFMA-path call on
 * a device looks the ring's address up (hipGetSymbolAddress): make it before a graph capture
 * begins.  K and V are addressed with 32-bit byte offsets inside a batch row's slab: shapes with
 * (kv_len + 128) * row stride in bytes >= 2^31 run on the generic kernel.
 * row_start (batch + 1 int32 on the device, or NULL): packed query rows, as in rd_rope_append:
 * query t of batch row b is row row_start[b] + t of q and of out (sequence stride; their batch
 * strides are unused), queries t >= row_start[b+1] - row_start[b] are neither read nor written.
 * The mask bits keep their (batch, n_q) rows.
 * kv_row_shift (rd_attn_prepare; batch int32 on the device, or NULL): recorded in the plan; the
 * attention then reads key column c of row b from cache row c - kv_row_shift[b] of k and v (see
 * rd_realign_plan).  Only cache rows of keys that some query of the row attends to are read (the
 * other keys of the first and last 64-key tile of a row count as zeros, which their zero
 * probabilities multiply), so nothing is asked of the memory around a row's live cache rows.
 * ------------------------------------------------------------------------------------------ */
RD_API size_t rd_attn_plan_ints(int batch, int n_q, int kv_len);
RD_API size_t rd_attn_bits_words(int batch, int n_q, int kv_len);
RD_API int rd_attn_prepare(const uint8_t* mask, int64_t mask_stride_b, int64_t mask_stride_q,
                           int batch, int n_q, int kv_len, int n_heads, int fix_empty_rows,
                           uint64_t* bits, int32_t* plan, const int32_t* kv_row_shift,
                           void* stream);
/* rd_tree_attn_prepare: for the packed tree of a verification step, what rd_tree_mask, rd_attn_prepare
 * and rd_position_ids produce one after the other -- the mask as bits, the plan, the position ids --
 * in one launch and without the (batch, n, prev + n) byte mask in between.  Replaces, for a caller
 * that goes straight to rd_verify_attention, tree_attention._get_causal_mask (tree_attention.py:191-298),
 * the row slice (:337), attention.bias (attention.py:75-88, called at modeling_llama.py:228) and the
 * position rule (recurrent_drafting.py:449-458).  unpacker, packed_token_indices, counts: as written
 * by rd_tree_build; n = counts[batch], the packed length (the caller has read it); padding_mask,
 * pm_elem_bytes, pm_row_stride, pm_pad_value, prev: as for rd_tree_mask.  bits: rd_attn_bits_words(
 * batch, n, prev + n) words, bit-identical to rd_attn_prepare on rd_tree_mask's output; plan:
 * rd_attn_plan_ints(batch, n, prev + n) ints.  position_ids (batch, n) int64 and left_pads (batch
 * int32: leading padding keys of every row; rd_realign_plan takes it) are optional.  prev <= 131072. */
RD_API int rd_tree_attn_prepare(const int64_t* unpacker, const int64_t* packed_token_indices,
                                const int32_t* counts, const void* padding_mask, int pm_elem_bytes,
                                int64_t pm_row_stride, int64_t pm_pad_value, int64_t prev, int batch,
                                int width, int length, int n, int n_heads, uint64_t* bits,
                                int32_t* plan, int64_t* position_ids, int32_t* left_pads,
                                const int32_t* kv_row_shift, void* stream);
RD_API size_t rd_attention_workspace_bytes(int batch, int n_heads, int n_q, int kv_len,
                                           int head_dim);
RD_API int rd_verify_attention(const void* q, const int64_t* q_strides, const void* k,
                               const int64_t* k_strides, const void* v, const int64_t* v_strides,
                               void* out, const int64_t* o_strides, int dtype, int batch,
                               int n_heads, int n_kv_heads, int n_q, int kv_len, int head_dim,
                               float scale, const uint64_t* bits, const int32_t* plan,
                               void* workspace, size_t workspace_bytes, int force_generic,
                               const int32_t* row_start, void* stream);
/* rd_rope_verify_attention: rd_rope_append followed by rd_verify_attention for the new tokens of one
 * layer, as ONE launch: modeling_llama.py:148-159 (rotation, kv_cache.py:24-32 append) and :161-169
 * (attention).  The attention kernel rotates its query rows in registers (q itself is left as it
 * was) and writes the rotated new keys and the new values to their cache rows before it reads them,
 * so the separate rotation kernel and its pass over q, k and v go away.  Output and cache hold the
 * same bits as after the two calls.
 * q (batch, n_heads, n_q, head_dim) through q_strides {batch, head, token}; k_new, v_new
 * (batch, n_q, n_kv_heads, head_dim) with heads head_dim apart, *_new_strides = {batch, token};
 * cos, sin, table_rows, position_ids, pos_batch_stride as for rd_rope_append; k_cache / v_cache
 * with cache_strides {batch, head, row} and max_len rows per slab; kv_len counts the cache rows
 * AFTER the append (new token t is key column kv_len - n_q + t); bits, plan (built for kv_len, with
 * the row shifts of the cache if it has any), workspace, row_start as for rd_verify_attention
 * (with row_start, k_new and v_new are packed like q and a row's missing tokens are not written).
 * Only bf16, head_dim 128, n_q <= 256, 16-byte aligned operands: rd_rope_verify_attention_eligible
 * says whether a shape qualifies, and a call that does not fails with RD_ELIMIT and enqueues
 * nothing (use the two calls then). */
RD_API int rd_rope_verify_attention_eligible(int dtype, int n_heads, int head_dim, int n_q);
RD_API int rd_rope_verify_attention(const void* q, const int64_t* q_strides, const void* k_new,
                                    const int64_t* k_new_strides, const void* v_new,
                                    const int64_t* v_new_strides, const void* cos, const void* sin,
                                    int64_t table_rows, const int64_t* position_ids,
                                    int64_t pos_batch_stride, void* k_cache, void* v_cache,
                                    const int64_t* cache_strides, int64_t max_len, void* out,
                                    const int64_t* o_strides, int dtype, int batch, int n_heads,
                                    int n_kv_heads, int n_q, int kv_len, int head_dim, float scale,
                                    const uint64_t* bits, const int32_t* plan, void* workspace,
                                    size_t workspace_bytes, const int32_t* row_start, void* stream);

/* ------------------------------------------------------------------------------------------
 * Causal mask from a padding mask: mask[b,i,j] = (j <= kv_len - query_len + i) && padding[b,j].
 * Replaces attention.causal_mask (attention.py:12-55) without the (kv_len, kv_len) temporary.
 * padding_mask as in rd_tree_mask; mask is (batch, query_len, kv_len) 0/1 bytes, contiguous.
 * ------------------------------------------------------------------------------------------ */
RD_API int rd_causal_mask(const void* padding_mask, int pm_elem_bytes, int64_t pm_row_stride,
                          int batch, int64_t kv_len, int64_t query_len, uint8_t* mask,
                          void* stream);

/* ------------------------------------------------------------------------------------------
 * One beam-search iteration after the drafter's lm_head GEMM.
 * Replaces maintain_logits (modeling_drafter.py:63-77), warp_logits (:80-99), log_softmax,
 * the beam-score add, torch.topk over width*vocab, % and // (:201-215), and the beams gather +
 * cat (:218-220).  Equal scores are ordered by the lower flat index beam*vocab + token
 * (torch.topk leaves that order unspecified).
 *
 * logits (batch*width, vocab) of `dtype`, row stride in elements, rows 16-byte aligned.
 * log_p_beam (batch,width) f32: running beam scores.  top_k / mask_value: 50 / -50000 upstream.
 * Outputs: new_log_p_beam (batch,width) f32 sorted descending, tokens and parents (batch,width).
 * beams_out (batch,width,t_len+1), optional: beams_in (batch,width,t_len) gathered by parent with
 * the new token appended.  logp_out, optional: (batch*width, vocab) f32 log-probabilities of the
 * new token under each INPUT beam (rounded through `dtype` as upstream), row stride in elements.
 * Limits: width <= 64, vocab <= 65536, top_k <= 512.  force_fallback != 0 runs the slow exact
 * path that otherwise only serves rows with very many tied logits.
 * Row (b, w) of the logits starts at logits + b*batch_stride + w*row_stride elements; batch_stride 0
 * stands for width*row_stride, and row_stride 0 (with a batch stride) lets every beam of a batch
 * row read the same logits -- the first iteration, in which all beams are copies of one.
 * ------------------------------------------------------------------------------------------ */
RD_API size_t rd_beam_topk_workspace_bytes(int batch, int width);
RD_API int rd_beam_topk(const void* logits, int dtype, int64_t row_stride, int64_t batch_stride,
                        int batch, int width, int vocab, const float* log_p_beam, int top_k, float mask_value,
                        const int64_t* beams_in, int t_len, float* new_log_p_beam, int64_t* tokens,
                        int64_t* parents, int64_t* beams_out, float* logp_out,
                        int64_t logp_row_stride, void* workspace, size_t workspace_bytes,
                        int force_fallback, void* stream);

/* rd_beam_init: the state a beam search starts from (modeling_drafter.py:170-189), in one launch
 * where the reference runs a fill, a slice assignment, two broadcasts and a zeros: log_p_beam
 * (batch, width) float32 = 0 for beam 0 and mask_value for the others; beams (batch, width) int64 =
 * the row's init token; head_in[b, w, 0 : hidden_bytes) = prompt_state[b] (the context half of the
 * [context, state] input of the head, modeling_drafter.py:199; rows head_in_row_bytes apart, the
 * state half is left alone); state (batch, state_rows, hidden_bytes), state_rows <= width: zeros.
 * Bytes are copied as they are, whatever the dtype; rows and strides are multiples of 16 bytes and
 * 16-byte aligned. */
RD_API int rd_beam_init(const void* prompt_state, int64_t ps_row_bytes, const int64_t* init_token,
                        int batch, int width, int64_t hidden_bytes, float mask_value,
                        float* log_p_beam, int64_t* beams, void* head_in, int64_t head_in_row_bytes,
                        void* state, int state_rows, void* stream);

/* rd_beam_topk_static: rd_beam_topk without the workspace argument, for callers that cannot
 * allocate device memory -- code under HIP graph capture, serving loops and harnesses that forbid
 * hipMalloc.  (No counterpart in the reference.)  The candidate lists that rd_beam_topk keeps in the
 * caller's workspace live in a 2 MiB device array that is part of the library, one copy per GPU; the
 * call allocates and frees nothing.  Limits: batch * width <= 4096 and width <= 64, beyond which the
 * call fails with RD_ELIMIT and enqueues nothing.  Every call on a GPU uses that GPU's one array:
 * calls that overlap in time on one GPU (two streams, two threads) race; calls on one stream do
 * not.  The first call on a device looks the array's address up (hipGetSymbolAddress); make it
 * before a graph capture begins. */
RD_API int rd_beam_topk_static(const void* logits, int dtype, int64_t row_stride, int64_t batch_stride,
                               int batch, int width, int vocab, const float* log_p_beam, int top_k,
                               float mask_value, const int64_t* beams_in, int t_len,
                               float* new_log_p_beam, int64_t* tokens, int64_t* parents,
                               int64_t* beams_out, float* logp_out, int64_t logp_row_stride,
                               int force_fallback, void* stream);

/* ------------------------------------------------------------------------------------------
 * Speculative-sampling acceptance.
 *
 * rd_verify_row_stats: per row of (rows, vocab) verify logits, the four floats from which the
 * log-probability of any token follows: {thr, zmax, log_sum, mask_z} with thr the top_k-th largest
 * logit, and zmax / log_sum / mask_z the maximum, log-sum-exp and filter value of
 * z = (logit >= thr ? logit : mask_value) / temperature, all in float32:
 *     log P(token) = (logit >= thr ? logit / T : mask_z) - zmax - log_sum.
 * Replaces warp_logits on the verify logits (recurrent_drafting.py:460) and
 * (logits / T).log_softmax (:86) without writing either tensor.  stats: rows * 4 floats.
 *
 * Both functions below take log P either as a dense float32 tensor (log_p_dense with HOST element
 * strides {batch, beam, position}, vocabulary contiguous; shape (batch, width, length, vocab)) or,
 * with log_p_dense == NULL, as packed logits (batch, n_rows, vocab) of `dtype` with HOST strides
 * {batch, row} + stats + unpacker.  log_q is the drafter's (batch, width, length-1, vocab) float32
 * tensor with HOST strides {batch, beam, position}.
 *
 * rd_accept_sample: token k+1 of a beam is accepted when uniforms[b,i,k] < exp(P - Q) at that
 * token; n = leading accepted run; first beam with the longest run.  Replaces
 * _choose_from_candidates (recurrent_drafting.py:499-556); the caller draws the uniforms
 * (torch.rand upstream, :545-547).
 *
 * rd_residual_probs: probs (batch, vocab) f32 = relu(exp P - exp Q) at position n of the chosen
 * beam, or exp P at position length-1 when n == length-1.  Replaces the arithmetic of
 * _prepare_next_input (recurrent_drafting.py:304-339); the draw itself stays with the caller.
 * ------------------------------------------------------------------------------------------ */
RD_API int rd_verify_row_stats(const void* logits, int dtype, int64_t row_stride, int64_t rows,
                               int vocab, int top_k, float mask_value, float temperature,
                               float* stats, int force_fallback, void* stream);
RD_API int rd_accept_sample(const int64_t* beams, const float* log_p_dense,
                            const int64_t* log_p_strides, const void* logits, int dtype,
                            const int64_t* logits_strides, const float* stats, int n_rows,
                            const int64_t* unpacker, float temperature, const float* log_q,
                            const int64_t* log_q_strides, const float* uniforms, int batch,
                            int width, int length, int vocab, int64_t* n_tokens_in_seq,
                            int64_t* seq_in_beam, void* stream);
RD_API int rd_residual_probs(const float* log_p_dense, const int64_t* log_p_strides,
                             const void* logits, int dtype, const int64_t* logits_strides,
                             const float* stats, int n_rows, const int64_t* unpacker,
                             float temperature, const float* log_q, const int64_t* log_q_strides,
                             const int64_t* seq_in_beam, const int64_t* n_tokens_in_seq, int batch,
                             int width, int length, int vocab, float* probs, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* REDRAFTER_HIP_H_ */
