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

/* Library version (major*10000 + minor*100 + patch). */
RD_API int rd_version(void);
/* Message of the last failed call on this thread ("" if none). */
RD_API const char* rd_last_error(void);

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
 * ------------------------------------------------------------------------------------------ */
RD_API size_t rd_tree_workspace_bytes(int batch, int width, int length);
RD_API int rd_tree_build(const int64_t* beams, int batch, int width, int length,
                  int64_t* prefix_tree, int64_t* unpacker,
                  int64_t* packed_tokens, int64_t* packed_token_indices,
                  int64_t* position_offsets, int32_t* counts,
                  void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * Tree attention mask, rows of the packed tokens only.
 * Replaces tree_attention._get_causal_mask_of_packed_beams (tree_attention.py:191-250),
 * _get_causal_mask (:253-298), attention.causal_mask on the extended padding mask
 * (attention.py:12-55) and the final row slice (tree_attention.py:337).
 *
 * padding_mask: (batch, prev) of pm_elem_bytes-wide integers (1, 4 or 8), row stride
 * pm_row_stride elements; non-zero = real token.  May be NULL when prev == 0.
 * mask: capacity batch*width*length*(prev+width*length) bytes, written as a contiguous
 * (batch, max_n, prev+max_n) array of 0/1 bytes with max_n = counts[batch].
 * ------------------------------------------------------------------------------------------ */
RD_API int rd_tree_mask(const int64_t* unpacker, const int64_t* packed_token_indices,
                 const int32_t* counts, const void* padding_mask, int pm_elem_bytes,
                 int64_t pm_row_stride, int64_t prev, int batch, int width, int length,
                 uint8_t* mask, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* REDRAFTER_HIP_H_ */
