"""Oracle (test infrastructure, never shipped): beams -> prefix tree -> packed tokens -> tree mask.

Restates, on NumPy int64 arrays, what recurrent_drafting/tree_attention.py and
recurrent_drafting/attention.py compute.  Two flavours per function where it helps:
`*_loops` is a literal brute-force definition for tiny inputs, the un-suffixed one is array code
that finishes in seconds at full benchmark sizes.  tests/test_oracle_tree.py checks the two against
each other, against every literal of the reference's own tests (tests/golden/reference_literals.json)
and against exhaustive enumeration of small beams.

Pin status
  dedup_prefix      pinned: PREFIX_TREE literal (tree_attention_test.py:19-24), doc example
                    (docs/beam_to_prefix_tree.md:8-14,86-90), exhaustive brute force W<=3,L<=3
  unpacker          pinned: UNPACKER literal (tree_attention_test.py:40-45), closed form, invariant
                    packed[unpacker]==beams (docs/tree_attention.md:174)
  pack_beams        pinned: PACKED_BEAMS / PACKED_TOKEN_INDICES literals incl. spill-over padding
                    (tree_attention_test.py:26-38); >=3-row spill-over and last-row clamp pinned by
                    vectors in tests/golden/reference_vectors.json
  tree_mask / pack  pinned: four literal masks (tree_attention_test.py:58-225), two more
                    (mlx/tree_attention_test.py:11-63), ancestor-set invariant
  causal_mask, bias, fully_masked_rows   pinned: literals attention_test.py:13-156
"""

from __future__ import annotations

import numpy as np

I64 = np.int64


# --------------------------------------------------------------------------------------------
# prefix dedup  (tree_attention.py:14-38)
# --------------------------------------------------------------------------------------------
def dedup_prefix_loops(beams: np.ndarray) -> np.ndarray:
    """prefix_tree[b,i,k] = smallest j whose first k+1 tokens equal beam i's first k+1 tokens.

    Literal definition (tree_attention.py:23-25, :34-37: argmax over j of an int 0/1 tensor
    returns the first j that matches)."""
    B, W, L = beams.shape
    out = np.zeros((B, W, L), dtype=I64)
    for b in range(B):
        for i in range(W):
            for k in range(L):
                for j in range(W):
                    if np.array_equal(beams[b, j, : k + 1], beams[b, i, : k + 1]):
                        out[b, i, k] = j
                        break
    return out


def dedup_prefix(beams: np.ndarray) -> np.ndarray:
    """Array form of dedup_prefix_loops: running AND of token equality along k, first true j."""
    beams = np.asarray(beams)
    eq = beams[:, :, None, :] == beams[:, None, :, :]  # [b, i, j, k]
    prefix_eq = np.logical_and.accumulate(eq, axis=3)
    return np.argmax(prefix_eq, axis=2).astype(I64)  # first True along j


# --------------------------------------------------------------------------------------------
# unpacker  (tree_attention.py:125-188)
# --------------------------------------------------------------------------------------------
def unpacker_loops(prefix_tree: np.ndarray) -> np.ndarray:
    """segment start of the owning beam + number of earlier positions in the same segment.

    Follows the two steps of tree_attention.py:142-188 literally."""
    B, W, L = prefix_tree.shape
    out = np.zeros((B, W, L), dtype=I64)
    for b in range(B):
        owned = [sum(1 for k in range(L) if prefix_tree[b, i, k] == i) for i in range(W)]
        start = [sum(owned[:i]) for i in range(W)]
        for i in range(W):
            seg = [start[prefix_tree[b, i, k]] for k in range(L)]
            for k in range(L):
                off = sum(1 for k2 in range(k) if seg[k2] == seg[k])
                out[b, i, k] = seg[k] + off
    return out


def unpacker(prefix_tree: np.ndarray) -> np.ndarray:
    B, W, L = prefix_tree.shape
    own = prefix_tree == np.arange(W, dtype=I64)[None, :, None]
    n_own = own.sum(axis=2)
    start = np.cumsum(n_own, axis=1) - n_own
    seg = np.take_along_axis(start, prefix_tree.reshape(B, W * L), axis=1).reshape(B, W, L)
    same = seg[:, :, :, None] == seg[:, :, None, :]  # [b,i,k,k2]
    earlier = np.tril(np.ones((L, L), dtype=bool), k=-1)  # k2 < k
    return (seg + (same & earlier[None, None]).sum(axis=3)).astype(I64)


def unpacker_closed_form(prefix_tree: np.ndarray) -> np.ndarray:
    """Ownership is a suffix of each beam, so slot = start[p] + k - (L - n_p), p = owner."""
    B, W, L = prefix_tree.shape
    own = prefix_tree == np.arange(W, dtype=I64)[None, :, None]
    n_own = own.sum(axis=2)
    start = np.cumsum(n_own, axis=1) - n_own
    p = prefix_tree.reshape(B, W * L)
    k = np.tile(np.arange(L, dtype=I64), W)[None, :]
    s = np.take_along_axis(start, p, axis=1)
    n = np.take_along_axis(n_own, p, axis=1)
    return (s + k - (L - n)).reshape(B, W, L).astype(I64)


# --------------------------------------------------------------------------------------------
# pack  (tree_attention.py:41-122)
# --------------------------------------------------------------------------------------------
def pack_beams(beams: np.ndarray, prefix_tree: np.ndarray):
    """Returns (packed_tokens (B,max_n), packed_token_indices (B,max_n), n_selected (B,)).

    The selected tokens of the whole batch form ONE vector in row-major order
    (tree_attention.py:78-86); row b then reads max_n consecutive entries starting at its own
    offset, clamped to the vector's last element (:102-110).  Slots past a row's own count thus
    hold the following rows' first tokens -- the reference's tests pin that
    (tree_attention_test.py:26-38)."""
    B, W, L = beams.shape
    own = (prefix_tree == np.arange(W, dtype=I64)[None, :, None]).reshape(B, W * L)
    rows, cols = np.nonzero(own)  # row-major, like torch.nonzero
    flat_tokens = beams.reshape(B, W * L)[rows, cols]
    n_sel = own.sum(axis=1).astype(I64)
    max_n = int(n_sel.max())
    starts = np.cumsum(n_sel) - n_sel
    pick = starts[:, None] + np.arange(max_n, dtype=I64)[None, :]
    pick = np.minimum(pick, flat_tokens.shape[0] - 1)
    return flat_tokens[pick].astype(I64), cols[pick].astype(I64), n_sel


def pack_beams_loops(beams: np.ndarray, prefix_tree: np.ndarray):
    B, W, L = beams.shape
    toks, idxs, counts = [], [], []
    for b in range(B):
        c = 0
        for i in range(W):
            for k in range(L):
                if prefix_tree[b, i, k] == i:
                    toks.append(int(beams[b, i, k]))
                    idxs.append(i * L + k)
                    c += 1
        counts.append(c)
    max_n = max(counts)
    pt = np.zeros((B, max_n), dtype=I64)
    pi = np.zeros((B, max_n), dtype=I64)
    for b in range(B):
        s = sum(counts[:b])
        for n in range(max_n):
            g = min(s + n, len(toks) - 1)
            pt[b, n] = toks[g]
            pi[b, n] = idxs[g]
    return pt, pi, np.asarray(counts, dtype=I64)


# --------------------------------------------------------------------------------------------
# masks  (attention.py:12-88, tree_attention.py:191-298)
# --------------------------------------------------------------------------------------------
def causal_mask(padding_mask: np.ndarray, query_len: int) -> np.ndarray:
    """(B, kv) padding mask -> (B, query_len, kv) bool: lower triangle AND key-not-padding, last
    query_len rows (attention.py:46-55)."""
    padding_mask = np.asarray(padding_mask)
    assert query_len > 0
    B, kv = padding_mask.shape
    tri = np.tril(np.ones((kv, kv), dtype=bool))
    m = tri[None] & (padding_mask != 0)[:, None, :]
    return m[:, kv - query_len :, :]


def fully_masked_rows_to_true(mask: np.ndarray) -> np.ndarray:
    """A row with no True becomes all True (attention.py:58-72)."""
    m = np.asarray(mask) != 0
    dead = ~m.any(axis=-1, keepdims=True)
    return m | dead


def bias(mask: np.ndarray, dtype) -> np.ndarray:
    """0 where attended, finfo(dtype).min where not (attention.py:75-88)."""
    out = np.zeros(np.shape(mask), dtype=dtype)
    out[np.asarray(mask) == 0] = np.finfo(dtype).min
    return out


def tree_mask_of_packed(unpack: np.ndarray, packed_token_indices: np.ndarray) -> np.ndarray:
    """(B, n, n) bool.  Row n, whose source is beam i position k, is True exactly at the packed
    slots of beam i's positions 0..k (tree_attention.py:214-250).  Padding slots carry another
    row's source index and are evaluated against THIS row's unpacker."""
    B, W, L = unpack.shape
    n_sel = packed_token_indices.shape[1]
    out = np.zeros((B, n_sel, n_sel), dtype=bool)
    for b in range(B):
        for n in range(n_sel):
            f = int(packed_token_indices[b, n])
            i, k = divmod(f, L)
            for k2 in range(L):
                out[b, n, unpack[b, i, k2]] = k2 <= k
    return out


def full_mask(padding_mask: np.ndarray, unpack: np.ndarray, packed_token_indices: np.ndarray):
    """(B, prev+n, prev+n) bool square mask (tree_attention.py:253-298)."""
    padding_mask = np.asarray(padding_mask)
    B, prev = padding_mask.shape
    n_sel = packed_token_indices.shape[1]
    ext = np.concatenate([padding_mask != 0, np.ones((B, n_sel), dtype=bool)], axis=1)
    m = causal_mask(ext, prev + n_sel).copy()
    m[:, prev:, prev:] = tree_mask_of_packed(unpack, packed_token_indices)
    return m


def pack(beams: np.ndarray, padding_mask: np.ndarray):
    """tree_attention.pack (tree_attention.py:301-338).

    Returns (packed_tokens (B,n), unpacker (B,W,L), mask (B,n,prev+n) bool, position_offsets (B,n))
    plus, as a fifth element for tests, packed_token_indices."""
    beams = np.asarray(beams, dtype=I64)
    L = beams.shape[2]
    tree = dedup_prefix(beams)
    unp = unpacker(tree)
    ptok, pidx, _ = pack_beams(beams, tree)
    n = ptok.shape[1]
    mask = full_mask(padding_mask, unp, pidx)[:, -n:, :]
    return ptok, unp, mask, pidx % L, pidx


def unpack_rows(packed: np.ndarray, unpack: np.ndarray) -> np.ndarray:
    """(B, n, F) gathered to (B, W, L, F) (tree_attention.py:341-387)."""
    B, W, L = unpack.shape
    out = np.empty((B, W, L, packed.shape[2]), dtype=packed.dtype)
    for b in range(B):
        out[b] = packed[b][unpack[b]]
    return out


def count_left_paddings(tokens: np.ndarray, pad_token_id: int) -> np.ndarray:
    """Length of the leading run of pad ids per row (recurrent_drafting.py:387-388)."""
    is_pad = np.asarray(tokens) == pad_token_id
    return np.cumprod(is_pad, axis=-1).sum(axis=-1).astype(I64)


# --------------------------------------------------------------------------------------------
# synthetic draft beams with shared prefixes (benchmark input; not a reference function)
# --------------------------------------------------------------------------------------------
def synthetic_beams(batch: int, width: int, length: int, vocab: int = 32000, seed: int = 123,
                    p_copy: float = 0.6, zipf_s: float = 1.1, n_first: int = 4) -> np.ndarray:
    """Token 0 from `n_first` values; position k>=1 of beam i copies beam i-1's token at k with
    probability p_copy (beam 0 always draws), else draws Zipf(s) over the vocabulary."""
    rng = np.random.default_rng(seed)
    ranks = np.arange(1, vocab + 1, dtype=np.float64)
    pz = ranks ** (-zipf_s)
    pz /= pz.sum()
    beams = np.zeros((batch, width, length), dtype=I64)
    beams[:, :, 0] = rng.integers(0, n_first, size=(batch, width))
    draws = rng.choice(vocab, size=(batch, width, length), p=pz)
    copy = rng.random((batch, width, length)) < p_copy
    for i in range(width):
        for k in range(1, length):
            take = copy[:, i, k] & (i > 0)
            beams[:, i, k] = np.where(take, beams[:, i - 1, k] if i > 0 else 0, draws[:, i, k])
    return beams
