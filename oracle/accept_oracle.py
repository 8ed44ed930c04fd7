"""Oracle (test infrastructure, never shipped): candidate acceptance and KV / ids re-alignment.

Restates the module-level functions of recurrent_drafting/recurrent_drafting.py and
recurrent_drafting/kv_cache.py with per-row Python loops over NumPy arrays.

Pin status
  greedy_choose          pinned: literal n=[3,1,0], beam=[0,1,0] (recurrent_drafting_test.py:34-69,
                         row 3 shows the first-maximum rule), maximality invariant
  greedy_next_input      pinned: property of recurrent_drafting_test.py:11-31
  sample_choose          pinned: brute-force leading-run count with injected uniforms, the recipe of
                         mlx/recurrent_drafting_test.py:176-204; degenerate p>=q accepts everything;
                         reference vectors of _choose_from_candidates under a recorded torch.rand
                         (tests/golden/reference_vectors.json, "choose_from_candidates")
  residual_probs         pinned: one-hot LLM distribution makes the draw deterministic
                         (mlx/recurrent_drafting_test.py:76-90); closed form relu(p-q); the probs the
                         reference's _prepare_next_input hands to Categorical ("prepare_next_input")
  kv_unpack              pinned: docstring example of Cache.unpack (kv_cache_test.py:38-93)
  update_kv_and_ids      pinned: docstring worked example (recurrent_drafting.py:142-160), live-region
                         invariant, and B>1 ragged vectors in tests/golden/reference_vectors.json
                         ("kv_update", and "accept_candidate_tokens" for the sampling caller)
"""

from __future__ import annotations

import numpy as np

from .tree_oracle import I64, count_left_paddings


def greedy_choose(beams_by_drafter: np.ndarray, beams_by_llm: np.ndarray):
    """(n_tokens_in_seq (B,), seq_in_beam (B,)): per beam, how many drafted tokens (positions 1..)
    equal the LLM's tokens (positions 0..) before the first mismatch; per row the FIRST beam that
    attains the maximum (recurrent_drafting.py:492-496; torch.max returns the first maximal index)."""
    B, W, L = beams_by_drafter.shape
    n_out = np.zeros(B, dtype=I64)
    s_out = np.zeros(B, dtype=I64)
    for b in range(B):
        best, arg = -1, 0
        for i in range(W):
            n = 0
            while n < L - 1 and beams_by_drafter[b, i, n + 1] == beams_by_llm[b, i, n]:
                n += 1
            if n > best:
                best, arg = n, i
        n_out[b], s_out[b] = best, arg
    return n_out, s_out


def greedy_next_input(beams_by_llm, hidden, seq_in_beam, n_tokens_in_seq):
    """(context (B,hid), next_token (B,)) picked at [b, s_b, n_b] (recurrent_drafting.py:261-268)."""
    B = beams_by_llm.shape[0]
    r = np.arange(B)
    return hidden[r, seq_in_beam, n_tokens_in_seq], beams_by_llm[r, seq_in_beam, n_tokens_in_seq]


def sample_choose(beams, log_p_llm, log_q_drafter, uniforms):
    """Speculative-sampling acceptance with the uniform draws supplied by the caller.

    beams (B,W,L); log_p_llm (B,W,L,V); log_q_drafter (B,W,L-1,V); uniforms (B,W,L-1).
    Token k+1 of a beam is accepted when u < exp(p - q) evaluated at that token
    (recurrent_drafting.py:532-547); n is the length of the leading accepted run (:551-555) and the
    first beam with the longest run wins (:556)."""
    B, W, L = beams.shape
    n_out = np.zeros(B, dtype=I64)
    s_out = np.zeros(B, dtype=I64)
    for b in range(B):
        best, arg = -1, 0
        for i in range(W):
            n = 0
            for k in range(L - 1):
                tok = beams[b, i, k + 1]
                ratio = np.exp(log_p_llm[b, i, k, tok] - log_q_drafter[b, i, k, tok])
                if uniforms[b, i, k] < ratio:
                    n += 1
                else:
                    break
            if n > best:
                best, arg = n, i
        n_out[b], s_out[b] = best, arg
    return n_out, s_out


def residual_probs(log_q_drafter, log_p_llm, seq_in_beam, n_tokens_in_seq):
    """Unnormalised distribution the next token is drawn from (recurrent_drafting.py:304-339):
    relu(P - Q) at the first rejected position, or P at the extra last position when the whole
    beam was accepted.  (B, V)."""
    B, W, Lm1, V = log_q_drafter.shape
    out = np.zeros((B, V), dtype=log_p_llm.dtype)
    for b in range(B):
        s, n = int(seq_in_beam[b]), int(n_tokens_in_seq[b])
        if n == Lm1:
            out[b] = np.exp(log_p_llm[b, s, Lm1])
        else:
            d = np.exp(log_p_llm[b, s, n]) - np.exp(log_q_drafter[b, s, n])
            out[b] = np.maximum(d, 0)
    return out


def kv_unpack(cache: np.ndarray, prompt_length: int, unpack: np.ndarray) -> None:
    """In place on cache (layers,2,B,H,max_len,D): slot prompt_length+t takes the row that sat at
    prompt_length+unpack_flat[b,t], t in [0, W*L) (kv_cache.py:86-95).  Reads use the state before
    the call."""
    B, W, L = unpack.shape
    src = cache.copy()
    for b in range(B):
        flat = unpack[b].reshape(-1)
        for t in range(W * L):
            cache[:, :, b, :, prompt_length + t, :] = src[:, :, b, :, prompt_length + flat[t], :]


def update_kv_and_ids(input_ids, n_tokens_in_seq, seq_in_beam, beams, cache, pad_token_id,
                      unpacked: bool = True, unpack: np.ndarray | None = None):
    """Append the accepted tokens and re-right-align every row (recurrent_drafting.py:163-232).

    cache: (layers,2,B,H,max_len,D) modified in place.  With unpacked=True the candidate rows of
    beam s sit at prev + s*L + j (the layout Cache.unpack leaves, recurrent_drafting.py:374-379,
    :186-198); with unpacked=False they are read from the packed slots prev + unpack[b,s,j].
    Returns (new_ids (B,M), M).  Positions outside [new_pads_b, M) keep whatever they held, except
    that [prev, prev+L) of every row first receives beam s's L rows (the `cat` at :197-198); the
    whole returned tensor therefore equals the reference's, stale regions included."""
    input_ids = np.asarray(input_ids)
    B, W, L = beams.shape
    prev = input_ids.shape[1]
    pads = count_left_paddings(input_ids, pad_token_id)
    n_new = np.asarray(n_tokens_in_seq, dtype=I64) + 1
    seq_len = prev - pads + n_new
    M = int(seq_len.max())
    new_pads = M - seq_len
    before = cache.copy()
    for b in range(B):
        s = int(seq_in_beam[b])
        # step 1: beam s's L candidate rows land at [prev, prev+L)
        staged = before[:, :, b].copy()  # (layers,2,H,max_len,D)
        for j in range(L):
            src = prev + (s * L + j if unpacked else int(unpack[b, s, j]))
            staged[:, :, :, prev + j, :] = before[:, :, b, :, src, :]
        cache[:, :, b, :, prev : prev + L, :] = staged[:, :, :, prev : prev + L, :]
        # step 2: shifted copy of [pads_b, prev+n_b+1) to [new_pads_b, M)
        start, end = int(pads[b]), prev + int(n_new[b])
        assert M - int(new_pads[b]) == end - start
        cache[:, :, b, :, int(new_pads[b]) : M, :] = staged[:, :, :, start:end, :]
    ids = np.full((B, M), pad_token_id, dtype=I64)
    for b in range(B):
        s = int(seq_in_beam[b])
        a = int(new_pads[b])
        e = a + prev - int(pads[b])
        ids[b, a:e] = input_ids[b, int(pads[b]) :]
        ids[b, e : e + int(n_new[b])] = beams[b, s, : int(n_new[b])]
    return ids, M
