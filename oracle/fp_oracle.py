"""Oracle (test infrastructure, never shipped): the floating-point parts of the decode step.

  masked_attention      textbook softmax(Q K^T / sqrt(D) + bias) V in float64
                        (modeling_llama.py:161-169 with attention.py:75-88 as the bias)
  warp_logits           top-k filter of modeling_drafter.py:80-99
  maintain_logits       modeling_drafter.py:63-77
  beam_search_step      one iteration of the post-GEMM chain, modeling_drafter.py:201-230
  beam_search_chain     init state + L-1 iterations given a logits callback (:170-232)
  argmax_first          first maximal index (torch.argmax, recurrent_drafting.py:52)

The chain uses torch on the CPU because the reference's rounding points matter in bf16: logits are
rounded after the max subtraction, the mask value -50000 becomes -49920, log_softmax rounds its
output to the input dtype, and only the beam score is float32 (the running score is created as
float32 at modeling_drafter.py:170-172, and bf16 + fp32 promotes to fp32).

log_softmax of a 16-bit tensor is a library routine whose last bit depends on the device: torch's
GPU kernel forms x - (max + log(sum)) in float32 and rounds the result once, its CPU kernel rounds
max + log(sum) to the 16-bit type first and the difference again (31 % of the surviving entries of
a flat row end up one bf16 step away from the correctly rounded value).  The reference runs its
16-bit models on a GPU, so `log_softmax_rounded_once` below takes the GPU kernel's rule: float32
arithmetic, one rounding.  Pinned by a float64 computation rounded once
(tests/test_oracle_fp.py) and, on the GPU box, by torch's own GPU log_softmax on the same tensor
(tests/test_gpu_beam.py).

Tie rule.  torch.topk leaves the order of equal elements unspecified and equal scores are certain
here (every filtered entry of a row has the same score).  The oracle, like the HIP kernel, breaks
ties by the LOWEST flat index (beam * V + token); comparisons with any other implementation are on
tie-free inputs or as multisets, as the reference's own cross-check does
(mlx/modeling_drafter_test.py:116-134).

Pin status
  masked_attention   pinned: all-True mask == torch SDPA; one beam == is_causal SDPA; n_q=1 == decode
                     attention; fully masked row == mean of V (finite-min bias)
  warp/maintain      pinned: max becomes 0, <= k survivors without ties, shift invariance
  beam_search_step   pinned on tie-free inputs: W=1 is an argmax chain; one iteration from the
                     initial state == argsort of row 0; sets-not-order check; the reference's own
                     beams (tests/golden/reference_vectors.json), two cases at width 64, where
                     ties are certain after the first iteration but cannot reach the final beams.
                     The order of tied candidates inside an iteration: parity unpinned against
                     torch.topk's order (documented rule above instead)
"""

from __future__ import annotations

import numpy as np
import torch

LOG_0 = -50000.0
LOG_1 = 0.0


def masked_attention(q, k, v, mask) -> np.ndarray:
    """q (B,H,nq,D), k/v (B,Hkv,kv,D), mask (B,nq,kv) bool -> (B,H,nq,D) float64.

    Masked scores get the most negative finite value of the compute type rather than -inf, as the
    additive bias of attention.py:87-88 does; a row with no attended key therefore averages V.
    That is the reference's CPU behaviour.  On a GPU the reference rewrites such rows to all-True
    before building the bias (modeling_llama.py:264-265, attention.py:58-72): callers that model
    the GPU path pass tree_oracle.fully_masked_rows_to_true(mask) instead."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    mask = np.asarray(mask) != 0
    B, H, nq, D = q.shape
    groups = H // k.shape[1]
    k = np.repeat(k, groups, axis=1)
    v = np.repeat(v, groups, axis=1)
    s = np.einsum("bhqd,bhkd->bhqk", q, k) / np.sqrt(D)
    dead = ~mask.any(axis=-1)  # (B,nq)
    s = np.where(mask[:, None], s, -np.inf)
    s = np.where(dead[:, None, :, None], 0.0, s)
    s = s - s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=-1, keepdims=True)
    return np.einsum("bhqk,bhkd->bhqd", p, v)


def maintain_logits(x: torch.Tensor) -> torch.Tensor:
    return x - x.max(dim=-1, keepdim=True).values


def kth_largest(x: torch.Tensor, k: int) -> torch.Tensor:
    k = min(k, x.shape[-1])
    return torch.sort(x.float(), dim=-1, descending=True).values[..., k - 1 : k].to(x.dtype)


def warp_logits(x: torch.Tensor, top_k: int = 50, mask_value: float = LOG_0) -> torch.Tensor:
    """Entries below the k-th largest of their row become mask_value (rounded to x's dtype)."""
    thr = kth_largest(x, top_k)
    return torch.where(x < thr, torch.tensor(mask_value, dtype=x.dtype), x)


def log_softmax_rounded_once(x: torch.Tensor) -> torch.Tensor:
    """log_softmax over the last axis in float32, rounded once to x's dtype (torch's GPU kernel)."""
    return x.float().log_softmax(dim=-1).to(x.dtype)


def stable_topk(scores: torch.Tensor, k: int):
    """Top-k along the last dim, sorted descending, equal scores in increasing index order."""
    order = torch.sort(scores, dim=-1, descending=True, stable=True)
    return order.values[..., :k], order.indices[..., :k]


def beam_search_step(logits: torch.Tensor, log_p_beam: torch.Tensor):
    """logits (B,W,V) in the drafter's dtype, log_p_beam (B,W) float32.

    Returns (new_log_p_beam (B,W) f32 sorted descending, token (B,W) i64, parent (B,W) i64,
    log_p_new_token (B,W,V) in logits' dtype)."""
    B, W, V = logits.shape
    logp = log_softmax_rounded_once(warp_logits(maintain_logits(logits)))
    scores = logp + log_p_beam.unsqueeze(-1)  # promotes to float32
    top, idx = stable_topk(scores.reshape(B, W * V), W)
    return top, idx % V, idx // V, logp


def beam_search_chain(logits_fn, init_token: torch.Tensor, width: int, length: int, vocab: int):
    """Runs length-1 iterations.  logits_fn(beams (B,W,t) i64, parent (B,W) i64 or None) -> (B,W,V).

    Returns (beams (B,W,L) i64, log_probs (B,W,L-1,V) float32)."""
    B = init_token.shape[0]
    log_p_beam = torch.full((B, width), LOG_0, dtype=torch.float32)
    log_p_beam[:, 0] = LOG_1
    beams = init_token.view(B, 1, 1).repeat(1, width, 1)
    hist = torch.zeros((B, width, 0, vocab), dtype=torch.float32)
    parent = None
    rows = torch.arange(B).unsqueeze(-1)
    for _ in range(length - 1):
        logits = logits_fn(beams, parent)
        log_p_beam, tok, parent, logp = beam_search_step(logits, log_p_beam)
        beams = torch.cat([beams[rows, parent], tok.unsqueeze(-1)], dim=-1)
        hist = torch.cat([hist[rows, parent], logp[rows, parent].unsqueeze(2).float()], dim=2)
    return beams, hist


def argmax_first(x: np.ndarray) -> np.ndarray:
    """First index of the maximum along the last axis (np.argmax has torch.argmax's rule)."""
    return np.argmax(np.asarray(x), axis=-1).astype(np.int64)
