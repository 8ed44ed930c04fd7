"""Comparison of one beam-search iteration with the oracle when scores may differ in their last
bits (bf16 log-probabilities: the logarithm of the row's sum is formed in another order, and a
score that is rounded to bf16 then moves by a whole bf16 step).

If every score of one implementation is within `tol` of the other's, then (1) the k-th best score
of the two differs by at most `tol`, and (2) a candidate that only one of them selects has a score
within 2 * tol of the other's cut (the W-th best score).  `check_selection` asserts exactly that,
for the selected (parent, token) pairs as sets, plus bit-equality wherever the scores agree
exactly.
"""

from __future__ import annotations

import torch


def check_selection(o_logp: torch.Tensor, log_p_beam: torch.Tensor, o_lpb: torch.Tensor, o_tok: torch.Tensor,
                    o_par: torch.Tensor, new_lpb: torch.Tensor, tok: torch.Tensor, par: torch.Tensor,
                    tol: float) -> float:
    """o_*: the oracle's log-probabilities (B, W, V), sorted scores, tokens, parents; the others the
    implementation's.  Returns the share of the implementation's picks that the oracle picked too."""
    B, W, V = o_logp.shape
    o_lpb, new_lpb = o_lpb.float().cpu(), new_lpb.float().cpu()
    assert (new_lpb[:, :-1] >= new_lpb[:, 1:]).all(), "scores not sorted"
    assert torch.allclose(new_lpb, o_lpb, atol=tol, rtol=0), (new_lpb - o_lpb).abs().max()
    got = (par.cpu() * V + tok.cpu())
    want = (o_par.cpu() * V + o_tok.cpu())
    if torch.equal(got, want):
        return 1.0
    flat = (o_logp.float().cpu() + log_p_beam.float().cpu()[:, :, None]).reshape(B, -1)
    shared = 0
    for b in range(B):
        g, w = set(got[b].tolist()), set(want[b].tolist())
        assert len(g) == W, f"row {b}: a candidate was selected twice"
        shared += len(g & w)
        cut = o_lpb[b, -1].item()
        for i in g ^ w:
            assert abs(flat[b, i].item() - cut) <= 2 * tol, \
                f"row {b}: candidate {i} (oracle score {flat[b, i].item()}) is not within {2 * tol} of the cut {cut}"
        # what both selected comes in the same order wherever the oracle's scores differ by more than 2 * tol
        common_got = [i for i in got[b].tolist() if i in w]
        common_want = [i for i in want[b].tolist() if i in g]
        for x, y in zip(common_got, common_want):
            assert x == y or abs(flat[b, x].item() - flat[b, y].item()) <= 2 * tol, (b, x, y)
    return shared / (B * W)
