"""Pins oracle/fp_oracle.py against library routines, closed forms and special cases."""
import numpy as np
import torch
import torch.nn.functional as F

from oracle import fp_oracle as O
from oracle import tree_oracle as T


def _rand_qkv(B, H, Hkv, nq, kv, D, seed=0):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((B, H, nq, D)), rng.standard_normal((B, Hkv, kv, D)),
            rng.standard_normal((B, Hkv, kv, D)))


def test_all_true_mask_is_plain_sdpa():
    q, k, v = _rand_qkv(2, 4, 4, 5, 11, 16)
    got = O.masked_attention(q, k, v, np.ones((2, 5, 11), dtype=bool))
    want = F.scaled_dot_product_attention(torch.tensor(q), torch.tensor(k), torch.tensor(v)).numpy()
    assert np.allclose(got, want, atol=1e-12)


def test_single_beam_is_causal_attention():
    """A tree with one beam and no cached prefix is a causal mask."""
    L = 6
    beams = np.arange(L)[None, None, :]
    _, _, mask, _, _ = T.pack(beams, np.zeros((1, 0), dtype=np.int64))
    assert np.array_equal(mask[0], np.tril(np.ones((L, L), dtype=bool)))
    q, k, v = _rand_qkv(1, 2, 2, L, L, 8, seed=1)
    got = O.masked_attention(q, k, v, mask)
    want = F.scaled_dot_product_attention(torch.tensor(q), torch.tensor(k), torch.tensor(v), is_causal=True).numpy()
    assert np.allclose(got, want, atol=1e-12)


def test_one_query_is_decode_attention_with_padding_and_gqa():
    q, k, v = _rand_qkv(3, 4, 2, 1, 9, 8, seed=2)
    pm = np.array([[0, 0, 1, 1, 1, 1, 1, 1, 1], [1] * 9, [0, 1, 0, 1, 1, 0, 1, 1, 1]])
    mask = T.causal_mask(pm, 1)
    got = O.masked_attention(q, k, v, mask)
    for b in range(3):
        keep = pm[b] != 0
        for h in range(4):
            s = (k[b, h // 2][keep] @ q[b, h, 0]) / np.sqrt(8)
            p = np.exp(s - s.max()); p /= p.sum()
            assert np.allclose(got[b, h, 0], p @ v[b, h // 2][keep], atol=1e-12)


def test_fully_masked_row_averages_values_like_a_finite_min_bias():
    q, k, v = _rand_qkv(1, 1, 1, 2, 5, 4, seed=3)
    mask = np.array([[[0, 0, 0, 0, 0], [1, 1, 0, 0, 0]]], dtype=bool)
    got = O.masked_attention(q, k, v, mask)
    assert np.allclose(got[0, 0, 0], v[0, 0].mean(axis=0), atol=1e-12)
    bias = torch.tensor(T.bias(mask, np.float32))[:, None]
    want = F.scaled_dot_product_attention(torch.tensor(q).float(), torch.tensor(k).float(), torch.tensor(v).float(), attn_mask=bias)
    assert np.allclose(got, want.numpy(), atol=1e-5)


def test_maintain_and_warp_properties():
    torch.manual_seed(0)
    x = torch.randn(3, 4, 500)
    m = O.maintain_logits(x)
    assert torch.equal(m.max(dim=-1).values, torch.zeros(3, 4))
    w = O.warp_logits(m)
    assert ((w > O.LOG_0).sum(dim=-1) == 50).all()  # tie-free input: exactly k survivors
    assert torch.equal(w.max(dim=-1).values, torch.zeros(3, 4))
    # shift invariance of the whole chain
    a = O.warp_logits(O.maintain_logits(x)).log_softmax(-1)
    b = O.warp_logits(O.maintain_logits(x + 7.0)).log_softmax(-1)
    assert torch.allclose(a, b, atol=1e-5)
    assert torch.tensor(O.LOG_0, dtype=torch.bfloat16).item() == -49920.0


def test_beam_width_one_is_an_argmax_chain():
    torch.manual_seed(1)
    V, L = 64, 5
    table = torch.randn(V, V)  # logits depend on the last token only

    def logits_fn(beams, parent):
        return table[beams[..., -1]]

    beams, hist = O.beam_search_chain(logits_fn, torch.tensor([3, 9]), 1, L, V)
    for b, tok in enumerate([3, 9]):
        seq = [tok]
        for _ in range(L - 1):
            seq.append(int(table[seq[-1]].argmax()))
        assert beams[b, 0].tolist() == seq
    assert hist.shape == (2, 1, L - 1, V) and hist.dtype == torch.float32


def test_first_iteration_is_a_sort_of_row_zero():
    torch.manual_seed(2)
    B, W, V = 2, 6, 200
    logits = torch.randn(B, W, V)
    lpb = torch.full((B, W), O.LOG_0); lpb[:, 0] = O.LOG_1
    top, tok, parent, logp = O.beam_search_step(logits, lpb)
    assert (parent == 0).all()
    want = torch.argsort(logits[:, 0], dim=-1, descending=True)[:, :W]
    assert torch.equal(tok, want)
    assert torch.allclose(top, logp[:, 0].gather(1, want))
    assert (top[:, :-1] >= top[:, 1:]).all()


def test_stable_topk_prefers_the_lowest_index_among_ties():
    x = torch.tensor([[0.0, 1.0, 1.0, 1.0, 1.0, 0.5, 1.0]])
    v, i = O.stable_topk(x, 3)
    assert i.tolist() == [[1, 2, 3]] and v.tolist() == [[1.0, 1.0, 1.0]]


def test_beam_search_matches_reference_vectors(ref_vectors):
    """Tie-free float32 drafter of the reference: same beams and same log-probs at the drafted
    tokens as the reference's beam_search_candidates (torch.topk order is determined there)."""
    for c in ref_vectors["beam_search"]:
        W, L, V, hid = c["W"], c["L"], c["V"], c["hidden"]
        wt = {k: torch.tensor(v, dtype=torch.float32).reshape(c["weight_shapes"][k]) / c["weight_scale"]
              for k, v in c["weights_x64"].items()}
        emb = torch.tensor(c["embedding_x64"], dtype=torch.float32).reshape(V, hid) / 64
        ctx = torch.tensor(c["prompt_state_x64"], dtype=torch.float32).reshape(-1, hid) / 64
        B = ctx.shape[0]
        state = {"s": torch.zeros(B, W, hid)}

        def logits_fn(beams, parent):
            s = state["s"]
            if parent is not None:
                s = s[torch.arange(B).unsqueeze(-1), parent]
            s = F.silu(emb[beams[..., -1]] @ wt["rnn_w.weight"].T + s @ wt["rnn_u.weight"].T + wt["rnn_u.bias"])
            state["s"] = s
            x = torch.cat([ctx[:, None, :].expand(B, W, hid), s], dim=-1)
            x = x + F.silu(x @ wt["lm_head.0.linear.weight"].T + wt["lm_head.0.linear.bias"])
            return x @ wt["lm_head.1.weight"].T

        beams, hist = O.beam_search_chain(logits_fn, torch.tensor(c["init_token"]), W, L, V)
        assert beams.tolist() == c["beams"]
        picked = torch.gather(hist, 3, beams[:, :, 1:, None]).squeeze(-1)
        assert torch.allclose(picked, torch.tensor(c["log_prob_of_drafted"]), atol=1e-5)
        assert torch.allclose(hist.max(-1).values, torch.tensor(c["log_prob_row_max"]), atol=1e-5)
        assert torch.allclose(hist.min(-1).values, torch.tensor(c["log_prob_row_min"]), atol=1e-2)


def test_log_softmax_of_16_bit_rows_is_rounded_once():
    """The float64 value rounded once to bf16 / fp16 is what the oracle returns (torch's GPU rule);
    torch's CPU kernel for 16-bit types, which rounds max + log(sum) first, is up to a step away."""
    torch.manual_seed(0)
    for dtype in (torch.bfloat16, torch.float16):
        x = O.warp_logits(O.maintain_logits((torch.randn(6, 4000) * 0.05).to(dtype)))
        want = (x.double() - torch.logsumexp(x.double(), dim=-1, keepdim=True)).to(dtype)
        got = O.log_softmax_rounded_once(x)
        live = want.float() > -1000
        assert got.dtype == dtype and torch.equal(got[live], want[live])
        assert torch.allclose(got.float(), want.float(), rtol=1e-6, atol=0)  # (the filtered class: sums near 50000)
    x32 = torch.randn(3, 100)
    assert torch.equal(O.log_softmax_rounded_once(x32), x32.log_softmax(-1))
