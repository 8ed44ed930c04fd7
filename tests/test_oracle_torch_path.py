"""Pins oracle/torch_path.py (the torch restatement of the whole step) against the NumPy oracles,
the reference's literals/vectors and the reference's own end-to-end greedy token streams."""
import os
import sys

import numpy as np
import pytest
import torch

from oracle import accept_oracle as Acc
from oracle import fp_oracle as O
from oracle import torch_path as P
from oracle import tree_oracle as T

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "golden"))
import tiny_models as tm  # noqa: E402


def test_pack_matches_numpy_oracle_and_literals(literals):
    t = literals["tree"]
    for case in literals["pack_masks"]["cases"]:
        tok, unp, mask, off = P.pack(torch.tensor(t["beams"]), torch.tensor(case["padding_mask"]))
        assert tok.tolist() == t["packed_beams"] and unp.tolist() == t["unpacker"]
        assert mask.long().tolist() == case["mask"] and off.tolist() == t["position_offsets"]
    rng = np.random.default_rng(0)
    for B, W, L, prev in [(3, 5, 4, 6), (8, 45, 5, 20), (2, 7, 6, 0)]:
        beams = rng.integers(0, 3, size=(B, W, L))
        pm = (rng.random((B, prev)) > 0.2).astype(np.int64)
        tok, unp, mask, off = P.pack(torch.tensor(beams), torch.tensor(pm))
        o_tok, o_unp, o_mask, o_off, _ = T.pack(beams, pm)
        assert np.array_equal(tok.numpy(), o_tok) and np.array_equal(unp.numpy(), o_unp)
        assert np.array_equal(mask.numpy(), o_mask) and np.array_equal(off.numpy(), o_off)
        x = torch.rand(B, tok.shape[1], 3)
        assert np.array_equal(P.unpack(x, unp).numpy(), T.unpack_rows(x.numpy(), o_unp))


def test_masks(literals):
    for case in literals["causal_mask"]["cases"]:
        assert P.causal_mask(torch.tensor(case["padding_mask"]), case["query_len"]).long().tolist() == case["mask"]
    for case in literals["fully_masked_rows"]["cases"]:
        assert P.rows_without_keys_to_true(torch.tensor(case["mask"])).long().tolist() == case["expected"]


def test_cache_unpack_and_realign_reference_vectors(ref_vectors):
    for c in ref_vectors["kv_update"]:
        sh = c["shape"]
        cache = P.Cache(sh["B"], sh["max_len"], sh["layers"], sh["H"], sh["D"], torch.float32, "cpu")
        shape = tuple(cache.data.shape)
        cache.data.copy_(torch.tensor(c["cache_before"], dtype=torch.float32).reshape(shape))
        cache.unpack(sh["prev"], torch.tensor(c["unpacker"]))
        assert cache.data.flatten().long().tolist() == c["cache_after_unpack"]
        ids = P.realign(torch.tensor(c["input_ids"]), torch.tensor(c["n_tokens_in_seq"]),
                        torch.tensor(c["seq_in_beam"]), torch.tensor(c["beams"]), cache, 0)
        assert ids.tolist() == c["new_ids"] and cache.length[0][0] == c["new_length"]
        assert cache.data.flatten().long().tolist() == c["cache_after_update"]


def test_greedy_choose(literals):
    g = literals["greedy_choose"]
    n, s = P.greedy_choose(torch.tensor(g["beams_by_drafter"]), torch.tensor(g["beams_by_llm"]))
    assert n.tolist() == g["n_tokens_in_seq"] and s.tolist() == g["seq_in_beam"]
    rng = np.random.default_rng(1)
    d, m = rng.integers(0, 2, size=(5, 6, 7)), rng.integers(0, 2, size=(5, 6, 7))
    n, s = P.greedy_choose(torch.tensor(d), torch.tensor(m))
    on, os_ = Acc.greedy_choose(d, m)
    assert np.array_equal(n.numpy(), on) and np.array_equal(s.numpy(), os_)


def _models(llama_sd, drafter_sd, dtype=torch.float32):
    import recurrent_drafting_amd as rd
    from transformers.models.llama.configuration_llama import LlamaConfig

    llm = rd.modeling_llama.LlamaForCausalLM(LlamaConfig(**tm.LLAMA))
    drafter = rd.modeling_drafter.Drafter(rd.configuration_drafter.DrafterConfig(**tm.DRAFTER))
    llm.load_state_dict(llama_sd, strict=False)
    drafter.load_state_dict(drafter_sd)
    return llm.to(dtype).eval(), drafter.to(dtype).eval()


def test_beam_search_matches_chain_oracle():
    llm, drafter = _models(tm.draw(tm.llama_shapes(), 5), tm.draw(tm.drafter_shapes(), 6))
    torch.manual_seed(0)
    ctx = torch.randn(2, 128)
    tok = torch.tensor([17, 400])
    with torch.no_grad():
        beams, hist = P.beam_search(drafter, llm.model.embed_tokens, ctx, tok, 5, 4)
        state = {"s": torch.zeros(2, 5, 128)}

        def logits_fn(b, parent):
            s = state["s"] if parent is None else state["s"][torch.arange(2)[:, None], parent]
            s = torch.nn.functional.silu(drafter.rnn_w(llm.model.embed_tokens(b[..., -1])) + drafter.rnn_u(s))
            state["s"] = s
            return drafter.lm_head(torch.cat([ctx[:, None].expand(2, 5, 128), s], -1))

        o_beams, o_hist = O.beam_search_chain(logits_fn, tok, 5, 4, 1000)
    assert torch.equal(beams, o_beams) and torch.allclose(hist, o_hist, atol=1e-6)


@pytest.mark.parametrize("case_index", [0, 1, 2, 3, 4, 5, 6])
def test_generate_matches_reference_token_streams(ref_vectors, case_index):
    """The reference's own greedy decode loop (CPU, float32) produced these streams.  Cases 5 and 6
    have beams wider than the top-50 filter (64 x 5): the first beam-search iteration then ends in
    certain ties among filtered tokens, whose order torch.topk leaves open -- the streams must not
    depend on it (the tied beams are gone after the second iteration)."""
    case = ref_vectors["end_to_end"][case_index]
    c = case["config"]
    if c.get("markov"):
        llama_sd, drafter_sd = tm.markov(c["seed"])
    else:
        llama_sd, drafter_sd = tm.draw(tm.llama_shapes(), c["seed"]), tm.draw(tm.drafter_shapes(), c["seed"] + 1000)
    llm, drafter = _models(llama_sd, drafter_sd)
    ids = tm.prompt(c["batch"], c["prompt_len"], tm.LLAMA["vocab_size"], c["seed"], c["left_pads"])
    steps = [t.tolist() for t, _ in P.generate_greedy(
        llm, drafter, ids, c["prompt_len"] + c["new_tokens"], c["W"], c["L"], pad=0, eos=None)]
    assert steps == case["steps"]


@pytest.mark.parametrize("B,W,L", [(1, 1, 2), (4, 4, 4), (13, 13, 13)])
def test_sampling_helpers_match_numpy_oracle(B, W, L):
    """Injected uniforms, as the reference's cross-implementation test does."""
    rng = np.random.default_rng(123)
    V = 3
    beams = rng.integers(0, V, size=(B, W, L))
    lp = rng.uniform(-10, 0, size=(B, W, L, V))
    lq = rng.uniform(-10, 0, size=(B, W, L - 1, V))
    u = rng.random((B, W, L - 1))
    n, s = P.sample_choose(torch.tensor(beams), torch.tensor(lp), torch.tensor(lq), torch.tensor(u))
    on, os_ = Acc.sample_choose(beams, lp, lq, u)
    assert np.array_equal(n.numpy(), on) and np.array_equal(s.numpy(), os_)
    s2 = rng.integers(0, W, size=B)
    n2 = rng.integers(0, L, size=B)
    got = P.residual_distribution(torch.tensor(lq), torch.tensor(lp), torch.tensor(s2), torch.tensor(n2))
    assert np.allclose(got.numpy(), Acc.residual_probs(lq, lp, s2, n2), atol=1e-12)
