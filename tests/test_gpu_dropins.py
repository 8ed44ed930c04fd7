"""The reference-shaped entry points of the package, driven the way upstream's own decode loop
drives them (recurrent_drafting.py:596-705): _comprehend_prompt -> beam_search_candidates ->
_verify_candidates -> _greedy_accept_candidate_tokens / _accept_candidate_tokens.  A caller that
keeps upstream's `_generate` goes through exactly these; the results must equal the token streams
the reference produced (tests/golden/reference_vectors.json) and those of the fused loop.

Also the speculative-sampling helpers against the reference's vectors, randomness replaced as in
tests/golden/make_reference_vectors.py (torch.rand a recorded tensor, Categorical.sample the mode).
"""
import os
import sys
import unittest.mock as mock

import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "golden"))
import tiny_models as tm  # noqa: E402

pytestmark = pytest.mark.gpu


class Mode:
    """Stands in for torch.distributions.Categorical: records the probs, draws their mode."""

    seen = []

    def __init__(self, probs=None, **kw):
        self.p = probs
        Mode.seen.append(probs)

    def sample(self):
        return self.p.argmax(dim=-1)


def f32(flat, *shape):
    return torch.tensor(flat, dtype=torch.float32).reshape(*shape).cuda()


def _models(c):
    import recurrent_drafting_amd as rd
    from transformers.models.llama.configuration_llama import LlamaConfig

    if c.get("markov"):
        llama_sd, drafter_sd = tm.markov(c["seed"])
    else:
        llama_sd, drafter_sd = tm.draw(tm.llama_shapes(), c["seed"]), tm.draw(tm.drafter_shapes(), c["seed"] + 1000)
    llm = rd.modeling_llama.LlamaForCausalLM(LlamaConfig(**tm.LLAMA))
    drafter = rd.modeling_drafter.Drafter(rd.configuration_drafter.DrafterConfig(**tm.DRAFTER))
    llm.load_state_dict(llama_sd, strict=False)
    drafter.load_state_dict(drafter_sd)
    return llm.cuda().eval(), drafter.cuda().eval()


def upstream_shaped_loop(llm, drafter, input_ids, max_length, beam_shape, sampling_args, special_tokens):
    """Upstream's `_generate`, call for call, on this package's drop-in functions."""
    import recurrent_drafting_amd as rd
    from recurrent_drafting_amd import recurrent_drafting as R

    B, seq_len = input_ids.shape
    cfg = llm.config
    cache = rd.kv_cache.Cache(
        batch_size=B, max_length=max_length + beam_shape.length * beam_shape.width,
        n_layers=cfg.num_hidden_layers, n_heads=cfg.num_key_value_heads,
        head_dim=cfg.hidden_size // cfg.num_attention_heads, dtype=llm.dtype, device=input_ids.device)
    tg = rd.stats.TextGeneration()
    with torch.inference_mode():
        context, init_tokens = R._comprehend_prompt(llm, input_ids, cache, sampling_args, special_tokens.pad)
        while seq_len < max_length:
            with tg.step() as step:
                with step.time("generate_candidates"):
                    beams, log_q = drafter.beam_search_candidates(
                        context, init_tokens, llm.base_model.get_input_embeddings(), beam_shape)
                with step.time("verify_candidates"):
                    hidden, logits = R._verify_candidates(step, llm, input_ids, beams, cache, special_tokens.pad)
                with step.time("accept_candidate_tokens"):
                    if sampling_args.greedy:
                        context, input_ids, init_tokens, n = R._greedy_accept_candidate_tokens(
                            input_ids, beams, logits, hidden, cache, special_tokens.pad, step)
                    else:
                        context, input_ids, init_tokens, n = R._accept_candidate_tokens(
                            input_ids, beams, log_q, logits, last_hidden_state=hidden, cache=cache,
                            pad_token_id=special_tokens.pad, temperature=sampling_args.temperature,
                            step_record=step)
                out = torch.cat((input_ids, init_tokens.unsqueeze(-1)), dim=-1)
                seq_len = out.shape[1]
                step.set({"input_id_length": seq_len, "avg_num_accepted": torch.sum(n).item() / B})
                yield out[:, :max_length] if seq_len > max_length else out
    assert set(tg.wall_times) >= {"generate_candidates", "verify_candidates", "accept_candidate_tokens",
                                  "base_forward", "choose_from_candidates", "update_kv_cache_and_input_ids"}


@pytest.mark.parametrize("case_index", [1, 3, 4, 5, 6])  # 5, 6: beam 64 x 5
def test_upstream_shaped_greedy_loop_reproduces_the_reference_streams(ref_vectors, case_index):
    import recurrent_drafting_amd as rd

    case = ref_vectors["end_to_end"][case_index]
    c = case["config"]
    llm, drafter = _models(c)
    ids = tm.prompt(c["batch"], c["prompt_len"], tm.LLAMA["vocab_size"], c["seed"], c["left_pads"]).cuda()
    args = (ids, c["prompt_len"] + c["new_tokens"], rd.BeamShape(c["W"], c["L"]), rd.SamplingArgs(1.0, True),
            rd.SpecialTokens(0, None))
    got = [t.cpu().tolist() for t in upstream_shaped_loop(llm, drafter, *args)]
    assert got == case["steps"]
    fused = [t.cpu().tolist() for t in rd.RecurrentDrafting(llm, drafter).generate(rd.stats.Ledger(), *args)]
    assert fused == got


def _rand_stream(seed):
    g = torch.Generator().manual_seed(seed)
    real = torch.rand

    def draw(*a, **k):
        if "generator" in k or k.get("device") is None:
            return real(*a, **k)
        shape = a[0] if len(a) == 1 else a
        return real(tuple(shape), generator=g).to(k["device"])
    return draw


@pytest.mark.parametrize("case_index", [0, 1, 2, 3])  # 3: beam 64 x 5
def test_sampling_loops_reproduce_the_reference_streams(ref_vectors, case_index):
    """torch.rand a fixed CPU stream and Categorical the mode, exactly as when the reference wrote
    the vectors: the upstream-shaped loop on the drop-ins and the fused loop give its tokens."""
    import recurrent_drafting_amd as rd

    case = ref_vectors["sampling_end_to_end"][case_index]
    c = case["config"]
    llm, drafter = _models(c)
    ids = tm.prompt(c["batch"], c["prompt_len"], tm.LLAMA["vocab_size"], c["seed"], c["left_pads"]).cuda()
    args = (ids, c["prompt_len"] + c["new_tokens"], rd.BeamShape(c["W"], c["L"]),
            rd.SamplingArgs(c["temperature"], False), rd.SpecialTokens(0, None))
    with mock.patch("torch.rand", side_effect=_rand_stream(c["rand_seed"])), \
            mock.patch("torch.distributions.Categorical", Mode):
        got = [t.cpu().tolist() for t in upstream_shaped_loop(llm, drafter, *args)]
    assert got == case["steps"]
    with mock.patch("torch.rand", side_effect=_rand_stream(c["rand_seed"])), \
            mock.patch("torch.distributions.Categorical", Mode):
        ledger = rd.stats.Ledger()
        fused = [t.cpu().tolist() for t in rd.RecurrentDrafting(llm, drafter).generate(ledger, *args)]
    assert fused == case["steps"]
    assert ledger.records[0]["avg_num_accepted"] == pytest.approx(case["avg_num_accepted"])


def test_choose_from_candidates_reference_vectors(ref_vectors):
    from recurrent_drafting_amd import recurrent_drafting as R

    for c in ref_vectors["choose_from_candidates"]:
        B, W, L, V = c["B"], c["W"], c["L"], c["V"]
        u = f32(c["uniforms"], B, W, L - 1)
        with mock.patch("torch.rand", side_effect=lambda *a, **k: u.clone()):
            n, s = R._choose_from_candidates(
                torch.tensor(c["beams"]).cuda(), f32(c["log_p"], B, W, L, V), f32(c["log_q"], B, W, L - 1, V))
        assert n.tolist() == c["n_tokens_in_seq"] and s.tolist() == c["seq_in_beam"]


def test_prepare_next_input_reference_vectors(ref_vectors):
    from recurrent_drafting_amd import recurrent_drafting as R

    for c in ref_vectors["prepare_next_input"]:
        B, W, L, V, H = c["B"], c["W"], c["L"], c["V"], c["H"]
        Mode.seen = []
        with mock.patch("torch.distributions.Categorical", Mode):
            state, tok = R._prepare_next_input(
                f32(c["log_q"], B, W, L - 1, V), f32(c["log_p"], B, W, L, V), f32(c["hidden"], B, W, L, H),
                torch.tensor(c["seq_in_beam"]).cuda(), torch.tensor(c["n_tokens_in_seq"]).cuda())
        assert len(Mode.seen) == 1
        # float32 exp on another device: 1e-5 relative, as stated for fp32 log-probabilities
        assert torch.allclose(Mode.seen[0], f32(c["probs"], B, V), rtol=1e-5, atol=1e-7)
        assert tok.tolist() == c["next_tokens"]
        assert torch.equal(state, f32(c["state"], B, H))


def test_accept_candidate_tokens_reference_vectors(ref_vectors):
    """The whole sampling acceptance on an unpacked cache: counts, ids, the live region of every
    cache slab ([new left padding, new length): outside it the reference leaves stale rows that
    nothing reads, and so does this build, other ones), the probs handed to Categorical, token
    and state.  The vectors use head_dim 2 (8-byte rows); the C ABI moves 16-byte lanes, so every
    value is repeated 4x along head_dim, which commutes with row movement."""
    import recurrent_drafting_amd as rd
    from recurrent_drafting_amd import recurrent_drafting as R

    for c in ref_vectors["accept_candidate_tokens"]:
        sh = c["shape"]
        B, W, L, V, H = sh["B"], sh["W"], sh["L"], sh["V"], sh["H"]
        cache = rd.kv_cache.Cache(B, sh["max_len"], sh["layers"], sh["heads"], sh["D"] * 4, torch.float32,
                                  torch.device("cuda"))
        shape = (sh["layers"], 2, B, sh["heads"], sh["max_len"], sh["D"])
        wide = lambda key: torch.tensor(c[key], dtype=torch.float32).reshape(shape).repeat_interleave(4, dim=-1)  # noqa: E731
        cache._cache.copy_(wide("cache_in"))
        cache.set_length(sh["prev"] + W * L)
        u = f32(c["uniforms"], B, W, L - 1)
        Mode.seen = []
        with mock.patch("torch.rand", side_effect=lambda *a, **k: u.clone()), \
                mock.patch("torch.distributions.Categorical", Mode):
            with rd.stats.TextGeneration().step() as step:
                state, ids, tok, n = R._accept_candidate_tokens(
                    torch.tensor(c["input_ids"]).cuda(), torch.tensor(c["beams"]).cuda(),
                    f32(c["log_q"], B, W, L - 1, V), f32(c["logits"], B, W, L, V), f32(c["hidden"], B, W, L, H),
                    cache, 0, c["temperature"], step)
        assert n.tolist() == c["n_tokens_in_seq"] and ids.tolist() == c["new_ids"]
        assert cache.sliced[0][0].length == c["new_length"]
        want = wide("cache_out")
        got = cache._cache.cpu()
        for b in range(B):
            row = c["new_ids"][b]
            lo = next((i for i, t in enumerate(row) if t != 0), len(row))
            assert torch.equal(got[:, :, b, :, lo:c["new_length"]], want[:, :, b, :, lo:c["new_length"]])
        assert torch.allclose(Mode.seen[0], f32(c["probs"], B, V), rtol=1e-5, atol=1e-7)
        assert tok.tolist() == c["next_tokens"]
        assert torch.equal(state, f32(c["state"], B, H))
