"""Writes tests/golden/reference_vectors.json by running the upstream reference ON THE CPU, in the
build container only (the reference checkout does not exist anywhere else).

Only functions that no literal of the reference's own tests and no closed form pins are sampled:
  * _pack_beams spill-over padding with >= 3 batch rows and the last-row clamp
  * _update_kv_cache_and_input_ids with batch > 1, ragged acceptance, mixed left/right shifts
    (preceded by Cache.unpack, as the decode loop calls them)
  * Drafter.beam_search_candidates on tie-free float32 logits (tokens, parents via beams)
  * a short greedy end-to-end token stream of the tiny float32 configuration
  * speculative sampling with the randomness replaced, the way the reference's own
    cross-implementation tests do it (mlx/recurrent_drafting_test.py:67-114, :154-204, :301-370):
    torch.rand returns a recorded tensor, Categorical(probs).sample() returns the mode of probs and
    the probs it was given are recorded.  _choose_from_candidates, _prepare_next_input,
    _accept_candidate_tokens (whole tensors incl. the cache) and two end-to-end sampling streams.

Usage:  python tests/golden/make_reference_vectors.py [/root/reference]
The output holds inputs and expected outputs as plain numbers; no reference source is copied.
"""

import json
import os
import sys
import types

import numpy as np
import torch

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.json")


def _import_reference():
    # The reference's stats module imports `jsonlines`, which is not installed here; the hot-path
    # functions never touch it, so an empty module of that name is enough to import the package.
    if "jsonlines" not in sys.modules:
        try:
            import jsonlines  # noqa: F401
        except ImportError:
            sys.modules["jsonlines"] = types.ModuleType("jsonlines")
    sys.path.insert(0, REF)
    import recurrent_drafting  # noqa: E402

    return recurrent_drafting


def pack_cases(rd):
    out = []
    rng = np.random.default_rng(7)
    shapes = [(3, 3, 3), (4, 4, 3), (5, 6, 4), (3, 2, 2)]
    for B, W, L in shapes:
        beams = rng.integers(1, 4, size=(B, W, L))
        beams[:, :, 0] = rng.integers(1, 3, size=(B, 1))
        # make the LAST row the shortest so that its padding clamps to the final element
        beams[-1] = beams[-1, 0][None, :]
        prev = int(rng.integers(0, 4))
        pm = (rng.random((B, prev)) > 0.3).astype(np.int64)
        t = torch.tensor(beams)
        tree = rd.tree_attention._dedup_prefix(t)
        ptok, pidx = rd.tree_attention._pack_beams(t, tree)
        pk, unp, mask, off = rd.tree_attention.pack(t, torch.tensor(pm))
        out.append(dict(beams=beams.tolist(), padding_mask=pm.tolist(), prefix_tree=tree.tolist(),
                        packed_beams=ptok.tolist(), packed_token_indices=pidx.tolist(),
                        unpacker=unp.tolist(), mask=mask.to(torch.int64).tolist(),
                        position_offsets=off.tolist()))
    return out


def kv_update_cases(rd):
    out = []
    rng = np.random.default_rng(11)
    for case in range(4):
        B, W, L = [(3, 3, 4), (4, 2, 3), (2, 4, 5), (5, 3, 3)][case]
        n_layers, H, D = 2, 2, 2
        prev = int(rng.integers(3, 8))
        max_len = prev + W * L + 2
        pads = rng.integers(0, 3, size=B)
        pads[rng.integers(0, B)] = 0
        ids = rng.integers(1, 50, size=(B, prev))
        for b in range(B):
            ids[b, : pads[b]] = 0
        beams = rng.integers(1, 50, size=(B, W, L))
        beams[:, :, 0] = beams[:, :1, 0]
        beams[:, 1:, 1] = np.where(rng.random((B, W - 1)) < 0.5, beams[:, :1, 1], beams[:, 1:, 1])
        t = torch.tensor(beams)
        packed, unp, _, _ = rd.tree_attention.pack(t, torch.tensor((ids != 0).astype(np.int64)))
        n_sel = packed.shape[1]
        cache = rd.kv_cache.Cache(B, max_len, n_layers, H, D, torch.float32, torch.device("cpu"))
        fill = rng.integers(-1000, 1000, size=(n_layers, 2, B, H, prev + n_sel, D)).astype(np.float32)
        for layer in range(n_layers):
            for kv in range(2):
                cache.sliced[layer][kv].cat(torch.tensor(fill[layer, kv]))
        # stale data beyond the live region must survive unchanged where the reference leaves it
        stale = rng.integers(-9, 9, size=cache._cache[..., prev + n_sel :, :].shape)
        cache._cache[..., prev + n_sel :, :] = torch.tensor(stale.astype(np.float32))
        before = cache._cache.clone()
        cache.unpack(prev, unp)
        after_unpack = cache._cache.clone()
        n_tok = rng.integers(0, L, size=B)
        s_beam = rng.integers(0, W, size=B)
        new_ids = rd.recurrent_drafting._update_kv_cache_and_input_ids(
            torch.tensor(ids), torch.tensor(n_tok), torch.tensor(s_beam), t, cache, 0)
        out.append(dict(
            shape=dict(B=B, W=W, L=L, layers=n_layers, H=H, D=D, prev=prev, max_len=max_len),
            input_ids=ids.tolist(), beams=beams.tolist(), unpacker=unp.tolist(),
            n_tokens_in_seq=n_tok.tolist(), seq_in_beam=s_beam.tolist(),
            cache_before=before.to(torch.int64).flatten().tolist(),
            cache_after_unpack=after_unpack.to(torch.int64).flatten().tolist(),
            cache_after_update=cache._cache.to(torch.int64).flatten().tolist(),
            new_ids=new_ids.tolist(), new_length=int(cache.sliced[0][0].length)))
    return out


def beam_search_cases(rd):
    """Tie-free float32 drafter: distinct logits everywhere, so torch.topk's order is determined."""
    out = []
    # the last two are wider than the top-50 filter (W = 64 > 50 < V): after the first iteration 14
    # beams are filtered tokens whose scores tie, and torch.topk's choice among them is unspecified;
    # from the second iteration on 50 live beams offer 2500 candidates, so the final beams (L >= 3)
    # descend from live beams only and do not depend on that choice
    for seed, (B, W, L, V, hid) in enumerate([(2, 3, 4, 64, 8), (1, 4, 3, 80, 8), (2, 5, 5, 96, 16),
                                              (2, 64, 4, 96, 16), (1, 64, 3, 120, 8)]):
        torch.manual_seed(100 + seed)
        cfg = rd.configuration_drafter.DrafterConfig(
            vocab_size=V, hidden_size=hid, exit_dim=2 * hid, num_draft_layers=1, rnn=True)
        try:
            drafter = rd.modeling_drafter.Drafter(cfg)
        except Exception as e:  # transformers version drift: an ordinary error, not a denial
            return dict(error=f"Drafter construction failed: {type(e).__name__}: {e}")
        drafter.eval()
        # every weight is an integer multiple of 1/64, stored below as that integer
        def dyadic(shape):
            return torch.randint(-48, 49, tuple(shape)).float() / 64.0

        with torch.no_grad():
            for p in drafter.parameters():
                p.copy_(dyadic(p.shape))
        emb = torch.nn.Embedding(V, hid)
        with torch.no_grad():
            emb.weight.copy_(dyadic(emb.weight.shape))
        state = dyadic((B, hid))
        tok = torch.randint(0, V, (B,))
        with torch.no_grad():
            beams, logp = drafter.beam_search_candidates(
                state, tok, emb, rd.modeling_drafter.BeamShape(W, L))
        def as_int(t):
            return (t.detach() * 64).round().to(torch.int64).flatten().tolist()

        sd = {k: as_int(v) for k, v in drafter.state_dict().items()}
        shapes = {k: list(v.shape) for k, v in drafter.state_dict().items()}
        picked = torch.gather(logp, 3, beams[:, :, 1:, None]).squeeze(-1)
        out.append(dict(B=B, W=W, L=L, V=V, hidden=hid, weight_scale=64, weights_x64=sd,
                        weight_shapes=shapes, embedding_x64=as_int(emb.weight),
                        prompt_state_x64=as_int(state), init_token=tok.tolist(),
                        beams=beams.tolist(), log_prob_of_drafted=picked.tolist(),
                        log_prob_row_max=logp.max(dim=-1).values.tolist(),
                        log_prob_row_min=logp.min(dim=-1).values.tolist()))
    return out


def end_to_end_cases(rd):
    """Greedy token streams of the tiny float32 configuration, straight from the reference loop."""
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import tiny_models as tm
    from transformers.models.llama.configuration_llama import LlamaConfig

    out = []
    try:
        cfg = LlamaConfig(**tm.LLAMA, rope_theta=10000.0)
        if not hasattr(cfg, "rope_theta"):
            cfg.rope_theta = 10000.0
        llm = rd.modeling_llama.LlamaForCausalLM(cfg)
        drafter = rd.modeling_drafter.Drafter(rd.configuration_drafter.DrafterConfig(**tm.DRAFTER))
    except Exception as e:  # library drift: an ordinary error
        return dict(error=f"model construction failed: {type(e).__name__}: {e}")
    llm.eval(); drafter.eval()
    cases = [dict(seed=123, batch=1, prompt_len=16, left_pads=[], W=4, L=3, new_tokens=32),
             dict(seed=7, batch=3, prompt_len=12, left_pads=[0, 3, 5], W=6, L=4, new_tokens=24),
             dict(seed=11, batch=2, prompt_len=9, left_pads=[2, 0], W=5, L=5, new_tokens=20),
             dict(seed=21, batch=4, prompt_len=10, left_pads=[0, 4, 1, 0], W=5, L=4, new_tokens=30,
                  markov=True),
             dict(seed=22, batch=2, prompt_len=6, left_pads=[0, 2], W=8, L=6, new_tokens=40,
                  markov=True),
             # beams wider than the top-50 filter: ties are certain in the first beam-search iteration
             dict(seed=31, batch=2, prompt_len=8, left_pads=[0, 3], W=64, L=5, new_tokens=24),
             dict(seed=32, batch=3, prompt_len=7, left_pads=[2, 0, 1], W=64, L=5, new_tokens=36,
                  markov=True)]
    for c in cases:
        if c.get("markov"):
            llama_sd, drafter_sd = tm.markov(c["seed"])
        else:
            llama_sd = tm.draw(tm.llama_shapes(), c["seed"])
            drafter_sd = tm.draw(tm.drafter_shapes(), c["seed"] + 1000)
        llm.load_state_dict(llama_sd, strict=False)  # rotary buffers are not part of the draw
        drafter.load_state_dict(drafter_sd)
        ids = tm.prompt(c["batch"], c["prompt_len"], tm.LLAMA["vocab_size"], c["seed"], c["left_pads"])
        model = rd.recurrent_drafting.RecurrentDrafting(llm, drafter)
        steps = []
        try:
            with torch.inference_mode():
                gen = model._generate(
                    text_generation=rd.stats.TextGeneration(), input_ids=ids,
                    max_length=c["prompt_len"] + c["new_tokens"],
                    beam_shape=rd.modeling_drafter.BeamShape(c["W"], c["L"]),
                    sampling_args=rd.recurrent_drafting.SamplingArgs(1.0, True),
                    special_tokens=rd.recurrent_drafting.SpecialTokens(0, None))
                for tokens in gen:
                    steps.append(tokens.tolist())
        except Exception as e:
            return dict(error=f"reference generate failed: {type(e).__name__}: {e}")
        out.append(dict(config=c, steps=steps))
    return out


class _Mode:
    """Stands in for torch.distributions.Categorical: records the probs, samples their mode."""

    seen = []

    def __init__(self, probs=None, logits=None, validate_args=None):
        assert probs is not None
        self.probs = probs
        _Mode.seen.append(probs.detach().clone())

    def sample(self):
        return self.probs.argmax(dim=-1)


def _floats(t):
    return t.detach().to(torch.float32).flatten().tolist()  # float32 -> double is exact


def _log_dists(rng, shape, peak):
    """Random log-distributions over the last axis; `peak` sharpens them."""
    x = torch.tensor(rng.normal(size=shape) * peak, dtype=torch.float32)
    return x.log_softmax(dim=-1)


def choose_cases(rd):
    """_choose_from_candidates with torch.rand replaced by a recorded tensor."""
    import unittest.mock as mock

    out = []
    rng = np.random.default_rng(31)
    for B, W, L, V, peak in [(1, 1, 2, 5, 1.0), (2, 3, 4, 7, 1.0), (3, 4, 5, 11, 2.0), (4, 6, 3, 9, 0.5),
                             (2, 5, 6, 8, 0.2)]:
        log_p = _log_dists(rng, (B, W, L, V), peak)
        # the drafter close to the LLM (so that runs of accepted tokens occur), plus noise
        log_q = (log_p[:, :, :-1, :] + torch.tensor(rng.normal(size=(B, W, L - 1, V)) * 0.4,
                                                   dtype=torch.float32)).log_softmax(dim=-1)
        beams = torch.tensor(rng.integers(0, V, size=(B, W, L)))
        # drafted tokens are mostly likely ones under q, as a beam search would pick them
        likely = log_q.argmax(dim=-1)
        pick = torch.tensor(rng.random((B, W, L - 1)) < 0.7)
        beams[:, :, 1:] = torch.where(pick, likely, beams[:, :, 1:])
        u = torch.tensor(rng.random((B, W, L - 1)), dtype=torch.float32)
        with mock.patch("torch.rand", side_effect=lambda *a, **k: u.clone()):
            n, s = rd.recurrent_drafting._choose_from_candidates(beams, log_p, log_q)
        out.append(dict(B=B, W=W, L=L, V=V, beams=beams.tolist(), log_p=_floats(log_p), log_q=_floats(log_q),
                        uniforms=_floats(u), n_tokens_in_seq=n.tolist(), seq_in_beam=s.tolist()))
    return out


def prepare_next_cases(rd):
    """_prepare_next_input: the probs handed to Categorical, the state and the (mode) token."""
    import unittest.mock as mock

    out = []
    rng = np.random.default_rng(37)
    for B, W, L, V, H in [(1, 1, 2, 6, 3), (3, 2, 4, 9, 4), (4, 3, 3, 12, 2), (5, 2, 5, 7, 3)]:
        log_p = _log_dists(rng, (B, W, L, V), 1.5)
        log_q = _log_dists(rng, (B, W, L - 1, V), 1.5)
        hidden = torch.tensor(rng.normal(size=(B, W, L, H)), dtype=torch.float32)
        s = torch.tensor(rng.integers(0, W, size=B))
        n = torch.tensor(rng.integers(0, L, size=B))
        n[0] = L - 1  # a row that accepted its whole beam: exp(P) at the last position
        if B > 1:
            n[1] = 0
        _Mode.seen = []
        with mock.patch("torch.distributions.Categorical", _Mode):
            state, tok = rd.recurrent_drafting._prepare_next_input(log_q, log_p, hidden, s, n)
        assert len(_Mode.seen) == 1
        out.append(dict(B=B, W=W, L=L, V=V, H=H, log_p=_floats(log_p), log_q=_floats(log_q),
                        hidden=_floats(hidden), seq_in_beam=s.tolist(), n_tokens_in_seq=n.tolist(),
                        probs=_floats(_Mode.seen[0]), state=_floats(state), next_tokens=tok.tolist()))
    return out


def accept_cases(rd):
    """_accept_candidate_tokens end to end (choose + cache/ids update + next input), both kinds of
    randomness replaced; the cache is filled and unpacked as the decode loop leaves it."""
    import unittest.mock as mock

    out = []
    rng = np.random.default_rng(41)
    for B, W, L, V, H, T in [(3, 3, 4, 9, 3, 1.0), (2, 4, 3, 8, 2, 0.7), (4, 2, 5, 10, 2, 1.3)]:
        n_layers, heads, D = 2, 2, 2
        prev = int(rng.integers(3, 7))
        max_len = prev + W * L + 2
        pads = rng.integers(0, 3, size=B)
        pads[rng.integers(0, B)] = 0
        ids = rng.integers(1, V, size=(B, prev))
        for b in range(B):
            ids[b, : pads[b]] = 0
        beams = rng.integers(1, V, size=(B, W, L))
        beams[:, :, 0] = beams[:, :1, 0]
        beams[:, 1:, 1] = np.where(rng.random((B, W - 1)) < 0.5, beams[:, :1, 1], beams[:, 1:, 1])
        t = torch.tensor(beams)
        packed, unp, _, _ = rd.tree_attention.pack(t, torch.tensor((ids != 0).astype(np.int64)))
        n_sel = packed.shape[1]
        cache = rd.kv_cache.Cache(B, max_len, n_layers, heads, D, torch.float32, torch.device("cpu"))
        fill = rng.integers(-1000, 1000, size=(n_layers, 2, B, heads, prev + n_sel, D)).astype(np.float32)
        for layer in range(n_layers):
            for kv in range(2):
                cache.sliced[layer][kv].cat(torch.tensor(fill[layer, kv]))
        cache.unpack(prev, unp)
        cache_in = cache._cache.clone()
        logits = torch.tensor(rng.normal(size=(B, W, L, V)) * 1.5, dtype=torch.float32)
        log_q = ((logits[:, :, :-1, :] / T).log_softmax(-1) + torch.tensor(
            rng.normal(size=(B, W, L - 1, V)) * 0.3, dtype=torch.float32)).log_softmax(-1)
        # drafted tokens the drafter finds likely, so that some get accepted
        likely = log_q.argmax(dim=-1)
        keep = torch.tensor(rng.random((B, W, L - 1)) < 0.7)
        t[:, :, 1:] = torch.where(keep, likely, t[:, :, 1:])
        hidden = torch.tensor(rng.normal(size=(B, W, L, H)), dtype=torch.float32)
        u = torch.tensor(rng.random((B, W, L - 1)), dtype=torch.float32)
        _Mode.seen = []
        with mock.patch("torch.rand", side_effect=lambda *a, **k: u.clone()), \
                mock.patch("torch.distributions.Categorical", _Mode):
            with rd.stats.TextGeneration().step() as step:
                state, new_ids, tok, n = rd.recurrent_drafting._accept_candidate_tokens(
                    torch.tensor(ids), t, log_q, logits, hidden, cache, 0, T, step)
        out.append(dict(
            shape=dict(B=B, W=W, L=L, V=V, H=H, layers=n_layers, heads=heads, D=D, prev=prev, max_len=max_len),
            temperature=T, input_ids=ids.tolist(), beams=t.tolist(), unpacker=unp.tolist(),
            logits=_floats(logits), log_q=_floats(log_q), hidden=_floats(hidden), uniforms=_floats(u),
            cache_in=cache_in.to(torch.int64).flatten().tolist(),
            cache_out=cache._cache.to(torch.int64).flatten().tolist(),
            new_length=int(cache.sliced[0][0].length), new_ids=new_ids.tolist(), state=_floats(state),
            next_tokens=tok.tolist(), n_tokens_in_seq=n.tolist(), probs=_floats(_Mode.seen[0])))
    return out


def sampling_stream_cases(rd):
    """End-to-end speculative-sampling token streams of the tiny float32 models: torch.rand is a
    fixed CPU stream (torch.Generator seeded per case, drawn in call order), Categorical the mode."""
    import unittest.mock as mock

    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import tiny_models as tm
    from transformers.models.llama.configuration_llama import LlamaConfig

    cfg = LlamaConfig(**tm.LLAMA, rope_theta=10000.0)
    if not hasattr(cfg, "rope_theta"):
        cfg.rope_theta = 10000.0
    llm = rd.modeling_llama.LlamaForCausalLM(cfg)
    drafter = rd.modeling_drafter.Drafter(rd.configuration_drafter.DrafterConfig(**tm.DRAFTER))
    llm.eval(); drafter.eval()
    cases = [dict(seed=5, batch=3, prompt_len=9, left_pads=[0, 2, 4], W=6, L=4, new_tokens=18,
                  temperature=0.9, rand_seed=77),
             dict(seed=21, batch=3, prompt_len=8, left_pads=[3, 0, 1], W=5, L=5, new_tokens=24,
                  temperature=1.0, rand_seed=78, markov=True),
             dict(seed=23, batch=2, prompt_len=7, left_pads=[0, 2], W=4, L=3, new_tokens=16,
                  temperature=1.7, rand_seed=79, markov=True),
             dict(seed=33, batch=2, prompt_len=8, left_pads=[1, 0], W=64, L=5, new_tokens=24,
                  temperature=1.0, rand_seed=80, markov=True)]
    out = []
    real_rand = torch.rand
    for c in cases:
        if c.get("markov"):
            llama_sd, drafter_sd = tm.markov(c["seed"])
        else:
            llama_sd = tm.draw(tm.llama_shapes(), c["seed"])
            drafter_sd = tm.draw(tm.drafter_shapes(), c["seed"] + 1000)
        llm.load_state_dict(llama_sd, strict=False)
        drafter.load_state_dict(drafter_sd)
        ids = tm.prompt(c["batch"], c["prompt_len"], tm.LLAMA["vocab_size"], c["seed"], c["left_pads"])
        g = torch.Generator().manual_seed(c["rand_seed"])
        model = rd.recurrent_drafting.RecurrentDrafting(llm, drafter)
        steps, accepted = [], []
        _Mode.seen = []
        with mock.patch("torch.rand", side_effect=lambda shape, **k: real_rand(tuple(shape), generator=g)), \
                mock.patch("torch.distributions.Categorical", _Mode), torch.inference_mode():
            tg = rd.stats.TextGeneration()
            gen = model._generate(
                text_generation=tg, input_ids=ids, max_length=c["prompt_len"] + c["new_tokens"],
                beam_shape=rd.modeling_drafter.BeamShape(c["W"], c["L"]),
                sampling_args=rd.recurrent_drafting.SamplingArgs(c["temperature"], False),
                special_tokens=rd.recurrent_drafting.SpecialTokens(0, None))
            for tokens in gen:
                steps.append(tokens.tolist())
        out.append(dict(config=c, steps=steps, avg_num_accepted=[float(a) for a in tg.stats["avg_num_accepted"]]))
    return out


def main():
    rd = _import_reference()
    torch.set_num_threads(1)
    vec = dict(
        _comment="Produced by tests/golden/make_reference_vectors.py from the upstream reference on "
                 "CPU (torch %s). Inputs and expected outputs only." % torch.__version__,
        pack=pack_cases(rd),
        kv_update=kv_update_cases(rd),
        beam_search=beam_search_cases(rd),
        end_to_end=end_to_end_cases(rd),
        choose_from_candidates=choose_cases(rd),
        prepare_next_input=prepare_next_cases(rd),
        accept_candidate_tokens=accept_cases(rd),
        sampling_end_to_end=sampling_stream_cases(rd),
    )
    with open(OUT, "w") as f:
        json.dump(vec, f, separators=(",", ":"))
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
