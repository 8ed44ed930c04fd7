"""Writes tests/golden/reference_vectors.json by running the upstream reference ON THE CPU, in the
build container only (the reference checkout does not exist anywhere else).

Only functions that no literal of the reference's own tests and no closed form pins are sampled:
  * _pack_beams spill-over padding with >= 3 batch rows and the last-row clamp
  * _update_kv_cache_and_input_ids with batch > 1, ragged acceptance, mixed left/right shifts
    (preceded by Cache.unpack, as the decode loop calls them)
  * Drafter.beam_search_candidates on tie-free float32 logits (tokens, parents via beams)
  * a short greedy end-to-end token stream of the tiny float32 configuration

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
    for seed, (B, W, L, V, hid) in enumerate([(2, 3, 4, 64, 8), (1, 4, 3, 80, 8), (2, 5, 5, 96, 16)]):
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
    )
    with open(OUT, "w") as f:
        json.dump(vec, f, separators=(",", ":"))
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
