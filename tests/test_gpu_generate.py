"""GPU end-to-end: RecurrentDrafting.generate on the HIP path.

float32 tiny models: token-identical to the reference's own greedy streams (fixtures) and to the
torch restatement run on the same GPU.  bf16: a short run of the tiny model is checked against the
restatement step by step here; the bf16 / head_dim 128 path of the large configuration (MFMA
attention, packed rows, cache rows in place) is compared teacher-forced in test_gpu_decode_bf16.py."""
import os
import sys

import pytest
import torch

from oracle import torch_path as P

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "golden"))
import tiny_models as tm  # noqa: E402

pytestmark = pytest.mark.gpu


def _models(llama_sd, drafter_sd, dtype=torch.float32, cfg=None, dcfg=None):
    import recurrent_drafting_amd as rd
    from transformers.models.llama.configuration_llama import LlamaConfig

    llm = rd.modeling_llama.LlamaForCausalLM(LlamaConfig(**(cfg or tm.LLAMA)))
    drafter = rd.modeling_drafter.Drafter(rd.configuration_drafter.DrafterConfig(**(dcfg or tm.DRAFTER)))
    llm.load_state_dict(llama_sd, strict=False)
    drafter.load_state_dict(drafter_sd)
    return llm.to(dtype).cuda().eval(), drafter.to(dtype).cuda().eval()


def _run(llm, drafter, ids, max_length, W, L, eos=None):
    import recurrent_drafting_amd as rd

    model = rd.RecurrentDrafting(llm, drafter)
    ledger = rd.stats.Ledger()
    steps = [t.cpu().tolist() for t in model.generate(
        ledger, ids.cuda(), max_length, rd.BeamShape(W, L), rd.SamplingArgs(1.0, True), rd.SpecialTokens(0, eos))]
    return steps, ledger


@pytest.mark.parametrize("case_index", [0, 1, 2, 3, 4, 5, 6])  # 5, 6: beam 64 x 5, certain ties in the first iteration
def test_generate_matches_reference_token_streams(ref_vectors, case_index):
    case = ref_vectors["end_to_end"][case_index]
    c = case["config"]
    if c.get("markov"):
        llama_sd, drafter_sd = tm.markov(c["seed"])
    else:
        llama_sd, drafter_sd = tm.draw(tm.llama_shapes(), c["seed"]), tm.draw(tm.drafter_shapes(), c["seed"] + 1000)
    llm, drafter = _models(llama_sd, drafter_sd)
    ids = tm.prompt(c["batch"], c["prompt_len"], tm.LLAMA["vocab_size"], c["seed"], c["left_pads"])
    steps, ledger = _run(llm, drafter, ids, c["prompt_len"] + c["new_tokens"], c["W"], c["L"])
    assert steps == case["steps"]
    rec = ledger.records[0]
    assert len(rec["avg_num_accepted"]) == len(steps)
    for key in ("generate_candidates", "verify_candidates", "base_forward", "accept_candidate_tokens",
                "choose_from_candidates", "update_kv_cache_and_input_ids", "greedy_prepare_next_input"):
        assert len(rec["wall_times"][key]) == len(steps), key


def test_generate_stops_at_eos_and_truncates():
    llama_sd, drafter_sd = tm.markov(21)
    llm, drafter = _models(llama_sd, drafter_sd)
    ids = tm.prompt(2, 8, 1000, 3)
    full, _ = _run(llm, drafter, ids, 8 + 17, 5, 4)
    assert all(len(row) <= 25 for step in full for row in step) and len(full[-1][0]) == 25
    eos = full[2][0][-1]  # a token both rows will have produced by some step
    short, _ = _run(llm, drafter, ids, 8 + 17, 5, 4, eos=eos)
    assert short == full[: len(short)] and len(short) <= len(full)
    last = torch.tensor(short[-1])
    assert ((last[:, 8:] == eos).sum(-1) > 0).all() or len(short) == len(full)


def test_generate_matches_torch_restatement_on_gpu_bigger_model():
    """A wider float32 pair (head_dim 64, GQA 8/4 heads, vocab 4000) with long ragged prompts, run
    through the restatement on the same GPU: identical streams, acceptance included."""
    cfg = dict(tm.LLAMA, vocab_size=4000, hidden_size=512, intermediate_size=1024, num_hidden_layers=3,
               num_attention_heads=8, num_key_value_heads=4)
    dcfg = dict(tm.DRAFTER, vocab_size=4000, hidden_size=512, exit_dim=1024)
    llama_sd = tm.draw(tm.llama_shapes(cfg), 31)
    drafter_sd = tm.draw(tm.drafter_shapes(dcfg), 32)
    llm, drafter = _models(llama_sd, drafter_sd, cfg=cfg, dcfg=dcfg)
    ids = tm.prompt(4, 300, 4000, 5, left_pads=[0, 120, 7, 299])
    steps, _ = _run(llm, drafter, ids, 300 + 12, 12, 5)
    want = [t.cpu().tolist() for t, _ in P.generate_greedy(llm, drafter, ids.cuda(), 300 + 12, 12, 5, pad=0, eos=None)]
    assert steps == want


@pytest.mark.parametrize("batch,W,L,prompt_len,left_pads,markov", [
    (1, 1, 2, 5, [0], True),          # the smallest beam: one candidate of one drafted token
    (1, 64, 5, 12, [3], False),       # the widest beam the kernels take, more than the top-50 filter keeps
    (3, 2, 6, 7, [0, 6, 2], True),    # a row that is almost all padding; beams longer than wide
    (5, 7, 3, 1, [0, 0, 0, 0, 0], True),  # one-token prompts
    (2, 45, 5, 40, [0, 17], True),    # the benchmark's beam shape
])
def test_generate_edge_shapes_match_the_restatement(batch, W, L, prompt_len, left_pads, markov):
    """Greedy token streams at the edges of the shape space (float32 tiny models) against the torch
    restatement on the same GPU, step by step; the last step must be cut at max_length."""
    seed = 100 + batch + W
    llama_sd, drafter_sd = tm.markov(seed) if markov else (tm.draw(tm.llama_shapes(), seed), tm.draw(tm.drafter_shapes(), seed + 1000))
    llm, drafter = _models(llama_sd, drafter_sd)
    ids = tm.prompt(batch, prompt_len, tm.LLAMA["vocab_size"], seed, left_pads)
    max_length = prompt_len + 11
    want = [t.cpu().tolist() for t, _ in P.generate_greedy(llm, drafter, ids.cuda(), max_length, W, L, pad=0, eos=None)]
    steps, _ = _run(llm, drafter, ids, max_length, W, L)
    assert steps == want
    assert len(steps[-1][0]) == max_length and all(len(s[0]) <= max_length for s in steps)
