"""GPU parity: one fused beam-search iteration (rd_beam_topk) and the whole beam search of the
drafter head against the torch-CPU oracle.  Scores/log-probs: 1e-5 in fp32, 2e-2 in bf16; tokens
and parents exact (inputs are either tie-free or ties are resolved by the documented rule)."""
import os
import sys

import numpy as np
import pytest
import torch

from oracle import fp_oracle as O
from oracle import torch_path as P

sys.path.insert(0, os.path.dirname(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(__file__), "golden"))
import tiny_models as tm  # noqa: E402

pytestmark = pytest.mark.gpu


def _step(logits, lpb, beams, want_log_probs=True, force_fallback=False):
    from recurrent_drafting_amd import modeling_drafter as md

    out = md.beam_topk_step(logits.cuda(), lpb.cuda(), beams.cuda(), want_log_probs, force_fallback)
    torch.cuda.synchronize()
    return [None if t is None else t.cpu() for t in out]


def _check_step(logits, lpb, beams, force_fallback, score_tol):
    new_lpb, tok, par, new_beams, logp = _step(logits, lpb, beams, True, force_fallback)
    o_lpb, o_tok, o_par, o_logp = O.beam_search_step(logits, lpb)
    B, W, V = logits.shape
    assert torch.allclose(logp, o_logp.float(), atol=score_tol, rtol=0), (logp - o_logp.float()).abs().max()
    assert torch.allclose(new_lpb, o_lpb, atol=score_tol, rtol=0)
    if not (torch.equal(tok, o_tok) and torch.equal(par, o_par)):
        # selections may differ only where the oracle's own scores are closer than the tolerance
        got = (par * V + tok).tolist(); want = (o_par * V + o_tok).tolist()
        flat = (o_logp.float() + lpb[:, :, None]).reshape(B, -1)
        for b in range(B):
            cut = o_lpb[b, -1].item()
            for i in set(got[b]) ^ set(want[b]):
                assert abs(flat[b, i].item() - cut) <= score_tol, (b, i)
    rows = torch.arange(B)[:, None]
    assert torch.equal(new_beams[..., :-1], beams[rows, par]) and torch.equal(new_beams[..., -1], tok)
    assert (new_lpb[:, :-1] >= new_lpb[:, 1:]).all()


@pytest.mark.parametrize("force_fallback", [False, True])
@pytest.mark.parametrize("B,W,V,t", [(2, 3, 64, 1), (1, 4, 1000, 2), (8, 45, 32000, 3), (2, 64, 32000, 1), (3, 5, 33, 1), (2, 6, 2500, 4)])
def test_step_fp32_tie_free(B, W, V, t, force_fallback):
    torch.manual_seed(V + W)
    logits = torch.randn(B, W, V) * 2
    lpb = -torch.rand(B, W) * 5
    beams = torch.randint(0, V, (B, W, t))
    _check_step(logits, lpb, beams, force_fallback, 1e-5)


@pytest.mark.parametrize("force_fallback", [False, True])
def test_step_first_iteration_only_beam_zero_alive_ties_by_lowest_index_rule(force_fallback):
    """Scores [0, -50000, ...]: every winner descends from beam 0; W=64 > 50 needs filtered tokens,
    which tie exactly and are taken in increasing token id."""
    torch.manual_seed(1)
    for W in (45, 64):
        logits = torch.randn(2, 1, 32000).repeat(1, W, 1) * 3  # all beams share state at iteration 1
        lpb = torch.full((2, W), O.LOG_0); lpb[:, 0] = O.LOG_1
        beams = torch.randint(0, 32000, (2, 1, 1)).repeat(1, W, 1)
        new_lpb, tok, par, new_beams, logp = _step(logits, lpb, beams, True, force_fallback)
        o_lpb, o_tok, o_par, o_logp = O.beam_search_step(logits, lpb)
        assert (par == 0).all() and torch.equal(tok, o_tok) and torch.equal(par, o_par)
        assert torch.allclose(new_lpb, o_lpb, atol=1e-2, rtol=0)  # sums near -50000: fp32 spacing 4e-3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("force_fallback", [False, True])
def test_step_reads_one_shared_row_in_place(dtype, force_fallback):
    """The first iteration's logits are one row per batch row shown W times (stride 0): the kernel
    reads that row in place and must return what it returns for W real copies."""
    from recurrent_drafting_amd import modeling_drafter as md

    torch.manual_seed(4)
    for B, W, V in ((2, 45, 32000), (3, 64, 32000), (2, 5, 1000)):
        one = (torch.randn(B, 1, V) * 3).to(dtype).cuda()
        lpb = torch.full((B, W), O.LOG_0); lpb[:, 0] = O.LOG_1
        beams = torch.randint(0, V, (B, 1, 1)).repeat(1, W, 1).cuda()
        shared = md.beam_topk_step(one.expand(B, W, V), lpb.cuda(), beams, True, force_fallback)
        copies = md.beam_topk_step(one.repeat(1, W, 1), lpb.cuda(), beams, True, force_fallback)
        for a, b in zip(shared, copies):
            assert torch.equal(a, b)


@pytest.mark.parametrize("force_fallback", [False, True])
@pytest.mark.parametrize("B,W,V,t,spread", [(4, 45, 32000, 2, 1.3), (8, 45, 32000, 4, 2.0), (16, 64, 32000, 3, 1.0)])
def test_step_bf16_rounding_points_ties_by_lowest_index_rule(B, W, V, t, spread, force_fallback):
    """bf16 logits: values rounded after the max subtraction, filter value -49920, log-softmax
    rounded to bf16, score float32.  Heavy ties among rounded scores -> lowest flat index wins.
    The log-probabilities may differ from the oracle's by one bf16 step of a row (the logarithm of
    the row sum is formed in another order); the selection is then compared as beam_band says: sorted
    scores within that step, and candidates that only one side selected within two steps of the cut.
    Where the log-probabilities agree bit for bit, tokens, parents and scores must too."""
    import beam_band

    torch.manual_seed(2 + B)
    logits = (torch.randn(B, W, V) * spread).to(torch.bfloat16)
    lpb = (-torch.rand(B, W) * 3).float()
    beams = torch.randint(0, V, (B, W, t))
    new_lpb, tok, par, new_beams, logp = _step(logits, lpb, beams, True, force_fallback)
    o_lpb, o_tok, o_par, o_logp = O.beam_search_step(logits, lpb)
    live = o_logp.float() > -1000
    diff = (logp - o_logp.float()).abs()
    step = 2.0 ** -7 * o_logp.float()[live].abs().max().item()  # one bf16 step of the largest magnitude
    assert diff.max() <= step
    # the filtered class stays one finite constant per row, about -49920 - log(sum)
    assert logp[0, 0].min().item() < -49000
    # one rounding of the float32 result: all but a few entries (those whose float32 value sits within
    # a float32 step of a bf16 rounding boundary) have the oracle's bits -- and the bits that torch's own
    # GPU log_softmax gives for the same tensor, which is the reference's op on this device
    assert (diff[live] > 0).float().mean() <= 1e-3, (diff[live] > 0).float().mean()
    y = O.warp_logits(O.maintain_logits(logits))
    torch_gpu = torch.log_softmax(y.cuda(), dim=-1).float().cpu()
    assert (torch_gpu[live] != logp[live]).float().mean() <= 1e-3
    if diff.max() == 0:
        assert torch.equal(tok, o_tok) and torch.equal(par, o_par) and torch.equal(new_lpb, o_lpb)
    shared = beam_band.check_selection(o_logp, lpb, o_lpb, o_tok, o_par, new_lpb, tok, par, tol=step)
    assert shared >= 0.97, shared
    rows = torch.arange(B)[:, None]
    assert torch.equal(new_beams[..., :-1], beams[rows, par]) and torch.equal(new_beams[..., -1], tok)


@pytest.mark.parametrize("force_fallback", [False, True])
def test_step_fp16_values_differ_below_the_upper_half_of_the_float(force_fallback):
    """A half carries 10 mantissa bits: 19 leading bits of the float differ between values, not the
    16 of bf16 (the pivot search walks over exactly those bits)."""
    import beam_band

    torch.manual_seed(12)
    B, W, V = 3, 10, 5000
    logits = (torch.randn(B, W, V) * 1.5).to(torch.float16)
    lpb = (-torch.rand(B, W) * 3).float()
    beams = torch.randint(0, V, (B, W, 2))
    new_lpb, tok, par, new_beams, logp = _step(logits, lpb, beams, True, force_fallback)
    o_lpb, o_tok, o_par, o_logp = O.beam_search_step(logits, lpb)
    live = o_logp.float() > -1000
    step = 2.0 ** -10 * o_logp.float()[live].abs().max().item()  # one fp16 step of the largest magnitude
    assert (logp - o_logp.float()).abs()[live].max() <= step
    shared = beam_band.check_selection(o_logp, lpb, o_lpb, o_tok, o_par, new_lpb, tok, par, tol=step)
    assert shared >= 0.97, shared


def test_step_many_ties_by_lowest_index_rule_overflow_to_exact_path():
    """All-equal and two-valued rows: every entry ties, the candidate list overflows, and the
    lowest indices must win."""
    V, W = 32000, 5
    logits = torch.zeros(1, W, V)
    logits[0, 1, 100:] = -1.0  # row 1: 100 large entries (> 50), the rest smaller
    lpb = torch.zeros(1, W)
    beams = torch.zeros(1, W, 1, dtype=torch.long)
    new_lpb, tok, par, _, logp = _step(logits, lpb, beams)
    o_lpb, o_tok, o_par, o_logp = O.beam_search_step(logits, lpb)
    assert torch.equal(tok, o_tok) and torch.equal(par, o_par)
    assert torch.allclose(new_lpb, o_lpb, atol=1e-5) and torch.allclose(logp, o_logp, atol=1e-5)


def test_step_adversarial_layout_overflows_pivot():
    """Large values concentrated where one thread sees them all defeats the per-wave pivot."""
    V, W = 32000, 3
    torch.manual_seed(3)
    logits = torch.randn(1, W, V) * 0.01 - 10
    idx = torch.arange(0, V, 8 * 1024)  # same thread, every vector chunk
    for e in range(8):
        logits[0, :, (idx + e).clamp(max=V - 1)] += 20 + torch.rand(len(idx))
    lpb = torch.zeros(1, W)
    beams = torch.zeros(1, W, 1, dtype=torch.long)
    _check_step(logits, lpb, beams, False, 1e-5)


def _models(seed, dtype):
    import recurrent_drafting_amd as rd
    from transformers.models.llama.configuration_llama import LlamaConfig

    llm = rd.modeling_llama.LlamaForCausalLM(LlamaConfig(**tm.LLAMA))
    drafter = rd.modeling_drafter.Drafter(rd.configuration_drafter.DrafterConfig(**tm.DRAFTER))
    llm.load_state_dict(tm.draw(tm.llama_shapes(), seed), strict=False)
    drafter.load_state_dict(tm.draw(tm.drafter_shapes(), seed + 1000))
    return llm.to(dtype).eval(), drafter.to(dtype).eval()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,W,hidden,state_rows", [(1, 1, 8, 1), (3, 7, 40, 1), (8, 45, 4096, 1), (2, 64, 256, 64), (5, 6, 24, 6)])
def test_beam_init_is_the_reference_initial_state(dtype, B, W, hidden, state_rows):
    """modeling_drafter.py:170-189 op by op, against the one launch; a strided prompt state and the
    state half of the head's input untouched."""
    from recurrent_drafting_amd import modeling_drafter as md

    if hidden * torch.empty((), dtype=dtype).element_size() % 16:
        pytest.skip("rows must be multiples of 16 bytes")
    g = torch.Generator().manual_seed(B * 1000 + W)
    wide = torch.randn(B, 2 * hidden, generator=g).to(dtype).cuda()
    prompt_state = wide[:, :hidden]  # row stride 2 * hidden
    init_token = torch.randint(0, 32000, (B,), generator=g).cuda()
    log_p_beam, beams, head_in, state = md.beam_init(prompt_state, init_token, W, state_rows)
    want_lpb = torch.full((B, W), md.LOG_0, dtype=torch.float32)
    want_lpb[:, 0] = md.LOG_1
    assert torch.equal(log_p_beam.cpu(), want_lpb) and log_p_beam.dtype == torch.float32
    assert torch.equal(beams.cpu(), init_token.cpu().view(B, 1, 1).expand(B, W, 1)) and beams.dtype == torch.long
    assert head_in.shape == (B, W, 2 * hidden) and head_in.dtype == dtype
    assert torch.equal(head_in[..., :hidden].cpu(), prompt_state.cpu().unsqueeze(1).expand(B, W, hidden))
    assert state.shape == (B, state_rows, hidden) and state.dtype == dtype and not state.cpu().float().abs().any()
    # what the launch must not touch: the state half of the head's input
    head_in2 = torch.full((B, W, 2 * hidden), 3.0, dtype=dtype, device="cuda")
    from recurrent_drafting_amd import _hip
    e = prompt_state.element_size()
    _hip.check(_hip.lib().rd_beam_init(_hip.ptr(prompt_state), prompt_state.stride(0) * e, _hip.ptr(init_token), B, W,
                                       hidden * e, md.LOG_0, _hip.ptr(log_p_beam), _hip.ptr(beams), _hip.ptr(head_in2),
                                       2 * hidden * e, _hip.ptr(state), state_rows, _hip.stream()))
    assert torch.equal(head_in2[..., hidden:].cpu(), torch.full((B, W, hidden), 3.0, dtype=dtype))
    assert torch.equal(head_in2[..., :hidden], head_in[..., :hidden])


def test_beam_search_candidates_matches_reference_vectors(ref_vectors):
    """The reference's own beams on tie-free float32 drafters (weights are multiples of 1/64)."""
    import recurrent_drafting_amd as rd

    for c in ref_vectors["beam_search"]:
        W, L, V, hid = c["W"], c["L"], c["V"], c["hidden"]
        drafter = rd.modeling_drafter.Drafter(rd.configuration_drafter.DrafterConfig(
            vocab_size=V, hidden_size=hid, exit_dim=2 * hid, num_draft_layers=1, rnn=True))
        sd = {k: torch.tensor(v, dtype=torch.float32).reshape(c["weight_shapes"][k]) / c["weight_scale"]
              for k, v in c["weights_x64"].items()}
        drafter.load_state_dict(sd)
        drafter = drafter.cuda().eval()
        emb = torch.nn.Embedding(V, hid)
        emb.weight.data = torch.tensor(c["embedding_x64"], dtype=torch.float32).reshape(V, hid) / 64
        emb = emb.cuda()
        ctx = (torch.tensor(c["prompt_state_x64"], dtype=torch.float32).reshape(-1, hid) / 64).cuda()
        with torch.inference_mode():
            beams, hist = drafter.beam_search_candidates(
                ctx, torch.tensor(c["init_token"]).cuda(), emb, rd.BeamShape(W, L))
        assert beams.cpu().tolist() == c["beams"]
        picked = torch.gather(hist, 3, beams[:, :, 1:, None]).squeeze(-1).cpu()
        assert torch.allclose(picked, torch.tensor(c["log_prob_of_drafted"]), atol=1e-4)
        assert torch.allclose(hist.max(-1).values.cpu(), torch.tensor(c["log_prob_row_max"]), atol=1e-4)


@pytest.mark.parametrize("W,L", [(4, 3), (10, 4), (45, 5)])
def test_beam_search_candidates_vs_torch_oracle_fp32(W, L):
    import recurrent_drafting_amd as rd

    llm, drafter = _models(5, torch.float32)
    torch.manual_seed(W)
    ctx = torch.randn(3, 128)
    tok = torch.randint(1, 1000, (3,))
    with torch.inference_mode():
        o_beams, o_hist = P.beam_search(drafter, llm.model.embed_tokens, ctx, tok, W, L)
        llm, drafter = llm.cuda(), drafter.cuda()
        beams, hist = drafter.beam_search_candidates(ctx.cuda(), tok.cuda(), llm.model.embed_tokens, rd.BeamShape(W, L))
        b2, none = drafter.beam_search_candidates(ctx.cuda(), tok.cuda(), llm.model.embed_tokens, rd.BeamShape(W, L), return_log_probs=False)
    assert none is None and torch.equal(b2, beams)
    assert hist.shape == (3, W, L - 1, 1000) and hist.dtype == torch.float32
    assert torch.equal(beams.cpu(), o_beams)
    assert torch.allclose(hist.cpu(), o_hist, atol=1e-4)
    assert (beams[:, :, 0].cpu() == tok[:, None]).all()
