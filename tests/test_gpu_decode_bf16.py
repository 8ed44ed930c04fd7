"""The configuration the headline number is measured on, under an oracle check: a bf16 model whose
heads are 128 wide (so the verification attention runs on the MFMA kernel), packed token rows and
cache rows kept in place, all together inside the decode loop -- compared with the torch
restatement step by step on the same inputs (tests/teacher_forced.py says what is compared and to
which bar).

1. a small pair (2 layers, 4 heads x 128, vocabulary 4000, batch 4 with ragged left padding, beam
   12 x 5) whose drafter mostly agrees with the LLM, so drafted tokens are accepted in ragged
   numbers and the cache rows shift;
2. the same shapes with random-init weights (attention and MLP at full strength) and the
   acceptance decision replaced by random accepted lengths;
3. one layer of the 7B shape (hidden 4096, 32 heads x 128, FFN 11008, vocabulary 32000; drafter
   4096/8192 with two blocks), batch 8, about 1500 tokens of context with ragged left padding,
   beam 45 x 5: forced ragged acceptance for a few steps, then teacher-forced steps;
4. speculative sampling at temperature 1 on the pair of 1: every step's acceptance and residual
   distribution against the oracle on the step's own logits, drafter log-probabilities and uniforms;
5. all 32 layers of the 7B shape, batch 8, ragged prompts of about 600 tokens, beam 45 x 5: the
   prefill and two teacher-forced steps after forced ragged acceptance (the composition of the layers:
   error growth through the residual stream, docs/parity_check.md:77-98).

Every case also checks the prefill (cache rows, last hidden state, first token) against the float32
restatement, and every beam-search iteration against the oracle's iteration on the same logits.
"""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(__file__), "golden"))
import teacher_forced  # noqa: E402
import tiny_models as tm  # noqa: E402

pytestmark = pytest.mark.gpu

CFG = dict(tm.LLAMA, vocab_size=4000, hidden_size=512, intermediate_size=1024, num_hidden_layers=2,
           num_attention_heads=4, num_key_value_heads=4)
DCFG = dict(tm.DRAFTER, vocab_size=4000, hidden_size=512, exit_dim=1024)


def _models(llama_sd, drafter_sd, cfg, dcfg):
    import recurrent_drafting_amd as rd
    from transformers.models.llama.configuration_llama import LlamaConfig

    llm = rd.modeling_llama.LlamaForCausalLM(LlamaConfig(**cfg))
    drafter = rd.modeling_drafter.Drafter(rd.configuration_drafter.DrafterConfig(**dcfg))
    llm.load_state_dict(llama_sd, strict=False)
    drafter.load_state_dict(drafter_sd)
    return llm.to(torch.bfloat16).cuda().eval(), drafter.to(torch.bfloat16).cuda().eval()


def _uses_mfma_kernel(fn):
    """Runs fn with the library's per-kernel timing on and returns the kernels that were launched."""
    from recurrent_drafting_amd import _hip

    _hip.timing_enable(True)
    try:
        out = fn()
        torch.cuda.synchronize()
        kernels = _hip.timing_collect()
    finally:
        _hip.timing_enable(False)
    return out, kernels


def _prefill_summary(pre):
    r = pre[0]
    return (f"prefill: S {r.seq} cache rows {r.kv_err:.2e} (torch {r.kv_err_torch:.2e}) last state {r.state_err:.2e} "
            f"(torch {r.state_err_torch:.2e}) first-token flips {r.token_flips} (margin {r.worst_flip_margin:.1e})")


def _summary(reports):
    return "\n".join(
        f"step {r.step}: prev {r.prev} n_q {r.n_q} rows {r.rows} beams_equal {r.beams_equal} shared {r.beams_shared:.2f} "
        f"picks on the same logits {r.beam_picks_shared:.3f} "
        f"logits {r.logits_err:.2e} (torch bf16 {r.logits_err_bf16_torch:.2e}) flips {r.flips} "
        f"(margin {r.worst_flip_margin:.1e}) n {r.n_tokens} shift {r.shifts} ctx {r.context_err:.1e} "
        f"(torch {r.context_err_bf16_torch:.1e}) kv {r.kv_err:.1e} (torch {r.kv_err_bf16_torch:.1e})" for r in reports)


def test_bf16_mfma_decode_loop_teacher_forced_with_accepted_drafts():
    llama_sd, drafter_sd = tm.markov(41, llama_cfg=CFG, drafter_cfg=DCFG, mix=0.05)
    llm, drafter = _models(llama_sd, drafter_sd, CFG, DCFG)
    ids = tm.prompt(4, 300, 4000, 5, left_pads=[0, 131, 3, 250]).cuda()
    pre = []
    reports, kernels = _uses_mfma_kernel(
        lambda: teacher_forced.run(llm, drafter, ids, 300 + 40, 12, 5, steps=12, prefill_report=pre))
    print(_prefill_summary(pre))
    print(_summary(reports))
    assert "attn_mfma_kernel" in kernels and "attn_generic_kernel" not in kernels
    assert len(reports) >= 8
    accepted = [n for r in reports for n in r.n_tokens]
    assert max(accepted) >= 2 and len(set(accepted)) >= 3, accepted  # ragged acceptance happened
    assert any(len(set(r.n_tokens)) > 1 for r in reports)
    assert any(any(x != 0 for x in r.shifts) for r in reports)  # rows shifted and stayed in place
    assert sum(r.beams_equal for r in reports) >= len(reports) - 1


@pytest.mark.parametrize("one_kernel,kv_heads", [(False, 4), (True, 4), (False, 2), (True, 1)])
def test_bf16_mfma_decode_loop_teacher_forced_random_weights_forced_acceptance(one_kernel, kv_heads, monkeypatch):
    # one_kernel: rotation, cache append and attention of a layer as one launch (rd_rope_verify_attention);
    # kv_heads below 4: grouped-query attention (the query heads of a group share cache rows)
    from recurrent_drafting_amd import modeling_llama
    monkeypatch.setattr(modeling_llama.LlamaAttention, "fused_rope_attention", None if one_kernel else False)
    cfg = dict(CFG, num_key_value_heads=kv_heads)
    llama_sd = tm.draw(tm.llama_shapes(cfg), 51)
    drafter_sd = tm.draw(tm.drafter_shapes(DCFG), 52)
    llm, drafter = _models(llama_sd, drafter_sd, cfg, DCFG)
    ids = tm.prompt(4, 200, 4000, 6, left_pads=[17, 0, 120, 64]).cuda()
    pre = []
    reports, kernels = _uses_mfma_kernel(
        lambda: teacher_forced.run(llm, drafter, ids, 200 + 60, 12, 5, steps=10,
                                   force=teacher_forced.forced_acceptance(9), prefill_report=pre))
    print(_prefill_summary(pre))
    print(_summary(reports))
    assert "attn_mfma_kernel" in kernels and "attn_generic_kernel" not in kernels
    assert ("rope_append_kernel" in kernels) == (not one_kernel), sorted(kernels)
    assert len(reports) == 10
    assert any(any(x != 0 for x in r.shifts) for r in reports)
    assert any(any(x < 0 for x in r.shifts) for r in reports) or any(any(x > 0 for x in r.shifts) for r in reports)


def test_bf16_7b_shape_one_layer_teacher_forced_steps_at_long_context():
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench

    torch.manual_seed(0)
    llm, drafter = bench.build_models("cuda:0", torch.bfloat16, 1, 7)
    B, S = 8, 1500
    g = torch.Generator().manual_seed(3)
    ids = torch.randint(1, 32000, (B, S), generator=g)
    for b, n in enumerate([0, 700, 13, 250, 999, 64, 1, 420]):
        ids[b, :n] = 0
    ids = ids.cuda()
    pre = []
    reports, kernels = _uses_mfma_kernel(
        lambda: teacher_forced.run(llm, drafter, ids, S + 64, 45, 5, steps=7, check_from=4,
                                   force=teacher_forced.forced_acceptance(4), prefill_report=pre))
    print(_prefill_summary(pre))
    print(_summary(reports))
    assert "attn_mfma_kernel" in kernels and "attn_generic_kernel" not in kernels
    assert len(reports) == 3 and pre[0].seq == S
    assert all(r.prev >= 1500 and r.n_q >= 100 for r in reports)
    # (beams_shared compares with a beam search on logits from GEMMs of other shapes and is only
    # reported; what is asserted is every iteration's selection on the same logits)
    assert all(r.beam_picks_shared >= 0.97 for r in reports)
    assert any(any(x != 0 for x in r.shifts) for r in reports)


def test_bf16_7b_shape_all_32_layers_prefill_and_teacher_forced_steps():
    """Configuration 4 at full depth: 32 layers of the 7B shape in bf16, batch 8, beam 45 x 5, ragged
    left-padded prompts of 600 tokens; the prefill and two steps (after two steps of forced ragged
    acceptance, so rows have shifted) against the float32 restatement of all 32 layers.  The bar is
    teacher_forced's, with the logit error also held against stock torch's bf16 error on the same
    inputs (at most three times that)."""
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench

    torch.manual_seed(0)
    llm, drafter = bench.build_models("cuda:0", torch.bfloat16, 32, 11)
    B, S = 8, 600
    g = torch.Generator().manual_seed(5)
    ids = torch.randint(1, 32000, (B, S), generator=g)
    for b, n in enumerate([0, 310, 7, 120, 455, 64, 1, 200]):
        ids[b, :n] = 0
    ids = ids.cuda()
    pre = []
    reports, kernels = _uses_mfma_kernel(
        lambda: teacher_forced.run(llm, drafter, ids, S + 48, 45, 5, steps=4, check_from=2, tol=0.15,
                                   force=teacher_forced.forced_acceptance(6), prefill_report=pre))
    print(_prefill_summary(pre))
    print(_summary(reports))
    assert "attn_mfma_kernel" in kernels and "attn_generic_kernel" not in kernels
    assert len(reports) == 2 and pre[0].seq == S
    assert all(r.prev >= 600 and r.n_q >= 100 for r in reports)
    assert all(r.beam_picks_shared >= 0.97 for r in reports)
    assert any(any(x != 0 for x in r.shifts) for r in reports)
    # The composition of 32 layers stays as close to float32 as stock torch's bf16 ops do: at this
    # depth the bar is not a fixed share of the scale (the run above only caps the error at 0.15 of it)
    # but three times what the same op sequence in stock torch bf16 makes of the same inputs
    for r in reports:
        assert r.logits_err <= 3 * r.logits_err_bf16_torch + 1e-3, (r.logits_err, r.logits_err_bf16_torch)
        assert r.kv_err <= 3 * r.kv_err_bf16_torch + 1e-3, (r.kv_err, r.kv_err_bf16_torch)
        assert r.context_err <= 3 * r.context_err_bf16_torch + 1e-3, (r.context_err, r.context_err_bf16_torch)


def test_bf16_mfma_sampling_loop_accepts_as_the_oracle_does_on_the_same_logits():
    """Speculative sampling at temperature 1 through the same bf16 / 128-wide-head path (MFMA
    attention, packed rows spread back to their slots for the head, cache rows in place).  Every
    step's acceptance runs on packed bf16 logits and four floats per row; the oracle gets the
    same logits unpacked and log-softmaxed as the reference materialises them, the same drafter
    log-probabilities and the same uniforms, and must accept the same tokens from the same beams
    and hand the same residual distribution to the draw (the draw itself is replaced by the mode)."""
    import unittest.mock

    import numpy as np

    import recurrent_drafting_amd as rd
    from oracle import fp_oracle as O
    from oracle import torch_path as P
    from oracle import tree_oracle as T
    from recurrent_drafting_amd import acceptance

    llama_sd, drafter_sd = tm.markov(43, llama_cfg=CFG, drafter_cfg=DCFG, mix=0.05)
    llm, drafter = _models(llama_sd, drafter_sd, CFG, DCFG)
    ids = tm.prompt(4, 260, 4000, 7, left_pads=[0, 100, 5, 200]).cuda()
    W, L, temperature, steps = 12, 5, 1.0, 10
    seen = []
    real_accept, real_residual = acceptance.sample_accept, acceptance.residual_probs

    def oracle_log_p(packed):
        unpacked = T.unpack_rows(packed.logits.float().cpu().numpy(), packed.unpacker.cpu().numpy())  # (B,W,L,V)
        return (O.warp_logits(torch.tensor(unpacked)) / packed.temperature).log_softmax(dim=-1)

    def w_accept(beams, log_p, log_q, uniforms):
        n, s = real_accept(beams, log_p, log_q, uniforms)
        ref = oracle_log_p(log_p)
        on, os_ = P.sample_choose(beams.cpu(), ref, log_q.cpu(), uniforms.cpu())
        tok = beams.cpu()[..., 1:, None]
        ratio = torch.exp(ref[:, :, :-1].gather(-1, tok).squeeze(-1) - log_q.cpu().gather(-1, tok).squeeze(-1))
        fragile = bool(((uniforms.cpu() - ratio).abs() < 1e-4 * ratio.clamp(min=1)).any())
        seen.append(dict(n=n.cpu(), s=s.cpu(), on=on, os=os_, fragile=fragile, ref=ref))
        return n, s

    def w_residual(log_q, log_p, seq_in_beam, n_tokens):
        got = real_residual(log_q, log_p, seq_in_beam, n_tokens)
        want = P.residual_distribution(log_q.cpu(), seen[-1]["ref"], seq_in_beam.cpu(), n_tokens.cpu())
        seen[-1]["residual_err"] = float((got.cpu() - want).abs().max())
        seen[-1]["residual_negative"] = bool((got < 0).any())
        return got

    class Mode:
        def __init__(self, probs=None, **kw):
            self.p = probs

        def sample(self):
            return self.p.argmax(dim=-1)

    def loop():
        model = rd.RecurrentDrafting(llm, drafter)
        out = []
        with unittest.mock.patch.object(acceptance, "sample_accept", w_accept), \
                unittest.mock.patch.object(acceptance, "residual_probs", w_residual), \
                unittest.mock.patch("torch.distributions.Categorical", Mode):
            torch.manual_seed(5)
            for i, t in enumerate(model.generate(rd.stats.Ledger(), ids, 260 + 60, rd.BeamShape(W, L),
                                                 rd.SamplingArgs(temperature, False), rd.SpecialTokens(0, None))):
                out.append(t)
                if i + 1 >= steps:
                    break
        return out

    out, kernels = _uses_mfma_kernel(loop)
    assert "attn_mfma_kernel" in kernels and "attn_generic_kernel" not in kernels
    assert {"row_stats_kernel", "accept_sample_kernel", "residual_probs_kernel"} <= set(kernels)
    assert len(seen) >= steps
    for k, st in enumerate(seen):
        if not st["fragile"]:
            assert torch.equal(st["n"], st["on"]) and torch.equal(st["s"], st["os"]), (k, st["n"], st["on"])
        assert st["residual_err"] < 1e-5 and not st["residual_negative"], (k, st["residual_err"])
    accepted = [int(x) for st in seen for x in st["n"]]
    print("accepted per row and step:", accepted)
    assert max(accepted) >= 2 and len(set(accepted)) >= 3  # ragged acceptance happened
    assert sum(not st["fragile"] for st in seen) >= len(seen) - 1
