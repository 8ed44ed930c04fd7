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
   beam 45 x 5: forced ragged acceptance for a few steps, then teacher-forced steps.
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


def _summary(reports):
    return "\n".join(
        f"step {r.step}: prev {r.prev} n_q {r.n_q} rows {r.rows} beams_equal {r.beams_equal} shared {r.beams_shared:.2f} "
        f"logits {r.logits_err:.2e} (torch bf16 {r.logits_err_bf16_torch:.2e}) flips {r.flips} "
        f"(margin {r.worst_flip_margin:.1e}) n {r.n_tokens} shift {r.shifts} ctx {r.context_err:.1e} "
        f"kv {r.kv_err:.1e}" for r in reports)


def test_bf16_mfma_decode_loop_teacher_forced_with_accepted_drafts():
    llama_sd, drafter_sd = tm.markov(41, llama_cfg=CFG, drafter_cfg=DCFG, mix=0.05)
    llm, drafter = _models(llama_sd, drafter_sd, CFG, DCFG)
    ids = tm.prompt(4, 300, 4000, 5, left_pads=[0, 131, 3, 250]).cuda()
    reports, kernels = _uses_mfma_kernel(
        lambda: teacher_forced.run(llm, drafter, ids, 300 + 40, 12, 5, steps=12))
    print(_summary(reports))
    assert "attn_mfma_kernel" in kernels and "attn_generic_kernel" not in kernels
    assert len(reports) >= 8
    accepted = [n for r in reports for n in r.n_tokens]
    assert max(accepted) >= 2 and len(set(accepted)) >= 3, accepted  # ragged acceptance happened
    assert any(len(set(r.n_tokens)) > 1 for r in reports)
    assert any(any(x != 0 for x in r.shifts) for r in reports)  # rows shifted and stayed in place
    assert sum(r.beams_equal for r in reports) >= len(reports) - 1


@pytest.mark.parametrize("one_kernel", [False, True])
def test_bf16_mfma_decode_loop_teacher_forced_random_weights_forced_acceptance(one_kernel, monkeypatch):
    # one_kernel: rotation, cache append and attention of a layer as one launch (rd_rope_verify_attention)
    from recurrent_drafting_amd import modeling_llama
    monkeypatch.setattr(modeling_llama.LlamaAttention, "fused_rope_attention", None if one_kernel else False)
    llama_sd = tm.draw(tm.llama_shapes(CFG), 51)
    drafter_sd = tm.draw(tm.drafter_shapes(DCFG), 52)
    llm, drafter = _models(llama_sd, drafter_sd, CFG, DCFG)
    ids = tm.prompt(4, 200, 4000, 6, left_pads=[17, 0, 120, 64]).cuda()
    reports, kernels = _uses_mfma_kernel(
        lambda: teacher_forced.run(llm, drafter, ids, 200 + 60, 12, 5, steps=10,
                                   force=teacher_forced.forced_acceptance(9)))
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
    reports, kernels = _uses_mfma_kernel(
        lambda: teacher_forced.run(llm, drafter, ids, S + 64, 45, 5, steps=7, check_from=4,
                                   force=teacher_forced.forced_acceptance(4)))
    print(_summary(reports))
    assert "attn_mfma_kernel" in kernels and "attn_generic_kernel" not in kernels
    assert len(reports) == 3
    assert all(r.prev >= 1500 and r.n_q >= 100 for r in reports)
    assert all(r.beams_shared >= 0.5 for r in reports)
    assert any(any(x != 0 for x in r.shifts) for r in reports)
