"""Teacher-forced comparison of the fused HIP decode loop with the torch restatement, step by step.

bf16 logits of two implementations tie within an ulp or two for a share of the positions, so two
correct decoders drift apart after a few tokens (the reference documents this for its own two
decoders, docs/parity_check.md:77-98).  A free-running comparison of token streams therefore says
nothing in bf16; what can be pinned is every step given the same inputs.  `run` drives
RecurrentDrafting.generate and, at every step, hands the state the HIP loop went into the step
with (token ids, drafter context, first token, KV cache contents) to oracle/torch_path on the
same GPU, then compares what came out:

  prefill          before the first step: the cache rows of every layer behind each row's left
                   padding, the last hidden state and the first token of _comprehend_prompt
                   (recurrent_drafting.py:391-434) against the float32 restatement of the prefill
                   (error within `tol` of the scale and within 3x the error of stock torch in the
                   model's dtype; the token may differ from the float32 argmax only inside the margin)
  beams            oracle beam search on the same context and token (same bf16 torch GEMMs), reported;
                   and, asserted, every beam-search iteration on ITS OWN logits: the oracle's
                   iteration (fp_oracle.beam_search_step, modeling_drafter.py:201-215) fed the logits
                   and scores the HIP kernel was fed must select the same (parent, token) pairs --
                   bit for bit where the log-probabilities agree bit for bit, otherwise as
                   tests/beam_band.py says
  tree             packed tokens, unpacker, position offsets and ids, left pad counts, and the mask
                   (unpacked from the bits the attention consumes) of the HIP beams: bit-exact
  packed logits    against the float32 restatement (bf16 weights upcast), within `tol` of the
                   logits' scale; the restatement run in bf16 with stock torch ops is measured
                   against the same float32 figures, as the yardstick for a bf16 implementation
  argmax           a token may differ from the float32 argmax only where the float32 margin
                   between the two tokens is below the tolerance
  acceptance       n_tokens_in_seq / seq_in_beam from the HIP argmax tokens: bit-exact
  next state       new ids bit-exact; next token = the HIP argmax at the chosen slot; drafter
                   context within tolerance; KV rows: kept rows bit-identical, accepted rows
                   bit-identical to the rows the HIP forward wrote, which in turn agree with the
                   restatement's K/V within tolerance

The functions of the package are observed by wrapping module attributes; nothing in the package
knows about this file.
"""

from __future__ import annotations

import copy
import dataclasses
import unittest.mock as mock
from typing import Callable, List, Optional

import numpy as np
import torch

import beam_band
from oracle import accept_oracle as Acc
from oracle import fp_oracle as O
from oracle import torch_path as P


@dataclasses.dataclass
class StepReport:
    step: int
    prev: int
    n_q: int
    rows: int
    beams_equal: bool
    beams_shared: float  # share of the HIP beams that are among the restatement's beams of the same row
    beam_picks_shared: float  # lowest share, over the iterations, of the HIP picks that the oracle makes on the same logits
    logits_err: float  # max |HIP - float32 restatement| / scale
    logits_err_bf16_torch: float  # the same for the bf16 restatement (stock torch ops)
    flips: int  # packed positions whose argmax differs from the float32 argmax
    worst_flip_margin: float  # largest float32 margin among them / scale
    n_tokens: List[int]
    shifts: List[int]  # cache row shifts going into the step
    context_err: float
    kv_err: float
    context_err_bf16_torch: float = 0.0  # the same two figures for the restatement in the model's dtype
    kv_err_bf16_torch: float = 0.0


@dataclasses.dataclass
class PrefillReport:
    seq: int
    kv_err: float  # max |HIP - float32 restatement| / scale over the cache rows behind the left padding, all layers
    kv_err_torch: float  # the same for stock torch in the model's dtype
    state_err: float
    state_err_torch: float
    token_flips: int
    worst_flip_margin: float


def _bits_to_mask(bits: torch.Tensor, kv_len: int) -> torch.Tensor:
    """(B, n, words) int64 words -> (B, n, kv_len) bool."""
    shifts = torch.arange(64, device=bits.device, dtype=torch.int64)
    flat = ((bits.unsqueeze(-1) >> shifts) & 1).flatten(2)
    assert not bool(flat[:, :, kv_len:].any())
    return flat[:, :, :kv_len].bool()


def _snapshot(cache, length: int):
    """Copy of the cache in the reference's layout (column c of row b in cache row c)."""
    from recurrent_drafting_amd import kv_cache

    n_layers, _, B, H, max_len, D = cache._cache.shape
    snap = kv_cache.Cache(B, max_len, n_layers, H, D, cache._cache.dtype, cache._cache.device)
    snap._storage.copy_(cache._storage)
    snap.shift.copy_(cache.shift)
    snap._rows_in_place = True
    snap._shifted = True
    snap.set_length(length)
    snap.materialize()
    torch.cuda.synchronize()
    return snap._cache


def forced_acceptance(seed: int) -> Callable:
    """Replaces the acceptance decision by random accepted lengths and beams (the token streams
    then mean nothing, but rows shift by different amounts at every step)."""
    gen = torch.Generator().manual_seed(seed)

    def force(beams, llm_tokens, unpacker, n, s, nxt, last):
        B, W, L = beams.shape
        n = torch.randint(0, L, (B,), generator=gen).to(beams.device)
        s = torch.randint(0, W, (B,), generator=gen).to(beams.device)
        rows = torch.arange(B, device=beams.device)
        last = unpacker[rows, s, n]
        nxt = llm_tokens[rows, last]
        return n, s, nxt, last
    return force


def run(llm, drafter, ids, max_length: int, W: int, L: int, steps: int, pad: int = 0,
        tol: float = 2e-2, force: Optional[Callable] = None, check_from: int = 0,
        log: Optional[Callable] = None, prefill_report: Optional[list] = None) -> List[StepReport]:
    """Runs `steps` decode steps of the fused loop; the prefill and the steps >= check_from are
    compared with the restatement.  Raises AssertionError on the first violation; returns the
    per-step reports (the PrefillReport is appended to `prefill_report` when a list is given)."""
    import recurrent_drafting_amd as rd
    from recurrent_drafting_amd import acceptance, modeling_drafter, tree_attention
    from recurrent_drafting_amd import recurrent_drafting as loop_module

    dev = ids.device
    llm32 = copy.deepcopy(llm).float()  # bf16 weights upcast (the drafter is compared in its own dtype)
    model = rd.RecurrentDrafting(llm, drafter)
    seen = {}
    real_prepare, real_argmax = tree_attention.prepare_attention, acceptance.argmax_rows
    real_accept, real_realign = acceptance.greedy_accept, acceptance.realign_enqueue
    real_draft = drafter.beam_search_candidates
    real_prefill, real_topk = loop_module._comprehend_prompt, modeling_drafter.beam_topk_step
    prefilled = {}
    iterations = []  # the beam-search iterations of the draft being made

    def w_prefill(llm_, input_ids, cache, sampling_args, pad_token_id):
        state, token = real_prefill(llm_, input_ids, cache, sampling_args, pad_token_id)
        S = input_ids.shape[1]
        prefilled.update(ids=input_ids, rows=cache._cache[:, :, :, :, :S].clone(), state=state.clone(),
                         token=token.clone())
        return state, token

    def w_topk(logits, log_p_beam, beams, want_log_probs, force_fallback=False):
        out = real_topk(logits, log_p_beam, beams, want_log_probs, force_fallback)
        iterations.append(dict(logits=logits, lpb=log_p_beam, new_lpb=out[0], tok=out[1], par=out[2]))
        return out

    def w_prepare(tree, padding_mask, pad_value=0, n_heads=32, kv_shift=None):
        out = real_prepare(tree, padding_mask, pad_value, n_heads, kv_shift)
        prepared, position_ids, left_pads = out
        seen.update(tree=tree, ids=padding_mask, bits=prepared.bits, position_ids=position_ids, left_pads=left_pads)
        return out

    def w_argmax(logits, rows=None):
        out = real_argmax(logits, rows)
        if "tree" in seen:  # (the prefill calls it too, before any tree exists)
            # (with `rows` the result sits at the (batch, slot) places: back to packed-row order)
            packed = out if rows is None else out.flatten().index_select(0, rows.index[: rows.total])
            seen.update(logits=logits, argmax=packed)
        return out

    def w_accept(beams, llm_tokens, unpacker=None):
        n, s, nxt, last = real_accept(beams, llm_tokens, unpacker)
        natural = (n, s)
        if force is not None:
            n, s, nxt, last = force(beams, llm_tokens, unpacker, n, s, nxt, last)
        seen.update(beams=beams, llm_tokens=llm_tokens, unpacker=unpacker, n=n, s=s, natural=natural,
                    next_tokens=nxt, last_slot=last)
        return n, s, nxt, last

    def w_realign(input_ids, n, s, beams, cache, pad_token_id, unpacker=None, left_pads=None, step_out=None):
        seen.update(cache=cache, shift=cache.shift.clone(),
                    snap=_snapshot(cache, cache.sliced[0][0].length))
        return real_realign(input_ids, n, s, beams, cache, pad_token_id, unpacker, left_pads, step_out)

    drafts = []  # draft k feeds step k; it is queued while step k-1 is being finished

    def w_draft(context, init_token, embeddings, beam_shape, return_log_probs=True):
        iterations.clear()
        out = real_draft(context, init_token, embeddings, beam_shape, return_log_probs=return_log_probs)
        drafts.append(dict(context=context.clone(), init=init_token.clone(), beams=out[0], iterations=list(iterations)))
        return out

    reports: List[StepReport] = []
    prev_step = None  # what the previous step left for the cache comparison
    with mock.patch.object(tree_attention, "prepare_attention", w_prepare), \
            mock.patch.object(acceptance, "argmax_rows", w_argmax), \
            mock.patch.object(acceptance, "greedy_accept", w_accept), \
            mock.patch.object(acceptance, "realign_enqueue", w_realign), \
            mock.patch.object(loop_module, "_comprehend_prompt", w_prefill), \
            mock.patch.object(modeling_drafter, "beam_topk_step", w_topk), \
            mock.patch.object(drafter, "beam_search_candidates", w_draft):
        stream = model.generate(rd.stats.Ledger(), ids, max_length, rd.BeamShape(W, L),
                                rd.SamplingArgs(1.0, True), rd.SpecialTokens(pad, None))
        for k in range(steps):
            seen.pop("tree", None)
            try:
                out = next(stream)
            except StopIteration:
                break
            assert len(drafts) == k + 2
            if k == 0:
                with torch.inference_mode():
                    report = check_prefill(prefilled, llm, llm32, pad, tol, log=print)
                prefilled.clear()
                if prefill_report is not None:
                    prefill_report.append(report)
            st = dict(seen)
            if k >= check_from:
                with torch.inference_mode():
                    reports.append(_check_step(k, st, drafts[k], drafts[k + 1], out, max_length, llm, llm32,
                                               drafter, W, L, pad, tol, prev_step,
                                               natural_accept=force is None))
                if log is not None:
                    log(reports[-1])
            prev_step = dict(snap=st["snap"], tree=st["tree"], unpacker=st["unpacker"], n=st["n"], s=st["s"],
                             ids=st["ids"], prev=st["ids"].shape[1])
            drafts[k]["iterations"] = None  # (logits of a whole beam-search: not kept)
        stream.close()
    return reports


def check_prefill(pf, llm, llm32, pad: int, tol: float, log: Optional[Callable] = None) -> PrefillReport:
    """The prefill of the HIP loop against oracle/torch_path's in float32 on the same token ids."""
    ids, rows = pf["ids"], pf["rows"]  # rows: (layers, 2, B, Hkv, S, D), the reference's layout
    dev = ids.device
    B, S = ids.shape
    n_layers, _, _, Hkv, _, D = rows.shape
    pads = P.count_left_pads(ids, pad)
    mask = P.causal_mask(ids != pad, S)
    pos = torch.arange(S, device=dev).expand(B, S) - pads[:, None]

    def restate(model, dtype):
        cache = P.Cache(B, S, n_layers, Hkv, D, dtype, dev)
        logits, hidden = P.llama_forward(model, ids, mask, pos, cache)
        return cache.data.float(), hidden[:, -1, :].float(), logits[:, -1, :]

    want_rows, want_state, want_logits = restate(llm32, torch.float32)
    torch_rows, torch_state, _ = restate(llm, rows.dtype)
    live = (torch.arange(S, device=dev)[None, :] >= pads[:, None])[None, None, :, None, :, None]
    zero = torch.zeros((), device=dev)
    # per layer (errors grow through the residual stream), each against the layer's own scale
    per_layer = lambda x: torch.where(live, x, zero).abs().amax(dim=(1, 2, 3, 4, 5))
    layer_scale = per_layer(want_rows)
    layer_err = per_layer(rows.float() - want_rows) / layer_scale
    layer_yard = per_layer(torch_rows - want_rows) / layer_scale
    kv_err, kv_yard = float(layer_err.max()), float(layer_yard.max())
    state_scale = float(want_state.abs().max())
    state_err = float((pf["state"].float() - want_state).abs().max()) / state_scale
    state_yard = float((torch_state - want_state).abs().max()) / state_scale
    if log is not None:
        log("prefill cache rows, error by layer (HIP / stock torch in the model's dtype): " + " ".join(
            f"{i}:{float(layer_err[i]):.1e}/{float(layer_yard[i]):.1e}" for i in sorted({0, n_layers // 4, n_layers // 2, 3 * n_layers // 4, n_layers - 1})))
        log(f"prefill last hidden state {state_err:.2e} (stock torch {state_yard:.2e})")
    # `tol` of the scale, or what stock torch's own ops in this dtype make of the same inputs (at
    # depth the rounding of 16-bit residual streams is the larger of the two)
    assert bool((layer_err <= torch.clamp(3 * layer_yard + 1e-3, min=tol)).all()), \
        f"prefill: cache rows off by {kv_err:.3g} of their scale, stock torch {kv_yard:.3g}"
    assert bool((layer_err <= 3 * layer_yard + 1e-3).all()), f"prefill: cache rows {kv_err:.3g} off, stock torch only {kv_yard:.3g}"
    assert state_err <= max(tol, 3 * state_yard + 1e-3), f"prefill: last hidden state off by {state_err:.3g} of its scale"
    assert state_err <= 3 * state_yard + 1e-3, f"prefill: last hidden state {state_err:.3g} off, stock torch only {state_yard:.3g}"
    o_tok = want_logits.argmax(dim=-1)
    flipped = (pf["token"] != o_tok).nonzero().flatten()
    scale = float(want_logits.abs().max())
    margins = (want_logits[flipped, o_tok[flipped]] - want_logits[flipped, pf["token"][flipped]]) / scale
    worst = float(margins.max()) if flipped.numel() else 0.0
    assert worst <= tol, f"prefill: first token flipped with float32 margin {worst:.3g} of the scale"
    return PrefillReport(S, kv_err, kv_yard, state_err, state_yard, int(flipped.numel()), worst)


def _check_beam_iterations(k, iterations) -> float:
    """Every iteration of the HIP beam search against the oracle's iteration on the same logits and
    scores (modeling_drafter.py:201-215).  Returns the lowest share of common picks."""
    lowest = 1.0
    for it, rec in enumerate(iterations):
        logits, lpb = rec["logits"].cpu(), rec["lpb"].cpu()
        o_lpb, o_tok, o_par, o_logp = O.beam_search_step(logits, lpb)
        live = o_logp.float() > -1000
        # one rounding step of a log-probability in the drafter's dtype (float32: of a score near 50000)
        tol = 2.0 ** -7 * float(o_logp.float()[live].abs().max()) if logits.dtype != torch.float32 else 1e-2
        try:
            shared = beam_band.check_selection(o_logp, lpb, o_lpb, o_tok, o_par, rec["new_lpb"], rec["tok"], rec["par"], tol)
        except AssertionError as e:
            raise AssertionError(f"step {k}, beam-search iteration {it}: {e}") from e
        lowest = min(lowest, shared)
    return lowest


def _check_step(k, st, draft_in, draft_next, out, max_length, llm, llm32, drafter, W, L, pad, tol, prev_step,
                natural_accept: bool) -> StepReport:
    tree, ids, beams = st["tree"], st["ids"], st["beams"]
    dev = ids.device
    B, prev = ids.shape
    n_q, total = tree.n, tree.total
    rows = tree.rows()
    slot_of_row = rows.index[:total]  # slot b * n_q + t of every packed row that exists
    assert torch.equal(beams, draft_in["beams"])

    # -- draft: the restatement's beam search on the same context and token -----------------------
    with torch.inference_mode():
        o_beams, _ = P.beam_search(drafter, llm.model.embed_tokens, draft_in["context"], draft_in["init"], W, L,
                                   want_log_probs=False)
    beams_equal = bool(torch.equal(o_beams, beams))
    # bf16 beam scores tie or nearly tie in numbers (the restatement computes the first iteration for
    # all W copies of the one live beam, the package once per row: other GEMM shapes, other rounding),
    # so the two searches may keep different candidates at the margin; the share in common is reported
    beams_shared = float((beams[:, :, None, :] == o_beams[:, None, :, :]).all(-1).any(-1).float().mean())
    assert torch.equal(beams[:, :, 0], draft_in["init"][:, None].expand(B, W))
    assert len(draft_in["iterations"]) == L - 1
    beam_picks_shared = _check_beam_iterations(k, draft_in["iterations"])
    assert beam_picks_shared >= 0.97, f"step {k}: only {beam_picks_shared:.3f} of the HIP picks are the oracle's on the same logits"

    # -- tree of the HIP beams: bit-exact ----------------------------------------------------------
    o_packed, o_unpacker, o_mask, o_off = P.pack(beams, (ids != pad).to(ids.dtype))
    assert o_packed.shape[1] == n_q, (o_packed.shape, n_q)
    assert torch.equal(tree.unpacker, o_unpacker) and torch.equal(tree.packed_beams, o_packed)
    assert torch.equal(tree.position_offsets, o_off) and torch.equal(_bits_to_mask(st["bits"], prev + n_q), o_mask)
    counts = tree.counts[:B].long()
    assert int(counts.sum()) == total and int(counts.max()) == n_q
    exists = (torch.arange(n_q, device=dev)[None, :] < counts[:, None]).flatten()
    assert torch.equal(exists.nonzero().flatten(), slot_of_row)

    # -- verify forward: float32 restatement (and the bf16 one as the yardstick) on the same cache ---
    snap = st["snap"]  # (layers, 2, B, H, max_len, D), columns in place, tree rows at [prev, prev+n_q)
    pos = (prev - P.count_left_pads(ids, pad))[:, None] + o_off
    assert torch.equal(st["position_ids"], pos) and torch.equal(st["left_pads"].long(), P.count_left_pads(ids, pad))
    n_layers, _, _, Hkv, max_len, D = snap.shape

    def restate(model, dtype):
        cache = P.Cache(B, prev + n_q, n_layers, Hkv, D, dtype, dev)
        cache.data[:, :, :, :, :prev] = snap[:, :, :, :, :prev].to(dtype)
        cache.set_length(prev)
        with torch.inference_mode():
            logits, hidden = P.llama_forward(model, o_packed, o_mask, pos, cache)
        return logits.flatten(0, 1)[slot_of_row], hidden.flatten(0, 1)[slot_of_row], cache

    want, want_hidden, o_cache = restate(llm32, torch.float32)
    torch_bf16, torch_hidden, torch_cache = restate(llm, snap.dtype)
    got = st["logits"][:total].float()
    scale = float(want.abs().max())
    logits_err = float((got - want).abs().max()) / scale
    yard = float((torch_bf16 - want).abs().max()) / scale
    assert logits_err <= tol, f"step {k}: packed logits off by {logits_err:.3g} of their scale"
    assert logits_err <= 3 * yard + 1e-3, \
        f"step {k}: HIP logits {logits_err:.3g} off, stock bf16 torch only {yard:.3g}"

    # -- argmax: flips only inside the tolerance band ---------------------------------------------------
    hip_tok = st["argmax"][:total]
    assert torch.equal(st["llm_tokens"].flatten()[slot_of_row], hip_tok)
    o_tok = want.argmax(dim=-1)
    flipped = (hip_tok != o_tok).nonzero().flatten()
    margins = (want[flipped, o_tok[flipped]] - want[flipped, hip_tok[flipped]]) / scale
    worst = float(margins.max()) if flipped.numel() else 0.0
    assert worst <= tol, f"step {k}: argmax flip with float32 margin {worst:.3g} of the scale"
    # and the HIP argmax is the first maximum of the HIP logits themselves
    assert torch.equal(hip_tok, st["logits"][:total].float().argmax(dim=-1))

    # -- acceptance from the HIP tokens: bit-exact -------------------------------------------------------
    llm_bwl = st["llm_tokens"].gather(1, o_unpacker.view(B, -1)).view(B, W, L)
    o_n, o_s = P.greedy_choose(beams, llm_bwl)
    nat_n, nat_s = st["natural"]
    assert torch.equal(o_n, nat_n) and torch.equal(o_s, nat_s)
    n, s = st["n"], st["s"]
    if natural_accept:
        assert torch.equal(n, nat_n) and torch.equal(s, nat_s)
    b_idx = torch.arange(B, device=dev)
    assert torch.equal(st["next_tokens"], llm_bwl[b_idx, s, n])
    assert torch.equal(st["last_slot"], o_unpacker[b_idx, s, n])

    # -- next state --------------------------------------------------------------------------------------
    dummy = np.zeros((1, 1, B, 1, prev + W * L, 1), dtype=np.float32)
    o_ids, M = Acc.update_kv_and_ids(ids.cpu().numpy(), n.cpu().numpy(), s.cpu().numpy(), beams.cpu().numpy(),
                                     dummy, pad)
    assert out.shape[1] == min(M + 1, max_length)
    if M + 1 <= max_length:  # (otherwise the yielded tokens are cut at max_length)
        assert np.array_equal(out[:, :-1].cpu().numpy(), o_ids)
        assert torch.equal(out[:, -1], st["next_tokens"])
    assert torch.equal(draft_next["init"], st["next_tokens"])
    ctx_want = want_hidden.new_zeros((B * n_q, want_hidden.shape[1])).index_copy_(0, slot_of_row, want_hidden)
    ctx_want = ctx_want[b_idx * n_q + st["last_slot"]]
    ctx_scale = float(want_hidden.abs().max())
    context_err = float((draft_next["context"].float() - ctx_want).abs().max()) / ctx_scale
    ctx_torch = torch_hidden.new_zeros((B * n_q, torch_hidden.shape[1])).index_copy_(0, slot_of_row, torch_hidden)
    context_yard = float((ctx_torch[b_idx * n_q + st["last_slot"]].float() - ctx_want).abs().max()) / ctx_scale
    assert context_err <= tol, f"step {k}: drafter context off by {context_err:.3g}"

    # -- KV cache: the rows the HIP forward wrote against the restatement's; the rows kept and moved ----
    hip_new = snap[:, :, :, :, prev : prev + n_q].float()
    o_new = o_cache.data[:, :, :, :, prev : prev + n_q]
    live = (torch.arange(n_q, device=dev)[None, :] < counts[:, None])[None, None, :, None, :, None]
    kv_scale = float(o_new.abs().max())
    kv_err = float(torch.where(live, hip_new - o_new, torch.zeros_like(o_new)).abs().max()) / kv_scale
    kv_yard = float(torch.where(live, torch_cache.data[:, :, :, :, prev : prev + n_q].float() - o_new,
                                torch.zeros_like(o_new)).abs().max()) / kv_scale
    assert kv_err <= tol, f"step {k}: appended K/V rows off by {kv_err:.3g}"
    if prev_step is not None:
        # what the previous step kept: its live columns, then the accepted rows of its chosen beam,
        # bit for bit, at the columns the re-alignment gave them
        p = prev_step
        old_pads = P.count_left_pads(p["ids"], pad)
        new_pads = P.count_left_pads(ids, pad)
        for b in range(B):
            keep = p["prev"] - int(old_pads[b])
            lo = int(new_pads[b])
            assert torch.equal(snap[:, :, b, :, lo : lo + keep], p["snap"][:, :, b, :, int(old_pads[b]) : p["prev"]]), \
                f"step {k}: kept cache rows of row {b} changed"
            for j in range(int(p["n"][b]) + 1):
                src = p["prev"] + int(p["unpacker"][b, int(p["s"][b]), j])
                assert torch.equal(snap[:, :, b, :, lo + keep + j], p["snap"][:, :, b, :, src]), \
                    f"step {k}: accepted cache row {j} of row {b}"
            assert lo + keep + int(p["n"][b]) + 1 == prev
    return StepReport(k, prev, n_q, total, beams_equal, beams_shared, beam_picks_shared, logits_err, yard, int(flipped.numel()), worst,
                      n.tolist(), st["shift"].tolist(), context_err, kv_err, context_yard, kv_yard)
