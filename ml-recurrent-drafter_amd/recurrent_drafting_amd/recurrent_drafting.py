"""The ReDrafter decode loop on the HIP hot path.

`RecurrentDrafting.generate` keeps the reference's signature and yields the same token tensors
(recurrent_drafting/recurrent_drafting.py:559-705).  One step is

    draft   beam search on the drafter head          rd_beam_topk x (L-1)      (+ torch GEMMs)
    verify  beams -> prefix tree, mask bits + plan +  rd_tree_build, rd_tree_attn_prepare,
            position ids, LLM forward                 rd_verify_attention per layer (+ torch GEMMs)
    accept  greedy: argmax over the packed rows,      rd_argmax_rows, rd_accept_greedy
            longest agreeing prefix
            sampling: row statistics of the packed    rd_verify_row_stats, rd_accept_sample,
            logits, u < P/Q run, residual resample    rd_residual_probs
            ids and KV re-aligned                     rd_realign_plan, rd_kv_compact

Greedy decoding never materialises the (B, W, L, V) logits, never unpacks the KV cache into W*L
slots and never clones it: argmax commutes with the unpack and with the top-50 filter, and the
accepted rows are taken straight from their packed slots.  One host read per step (new sequence
length, accepted tokens, packed tree length and slots of the coming step) where the reference has
more than ten.

The module-level helpers of the reference are re-exported with their names for code and tests that
call them directly.
"""

from __future__ import annotations

import contextlib
from dataclasses import dataclass
from typing import Generator, Optional, Tuple

import torch
import torch.distributions as dist
import transformers

from . import acceptance, attention, kv_cache, modeling_drafter, modeling_llama, stats, tree_attention
from .acceptance import (  # noqa: F401  (re-exported: the reference's helper names)
    _choose_from_candidates,
    _count_left_paddings,
    _greedy_choose_from_candidates,
    _greedy_prepare_next_input,
    _prepare_next_input,
    _select_one_per_row,
    _update_kv_cache_and_input_ids,
)

dist.Distribution.set_default_validate_args(False)


@dataclass
class SamplingArgs:
    temperature: float
    greedy: bool


@dataclass
class SpecialTokens:
    pad: int
    eos: Optional[int] = 1


def _comprehend_prompt(
    llm: transformers.PreTrainedModel,
    input_ids: torch.Tensor,
    cache: kv_cache.Cache,
    sampling_args: SamplingArgs,
    pad_token_id: int,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Prefill: fills the cache from the prompt and returns (last hidden state (B, hidden), first
    generated token (B,)) (recurrent_drafting.py:391-434)."""
    assert input_ids.dtype in [torch.int32, torch.int64]
    seq = input_ids.shape[1]
    mask = attention.causal_mask(input_ids != pad_token_id, seq, input_ids.device)
    pads = _count_left_paddings(input_ids.to(torch.long), pad_token_id)
    position_ids = torch.arange(seq, dtype=torch.long, device=input_ids.device).expand(
        input_ids.shape
    ) - pads.unsqueeze(-1)
    hidden = llm.hidden_states(input_ids, mask, position_ids, cache.sliced)
    last_state = hidden[:, -1, :]
    last_logits = llm.lm_head(last_state)  # argmax ignores the top-50 filter and the fp32 cast
    if sampling_args.greedy:
        next_token = acceptance.argmax_rows(last_logits)
    else:
        filtered = modeling_drafter.warp_logits(last_logits.float())
        probs = torch.softmax(filtered / sampling_args.temperature, dim=-1)
        next_token = dist.Categorical(probs=probs).sample()
    return last_state, next_token


def _verify_candidates(
    step_record: stats.TextGeneration.Step,
    llm: transformers.PreTrainedModel,
    input_ids: torch.Tensor,
    beams: torch.Tensor,
    cache: kv_cache.Cache,
    pad_token_id: int,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Drop-in for recurrent_drafting.py:437-465: returns unpacked (hidden (B,W,L,hid), filtered
    logits (B,W,L,V) float32) and leaves the cache unpacked.  `generate` does not use this form."""
    packed, unpacker, mask, offsets = tree_attention.pack(beams, input_ids != pad_token_id)
    pads = _count_left_paddings(input_ids, pad_token_id)
    position_ids = (cache.sliced[0][0].length - pads).unsqueeze(-1) + offsets
    with step_record.time("base_forward"):
        out = llm(packed, attention_mask=mask, past_key_values=cache.sliced, position_ids=position_ids)
    logits = modeling_drafter.warp_logits(out.logits)
    hidden = tree_attention.unpack(out.hidden_states, unpacker)
    logits = tree_attention.unpack(logits, unpacker)
    cache.unpack(input_ids.shape[-1], unpacker)
    return hidden, logits


def _greedy_accept_candidate_tokens(input_ids, beams_by_drafter, logits_by_llm, last_hidden_state,
                                    cache, pad_token_id, step_record):
    """Drop-in for recurrent_drafting.py:43-72 (unpacked logits and hidden states, unpacked cache)."""
    beams_by_llm = acceptance.argmax_rows(logits_by_llm)
    with step_record.time("choose_from_candidates"):
        n_tokens, seq_in_beam = _greedy_choose_from_candidates(beams_by_drafter, beams_by_llm)
    with step_record.time("update_kv_cache_and_input_ids"):
        input_ids = _update_kv_cache_and_input_ids(
            input_ids, n_tokens, seq_in_beam, beams_by_drafter, cache, pad_token_id)
    with step_record.time("greedy_prepare_next_input"):
        state, next_tokens = _greedy_prepare_next_input(
            beams_by_llm, last_hidden_state, seq_in_beam, n_tokens)
    return state, input_ids, next_tokens, n_tokens


def _accept_candidate_tokens(input_ids, beams, log_probs_by_drafter, logits_by_llm,
                             last_hidden_state, cache, pad_token_id, temperature, step_record):
    """Drop-in for recurrent_drafting.py:75-111.  This form materialises the (B, W, L, V)
    log-softmax like the reference; `generate` uses the packed form instead."""
    log_probs_by_llm = (logits_by_llm / temperature).log_softmax(dim=-1)
    with step_record.time("choose_from_candidates"):
        n_tokens, seq_in_beam = _choose_from_candidates(beams, log_probs_by_llm, log_probs_by_drafter)
    with step_record.time("update_kv_cache_and_input_ids"):
        input_ids = _update_kv_cache_and_input_ids(
            input_ids, n_tokens, seq_in_beam, beams, cache, pad_token_id)
    with step_record.time("prepare_next_input"):
        state, next_tokens = _prepare_next_input(
            log_probs_by_drafter, log_probs_by_llm, last_hidden_state, seq_in_beam, n_tokens)
    return state, input_ids, next_tokens, n_tokens


class RecurrentDrafting(torch.nn.Module):
    def __init__(self, llm: transformers.PreTrainedModel, drafter: modeling_drafter.Drafter):
        super().__init__()
        self.llm = llm
        self.drafter = drafter
        # True: the decode loop leaves the KV cache rows where they are when the ids are re-aligned
        # (kv_cache.Cache.rows_in_place); False: it moves them every step, as the reference does.
        self.kv_rows_in_place = True

    def llm_n_kv_heads(self) -> int:
        if isinstance(self.llm, modeling_llama.LlamaForCausalLM):
            return self.llm.config.num_key_value_heads
        raise TypeError(f"Unsupported base model type {type(self.llm)}")

    def generate(
        self,
        ledger: stats.Ledger,
        input_ids: torch.Tensor,
        max_length: int,
        beam_shape: modeling_drafter.BeamShape = modeling_drafter.BeamShape(10, -1),
        sampling_args: SamplingArgs = SamplingArgs(1.0, False),
        special_tokens: SpecialTokens = SpecialTokens(0, 1),
    ) -> Generator[torch.Tensor, None, None]:
        with torch.inference_mode():
            with stats.text_generation(ledger) as record:
                yield from self._generate(
                    record, input_ids, max_length, beam_shape, sampling_args, special_tokens
                )

    # -- the fused path ---------------------------------------------------------------------------
    # A step is split where its host reads are.  `_draft` queues the beam search and the tree
    # build of the COMING step; `_verify_and_accept` queues mask, model forward, acceptance and
    # re-alignment of the current one.  Between two steps the host then needs four integers (new
    # sequence length, accepted tokens, packed tree length, tree slots) and fetches them in ONE
    # read, after the next step's draft has been queued: the drafter's many small launches run
    # behind the model forward instead of in front of an idle GPU.
    def _draft(self, step_record, context, init_tokens, beam_shape, greedy, counts=None) -> "_Drafted":
        # every step times one draft, the one it queues for its successor; the very first draft
        # (step_record None) is not timed, so that each timer key keeps one entry per step
        timer = step_record.time("generate_candidates") if step_record is not None else contextlib.nullcontext()
        with timer:
            beams, log_q = self.drafter.beam_search_candidates(
                context, init_tokens, self.llm.base_model.get_input_embeddings(), beam_shape,
                return_log_probs=not greedy,
            )
            return _Drafted(beams, log_q, tree_attention.build_tree_enqueue(beams, counts))

    def _verify_and_accept(self, step_record, drafted, tree, input_ids, cache, pad, sampling_args, step_out=None):
        """-> (context, next_tokens, n_tokens, realignment still to be finished)."""
        llm, beams = self.llm, drafted.beams
        greedy = sampling_args.greedy
        with step_record.time("verify_candidates"):
            # mask bits, work plan, position ids and left pad counts of the packed tree in one launch:
            # no byte mask, no `input_ids != pad`
            mask, position_ids, left_pads = tree_attention.prepare_attention(
                tree, input_ids, pad_value=pad, n_heads=llm.config.num_attention_heads,
                kv_shift=cache.shift if cache.rows_in_place else None)
            # the slots past a row's own tree are padding (other rows' tokens, tree_attention.py:70-122)
            # that the reference computes and never reads: the model runs on the slots that exist
            rows = tree.rows()
            with step_record.time("base_forward"):
                hidden = llm.hidden_states(tree.packed_beams, mask, position_ids, cache.sliced, rows)
                if greedy:
                    logits = llm.lm_head(hidden)  # (total, V) in the model's dtype
                else:
                    # the hidden states go back to their slots before the head: the sampling
                    # kernels address the logits as (batch row, slot)
                    hidden = rows.spread(hidden)
                    logits = llm.lm_head(hidden)
        with step_record.time("accept_candidate_tokens"):
            if greedy:
                llm_tokens = acceptance.argmax_rows(logits, rows)  # (B, n): per packed slot, written in place
                with step_record.time("choose_from_candidates"):
                    n_tokens, seq_in_beam, next_tokens, last_slot = acceptance.greedy_accept(
                        beams, llm_tokens, tree.unpacker
                    )
            else:
                # four floats per packed row stand in for the filtered, tempered log-softmax tensors
                temperature = sampling_args.temperature
                log_p = acceptance.PackedLogP(
                    logits, acceptance.verify_row_stats(logits, temperature), tree.unpacker, temperature)
                with step_record.time("choose_from_candidates"):
                    B, W, L = beams.shape
                    uniforms = torch.rand((B, W, L - 1), device=beams.device)
                    n_tokens, seq_in_beam = acceptance.sample_accept(beams, log_p, drafted.log_q, uniforms)
            with step_record.time("update_kv_cache_and_input_ids"):
                realignment = acceptance.realign_enqueue(
                    input_ids, n_tokens, seq_in_beam, beams, cache, pad, unpacker=tree.unpacker,
                    left_pads=left_pads, step_out=step_out,
                )
            if greedy:
                with step_record.time("greedy_prepare_next_input"):
                    context = tree_attention.gather_rows(hidden, last_slot.unsqueeze(-1), rows=rows)[:, 0, :]
            else:
                with step_record.time("prepare_next_input"):
                    probs = acceptance.residual_probs(drafted.log_q, log_p, seq_in_beam, n_tokens)
                    next_tokens = dist.Categorical(probs=probs).sample()
                    batch_rows = torch.arange(B, device=beams.device)
                    last_slot = tree.unpacker[batch_rows, seq_in_beam, n_tokens]
                    context = tree_attention.gather_rows(hidden, last_slot.unsqueeze(-1))[:, 0, :]
        return context, next_tokens, n_tokens, realignment

    def _generate(self, text_generation, input_ids, max_length, beam_shape, sampling_args,
                  special_tokens) -> Generator[torch.Tensor, None, None]:
        assert input_ids.dtype == torch.long, f"input_ids.dtype {input_ids.dtype} is not long"
        batch_size, seq_len = input_ids.shape
        init_seq_len = seq_len
        cfg = self.llm.config
        # The cache rows stay in place when the ids are re-aligned (kv_cache.Cache.rows_in_place): a row
        # can then end up to its initial left padding further right than the ids do.
        initial_pads = int(acceptance._count_left_paddings(input_ids, special_tokens.pad).max()) if seq_len else 0
        cache = kv_cache.Cache(
            batch_size=batch_size,
            max_length=max_length + beam_shape.length * beam_shape.width + initial_pads,
            n_layers=cfg.num_hidden_layers,
            n_heads=self.llm_n_kv_heads(),
            head_dim=cfg.hidden_size // cfg.num_attention_heads,
            dtype=self.llm.dtype,
            device=input_ids.device,
        )
        context, init_tokens = _comprehend_prompt(
            self.llm, input_ids, cache, sampling_args, special_tokens.pad
        )
        cache.rows_in_place = self.kv_rows_in_place
        drafted, tree = None, None  # what has been drafted for the coming step
        while seq_len < max_length:
            with text_generation.step() as step_record:
                if drafted is None:  # first step: nothing was drafted ahead
                    drafted = self._draft(None, context, init_tokens, beam_shape, sampling_args.greedy)
                    tree = drafted.tree.finish(*drafted.tree.sizes.tolist())
                # what the host needs between two steps lands in one small buffer: the coming tree's
                # counts, sizes and row starts (2B+3 ints), then the new length and the accepted tokens
                step_ints = torch.empty(2 * batch_size + 5, dtype=torch.int32, device=input_ids.device)
                context, init_tokens, n_tokens, realignment = self._verify_and_accept(
                    step_record, drafted, tree, input_ids, cache, special_tokens.pad, sampling_args,
                    step_out=step_ints[2 * batch_size + 3:])
                drafted = self._draft(step_record, context, init_tokens, beam_shape, sampling_args.greedy,
                                      counts=step_ints)
                # the one host read of the step
                read = step_ints[batch_size:].tolist()
                tree_n, tree_total, new_len, n_accepted = read[0], read[1], read[-2], read[-1]
                input_ids = realignment.finish(new_len)
                tree = drafted.tree.finish(tree_n, tree_total)
                output_tokens = torch.cat((input_ids, init_tokens.unsqueeze(-1)), dim=-1)
                seq_len = output_tokens.shape[1]
                step_record.set(
                    {
                        "input_id_length": seq_len,
                        "avg_num_accepted": n_accepted / batch_size,
                    }
                )
                yield output_tokens[:, :max_length] if seq_len > max_length else output_tokens
                if special_tokens.eos is not None:
                    ended = (output_tokens[:, init_seq_len:] == special_tokens.eos).any(dim=-1)
                    if bool(ended.all()):
                        break


@dataclass
class _Drafted:
    beams: torch.Tensor  # (B, W, L) int64
    log_q: Optional[torch.Tensor]  # (B, W, L-1, V) float32, sampling only
    tree: tree_attention.PendingTree
