"""Acceptance of drafted tokens and re-alignment of ids and KV cache (HIP kernels underneath).

Function names and argument meaning follow the module-level functions of the reference's
recurrent_drafting/recurrent_drafting.py; that module re-exports them.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _hip, kv_cache, tree_attention


def _select_one_per_row(x: torch.Tensor, batch_index: torch.Tensor) -> torch.Tensor:
    """x (B, S, ...), batch_index (B,) -> x[b, batch_index[b]] (recurrent_drafting.py:37-40)."""
    B, S = x.shape[0], x.shape[1]
    rest = x.shape[2:]
    flat = x.reshape(B, S, -1)
    out = tree_attention.gather_rows(flat, batch_index.reshape(B, 1).to(torch.long))
    return out.view((B,) + tuple(rest))


def argmax_rows(logits: torch.Tensor) -> torch.Tensor:
    """torch.argmax(logits, dim=-1) with the first-maximum rule, one pass over the logits."""
    V = logits.shape[-1]
    lead = logits.shape[:-1]
    x = logits.reshape(-1, V)
    if x.stride(1) != 1:
        x = x.contiguous()
    out = torch.empty(x.shape[0], dtype=torch.long, device=x.device)
    _hip.check(
        _hip.lib().rd_argmax_rows(
            _hip.ptr(x), _hip.dtype_code(x.dtype), x.shape[0], V, x.stride(0), _hip.ptr(out),
            _hip.stream(),
        )
    )
    return out.view(lead)


def _count_left_paddings(tokens: torch.Tensor, pad_token_id: int) -> torch.Tensor:
    """Leading run of pad ids per row, int64 (B,) (recurrent_drafting.py:387-388)."""
    assert tokens.dim() == 2 and tokens.dtype == torch.long
    if tokens.shape[1] > 0 and tokens.stride(1) != 1:
        tokens = tokens.contiguous()
    B, prev = tokens.shape
    pads = torch.empty(B, dtype=torch.int32, device=tokens.device)
    _hip.check(
        _hip.lib().rd_count_left_paddings(
            _hip.ptr(tokens) if prev > 0 else None, tokens.stride(0), prev, B, pad_token_id,
            _hip.ptr(pads), _hip.stream(),
        )
    )
    return pads.to(torch.long)


def greedy_accept(
    beams_by_drafter: torch.Tensor,
    llm_tokens: torch.Tensor,
    unpacker: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(n_tokens_in_seq, seq_in_beam, next_token, last_slot), each (B,) int64.

    llm_tokens is (B, W, L) when unpacker is None, else (B, n) indexed per packed slot."""
    B, W, L = beams_by_drafter.shape
    assert beams_by_drafter.dtype == torch.long and llm_tokens.dtype == torch.long
    beams_by_drafter = beams_by_drafter.contiguous()
    llm_tokens = llm_tokens.contiguous()
    stride = llm_tokens.shape[1] if unpacker is not None else W * L
    if unpacker is not None:
        unpacker = unpacker.contiguous()
        assert unpacker.shape == (B, W, L)
    else:
        assert llm_tokens.shape == (B, W, L)
    out = torch.empty((4, B), dtype=torch.long, device=beams_by_drafter.device)
    _hip.check(
        _hip.lib().rd_accept_greedy(
            _hip.ptr(beams_by_drafter), _hip.ptr(llm_tokens), stride, _hip.ptr(unpacker), B, W, L,
            _hip.ptr(out[0]), _hip.ptr(out[1]), _hip.ptr(out[2]), _hip.ptr(out[3]), _hip.stream(),
        )
    )
    return out[0], out[1], out[2], out[3]


def _greedy_choose_from_candidates(
    beams_by_drafter: torch.Tensor, beams_by_llm: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor]:
    """(n_tokens_in_seq, seq_in_beam) (recurrent_drafting.py:468-496)."""
    n, s, _, _ = greedy_accept(beams_by_drafter.to(torch.long), beams_by_llm.to(torch.long))
    return n, s


def _greedy_prepare_next_input(
    beams_by_llm: torch.Tensor,
    last_hidden_state: torch.Tensor,
    seq_in_beam: torch.Tensor,
    n_tokens_in_seq: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """(context (B, hidden), next_tokens (B,)) at [b, seq_in_beam, n_tokens_in_seq]
    (recurrent_drafting.py:235-268)."""
    B, W, L = beams_by_llm.shape
    flat = (seq_in_beam * L + n_tokens_in_seq).to(torch.long)
    next_tokens = _select_one_per_row(beams_by_llm.reshape(B, W * L), flat)
    state = _select_one_per_row(last_hidden_state.reshape(B, W * L, -1), flat)
    return state, next_tokens


def realign(
    input_ids: torch.Tensor,
    n_tokens_in_seq: torch.Tensor,
    seq_in_beam: torch.Tensor,
    beams: torch.Tensor,
    cache: kv_cache.Cache,
    pad_token_id: int,
    unpacker: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Appends the accepted tokens to ids and cache and re-right-aligns both.

    With unpacker=None the cache must already be unpacked (Cache.unpack); with the unpacker given
    the accepted rows are taken straight from the packed slots and the unpack step is not needed.
    One host read (the new length)."""
    assert input_ids.dtype == torch.long, f"prev_input_ids.dtype {input_ids.dtype} is not long"
    B, W, L = beams.shape
    prev = input_ids.shape[1]
    if prev > 0 and input_ids.stride(1) != 1:
        input_ids = input_ids.contiguous()
    beams = beams.contiguous()
    n_tokens_in_seq = n_tokens_in_seq.to(torch.long).contiguous()
    seq_in_beam = seq_in_beam.to(torch.long).contiguous()
    if unpacker is not None:
        unpacker = unpacker.contiguous()
    lib = _hip.lib()
    dev = input_ids.device
    plan = torch.empty(lib.rd_realign_plan_ints(B, L), dtype=torch.int32, device=dev)
    ids_buf = torch.empty(B * (prev + L), dtype=torch.long, device=dev)
    _hip.check(
        lib.rd_realign_plan(
            _hip.ptr(input_ids) if prev > 0 else None, input_ids.stride(0), prev,
            _hip.ptr(n_tokens_in_seq), _hip.ptr(seq_in_beam), _hip.ptr(beams), _hip.ptr(unpacker),
            B, W, L, pad_token_id, _hip.ptr(plan), _hip.ptr(ids_buf), _hip.stream(),
        )
    )
    # the KV move does not depend on the host read below, so it is enqueued first
    _hip.check(
        lib.rd_kv_compact(
            _hip.ptr(cache._cache), *cache._geometry()[:4], cache._geometry()[4], prev, L,
            _hip.ptr(plan), _hip.stream(),
        )
    )
    new_len = int(plan[0].item())
    cache.set_length(new_len)
    return ids_buf[: B * new_len].view(B, new_len)


def _update_kv_cache_and_input_ids(
    input_ids: torch.Tensor,
    n_tokens_in_seq: torch.Tensor,
    seq_in_beam: torch.Tensor,
    beams: torch.Tensor,
    cache: kv_cache.Cache,
    pad_token_id: int,
) -> torch.Tensor:
    """Drop-in for recurrent_drafting.py:114-232: expects the cache unpacked by Cache.unpack."""
    return realign(input_ids, n_tokens_in_seq, seq_in_beam, beams, cache, pad_token_id)
