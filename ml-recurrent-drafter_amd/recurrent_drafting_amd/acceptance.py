"""Acceptance of drafted tokens and re-alignment of ids and KV cache (HIP kernels underneath).

Function names and argument meaning follow the module-level functions of the reference's
recurrent_drafting/recurrent_drafting.py; that module re-exports them.
"""

from __future__ import annotations

from dataclasses import dataclass
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


def argmax_rows(logits: torch.Tensor, rows=None) -> torch.Tensor:
    """torch.argmax(logits, dim=-1) with the first-maximum rule, one pass over the logits.

    rows (a packed_rows.PackedRows): logits holds one row per packed row, and the result comes back
    as (batch, n) with the argmax of every slot that exists at its place -- the kernel writes it
    there; the slots that do not exist hold whatever the allocation held (nothing reads them: the
    unpacker only names slots that exist)."""
    V = logits.shape[-1]
    lead = logits.shape[:-1]
    x = logits.reshape(-1, V)
    if x.stride(1) != 1:
        x = x.contiguous()
    if rows is None:
        n_rows, out, where = x.shape[0], torch.empty(x.shape[0], dtype=torch.long, device=x.device), None
    else:
        assert x.shape[0] == rows.rows
        n_rows, where = rows.total, rows.index
        out = torch.empty(rows.batch * rows.n, dtype=torch.long, device=x.device)
    _hip.check(
        _hip.lib().rd_argmax_rows(
            _hip.ptr(x), _hip.dtype_code(x.dtype), n_rows, V, x.stride(0), _hip.ptr(out), _hip.ptr(where),
            _hip.stream(),
        )
    )
    return out.view(lead) if rows is None else out.view(rows.batch, rows.n)


def _count_left_paddings(tokens: torch.Tensor, pad_token_id: int) -> torch.Tensor:
    """Leading run of pad ids per row, int64 (B,) (recurrent_drafting.py:387-388)."""
    return _count_left_paddings_int32(tokens, pad_token_id).to(torch.long)


def _count_left_paddings_int32(tokens: torch.Tensor, pad_token_id: int) -> torch.Tensor:
    """The same counts as the kernel leaves them (int32): one launch less for callers that only do
    arithmetic with them."""
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
    return pads


def tree_position_ids(input_ids: torch.Tensor, pad_token_id: int, position_offsets: torch.Tensor) -> torch.Tensor:
    """(B, n) int64 positions of the packed tree tokens: each row's token count so far (its length
    minus its left padding) plus the token's depth in the tree (recurrent_drafting.py:449-458)."""
    assert input_ids.dim() == 2 and input_ids.dtype == torch.long
    assert position_offsets.dim() == 2 and position_offsets.dtype == torch.long and position_offsets.stride(1) == 1
    if input_ids.shape[1] > 0 and input_ids.stride(1) != 1:
        input_ids = input_ids.contiguous()
    B, prev = input_ids.shape
    n = position_offsets.shape[1]
    assert position_offsets.shape[0] == B
    out = torch.empty((B, n), dtype=torch.long, device=input_ids.device)
    _hip.check(
        _hip.lib().rd_position_ids(
            _hip.ptr(input_ids) if prev > 0 else None, input_ids.stride(0), prev, B, pad_token_id,
            _hip.ptr(position_offsets), position_offsets.stride(0), n, _hip.ptr(out), _hip.stream(),
        )
    )
    return out


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


@dataclass
class PendingRealign:
    """The launches of `realign` are queued; the new length (one int32 at `new_len`, on the
    device) still has to reach the host."""

    ids_buf: torch.Tensor
    plan: torch.Tensor
    cache: kv_cache.Cache
    batch: int

    @property
    def new_len(self) -> torch.Tensor:
        return self.plan[:1]

    def finish(self, new_len: int) -> torch.Tensor:
        self.cache.set_length(new_len)
        return self.ids_buf[: self.batch * new_len].view(self.batch, new_len)


def realign_enqueue(
    input_ids: torch.Tensor,
    n_tokens_in_seq: torch.Tensor,
    seq_in_beam: torch.Tensor,
    beams: torch.Tensor,
    cache: kv_cache.Cache,
    pad_token_id: int,
    unpacker: Optional[torch.Tensor] = None,
    left_pads: Optional[torch.Tensor] = None,
    step_out: Optional[torch.Tensor] = None,
) -> PendingRealign:
    """Appends the accepted tokens to ids and cache and re-right-aligns both; nothing is read back.

    With unpacker=None the cache must already be unpacked (Cache.unpack); with the unpacker given
    the accepted rows are taken straight from the packed slots and the unpack step is not needed.
    left_pads: (B,) int32 leading pad counts of input_ids, if the caller has them already.
    step_out: two int32 on the device that receive the new length and the accepted tokens summed
    over the rows (for a caller that reads them together with something else)."""
    assert input_ids.dtype == torch.long, f"prev_input_ids.dtype {input_ids.dtype} is not long"
    B, W, L = beams.shape
    prev = input_ids.shape[1]
    assert left_pads is None or (left_pads.shape == (B,) and left_pads.dtype == torch.int32 and left_pads.is_contiguous())
    assert step_out is None or (step_out.shape == (2,) and step_out.dtype == torch.int32 and step_out.is_contiguous())
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
            B, W, L, pad_token_id, _hip.ptr(plan), _hip.ptr(ids_buf),
            _hip.ptr(cache.shift) if cache.rows_in_place else None, _hip.ptr(left_pads), _hip.ptr(step_out),
            _hip.stream(),
        )
    )
    if cache.rows_in_place:
        cache._shifted = True
    n_layers, batch, n_heads, max_len, row_bytes = cache._geometry()
    if cache.rows_in_place and L * (row_bytes // 16) <= 256:
        # no row moves: the accepted rows are appended behind the live ones
        _hip.check(
            lib.rd_kv_append(
                _hip.ptr(cache._cache), n_layers, batch, n_heads, max_len, row_bytes, L,
                _hip.ptr(plan), _hip.stream(),
            )
        )
    else:
        _hip.check(
            lib.rd_kv_compact(
                _hip.ptr(cache._cache), n_layers, batch, n_heads, max_len, row_bytes, prev, L,
                _hip.ptr(plan), _hip.stream(),
            )
        )
    return PendingRealign(ids_buf, plan, cache, B)


def realign(
    input_ids: torch.Tensor,
    n_tokens_in_seq: torch.Tensor,
    seq_in_beam: torch.Tensor,
    beams: torch.Tensor,
    cache: kv_cache.Cache,
    pad_token_id: int,
    unpacker: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """`realign_enqueue` and the one host read (the new length)."""
    pending = realign_enqueue(input_ids, n_tokens_in_seq, seq_in_beam, beams, cache, pad_token_id,
                              unpacker)
    return pending.finish(int(pending.new_len.item()))


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


# ---------------------------------------------------------------------------------------------
# speculative sampling
# ---------------------------------------------------------------------------------------------
import ctypes as _C  # noqa: E402
from dataclasses import dataclass  # noqa: E402

from . import modeling_drafter as _md  # noqa: E402


def _host_strides(t: torch.Tensor, n: int):
    assert t.stride(-1) == 1, "vocabulary dimension must be contiguous"
    return (_C.c_int64 * n)(*[t.stride(i) for i in range(n)])


@dataclass
class PackedLogP:
    """LLM log-probabilities in packed form: logits (B, n, V) + 4 floats per packed row."""

    logits: torch.Tensor
    stats: torch.Tensor  # (B, n, 4) float32
    unpacker: torch.Tensor  # (B, W, L) int64
    temperature: float


def verify_row_stats(logits: torch.Tensor, temperature: float, force_fallback: bool = False) -> torch.Tensor:
    """(B, n, V) verify logits -> (B, n, 4) float32 {thr, zmax, log_sum, mask_z}."""
    B, n, V = logits.shape
    x = _hip.aligned_rows(logits.reshape(B * n, V))
    stats = torch.empty((B, n, 4), dtype=torch.float32, device=logits.device)
    _hip.check(
        _hip.lib().rd_verify_row_stats(
            _hip.ptr(x), _hip.dtype_code(x.dtype), x.stride(0), B * n, V, _md.TOP_K, _md.LOG_0,
            float(temperature), _hip.ptr(stats), int(force_fallback), _hip.stream(),
        )
    )
    return stats


def _p_args(log_p):
    """Argument block (dense, dense_strides, logits, dtype, logits_strides, stats, n_rows, unpacker, T)."""
    if isinstance(log_p, PackedLogP):
        lg = log_p.logits
        assert lg.dim() == 3
        keep = (lg, log_p.stats, log_p.unpacker.contiguous())
        return keep, (None, None, _hip.ptr(lg), _hip.dtype_code(lg.dtype), _host_strides(lg, 2),
                      _hip.ptr(log_p.stats), lg.shape[1], _hip.ptr(keep[2]), float(log_p.temperature))
    assert log_p.dim() == 4 and log_p.dtype == torch.float32
    return (log_p,), (_hip.ptr(log_p), _host_strides(log_p, 3), None, 0, None, None, 0, None, 1.0)


def sample_accept(beams, log_p, log_q, uniforms) -> Tuple[torch.Tensor, torch.Tensor]:
    """(n_tokens_in_seq, seq_in_beam) with caller-supplied uniforms (B, W, L-1).

    log_p: dense (B, W, L, V) float32 or PackedLogP; log_q: (B, W, L-1, V) float32."""
    B, W, L = beams.shape
    V = log_q.shape[-1]
    assert beams.dtype in (torch.int32, torch.int64)
    beams = beams.to(torch.long).contiguous()
    assert log_q.shape == (B, W, L - 1, V) and log_q.dtype == torch.float32
    uniforms = uniforms.to(torch.float32).contiguous()
    assert uniforms.shape == (B, W, L - 1)
    keep, p_args = _p_args(log_p)
    out = torch.empty((2, B), dtype=torch.long, device=beams.device)
    _hip.check(
        _hip.lib().rd_accept_sample(
            _hip.ptr(beams), *p_args, _hip.ptr(log_q), _host_strides(log_q, 3), _hip.ptr(uniforms),
            B, W, L, V, _hip.ptr(out[0]), _hip.ptr(out[1]), _hip.stream(),
        )
    )
    return out[0], out[1]


def residual_probs(log_q, log_p, seq_in_beam, n_tokens_in_seq) -> torch.Tensor:
    """Unnormalised distribution of the next token, (B, V) float32."""
    B, W, Lm1, V = log_q.shape
    keep, p_args = _p_args(log_p)
    seq_in_beam = seq_in_beam.to(torch.long).contiguous()
    n_tokens_in_seq = n_tokens_in_seq.to(torch.long).contiguous()
    probs = torch.empty((B, V), dtype=torch.float32, device=log_q.device)
    _hip.check(
        _hip.lib().rd_residual_probs(
            *p_args, _hip.ptr(log_q), _host_strides(log_q, 3), _hip.ptr(seq_in_beam),
            _hip.ptr(n_tokens_in_seq), B, W, Lm1 + 1, V, _hip.ptr(probs), _hip.stream(),
        )
    )
    return probs


def _choose_from_candidates(beams, log_probs_by_llm, log_probs_by_drafter):
    """Drop-in for recurrent_drafting.py:499-556: draws torch.rand like the reference does."""
    B, W, L = beams.shape
    u = torch.rand((B, W, L - 1), device=log_probs_by_drafter.device)
    return sample_accept(beams, log_probs_by_llm.float(), log_probs_by_drafter.float(), u)


def _prepare_next_input(log_probs_by_drafter, log_probs_by_llm, last_hidden_state, seq_in_beam,
                        n_tokens_in_seq):
    """Drop-in for recurrent_drafting.py:271-343: (context (B, hidden), next_tokens (B,))."""
    import torch.distributions as dist

    probs = residual_probs(log_probs_by_drafter.float(), log_probs_by_llm.float(), seq_in_beam, n_tokens_in_seq)
    next_tokens = dist.Categorical(probs=probs).sample()
    B, W, L = last_hidden_state.shape[:3]
    flat = (seq_in_beam * L + n_tokens_in_seq).to(torch.long)
    state = _select_one_per_row(last_hidden_state.reshape(B, W * L, -1), flat)
    return state, next_tokens
