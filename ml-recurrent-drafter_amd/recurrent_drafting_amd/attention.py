"""Attention masks and the masked attention itself.

`causal_mask`, `set_sdpa_fully_masked_rows` and `bias` keep the reference's signatures
(recurrent_drafting/attention.py).  The model forward does not build an additive bias: it calls
`prepare` once per forward (where the reference calls `bias`) and `masked_attention` per layer
(where the reference calls F.scaled_dot_product_attention).
"""

from __future__ import annotations

import ctypes as C
import math
from dataclasses import dataclass
from typing import Optional

import torch

from . import _hip
from .packed_rows import PackedRows


def causal_mask(padding_mask: torch.Tensor, query_len: int, device: torch.device) -> torch.Tensor:
    """(batch, kv) padding mask -> (batch, query_len, kv) bool (attention.py:12-55)."""
    assert padding_mask.dtype in [torch.int32, torch.int64, torch.bool]
    assert query_len > 0
    batch, kv_len = padding_mask.shape
    if padding_mask.stride(1) != 1:
        padding_mask = padding_mask.contiguous()
    out = torch.empty((batch, query_len, kv_len), dtype=torch.bool, device=padding_mask.device)
    _hip.check(
        _hip.lib().rd_causal_mask(
            _hip.ptr(padding_mask), padding_mask.element_size(), padding_mask.stride(0), batch,
            kv_len, query_len, _hip.ptr(out), _hip.stream(),
        )
    )
    return out


def set_sdpa_fully_masked_rows(causal_mask: torch.Tensor) -> torch.Tensor:
    """A row that attends to nothing attends to everything (attention.py:58-72)."""
    assert causal_mask.dtype in [torch.int32, torch.int64, torch.bool]
    dead = causal_mask.eq(0).all(dim=-1, keepdim=True)
    return causal_mask.masked_fill(dead, True)


def bias(causal_mask: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """0 where attended, finfo(dtype).min elsewhere (attention.py:75-88).  Kept for callers that
    want the additive form; the HIP attention consumes the mask itself."""
    out = torch.zeros(causal_mask.shape, dtype=dtype, device=causal_mask.device)
    return out.masked_fill_(causal_mask.logical_not(), torch.finfo(dtype).min)


@dataclass
class PreparedMask:
    """Bit-packed mask and work plan shared by every layer of one forward."""

    bits: torch.Tensor  # (B, n_q, words) int64 holding uint64 words
    plan: torch.Tensor  # int32
    batch: int
    n_q: int
    kv_len: int
    workspace: Optional[torch.Tensor] = None
    shifted: bool = False  # the plan was built with per-row cache shifts (kv_cache.Cache.shift)


def prepare(mask: torch.Tensor, fix_empty_rows: bool = True, n_heads: int = 32,
            kv_shift: Optional[torch.Tensor] = None) -> PreparedMask:
    """mask: (B, n_q, kv_len) bool/uint8, keys contiguous.  n_heads: query heads of the attention
    calls that will use the result (only sizes the work items).  kv_shift: (B,) int32 or None; key
    column c of row b is then read from row c - kv_shift[b] of k and v (kv_cache.Cache.shift)."""
    assert mask.dim() == 3 and mask.dtype in (torch.bool, torch.uint8)
    if mask.stride(2) != 1:
        mask = mask.contiguous()
    B, n_q, kv_len = mask.shape
    assert kv_shift is None or (kv_shift.shape == (B,) and kv_shift.dtype == torch.int32 and kv_shift.is_contiguous())
    lib = _hip.lib()
    dev = mask.device
    bits = torch.empty(lib.rd_attn_bits_words(B, n_q, kv_len), dtype=torch.int64, device=dev)
    plan = torch.empty(lib.rd_attn_plan_ints(B, n_q, kv_len), dtype=torch.int32, device=dev)
    _hip.check(
        lib.rd_attn_prepare(
            _hip.ptr(mask), mask.stride(0), mask.stride(1), B, n_q, kv_len, int(n_heads),
            int(fix_empty_rows),
            _hip.ptr(bits), _hip.ptr(plan), _hip.ptr(kv_shift), _hip.stream(),
        )
    )
    return PreparedMask(bits.view(B, n_q, -1), plan, B, n_q, kv_len, shifted=kv_shift is not None)


# When set to a list, every masked_attention call appends (batch, n_q, kv_len, query rows): measurement
# harnesses pair it with the library's per-kernel event timing to price the work that was done.
shape_log: Optional[list] = None


def _strides3(t: torch.Tensor):
    assert t.dim() == 4 and t.stride(3) == 1, "last dimension must be contiguous"
    return (C.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2))


def masked_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    prepared: PreparedMask,
    scale: Optional[float] = None,
    force_generic: bool = False,
    rows: Optional[PackedRows] = None,
) -> torch.Tensor:
    """q (B, H, n_q, D) [any strides with D contiguous], k/v (B, Hkv, kv_len, D) strided views.

    Returns (B, n_q, H*D), i.e. already in the layout o_proj consumes.  With `rows`, q is
    (rows.rows, H, D), the query rows that exist (and the stand-in rows behind them, which are
    neither read nor written), and the result is (rows.rows, H*D)."""
    Bk, Hkv, kv_len, Dk = k.shape
    if rows is None:
        B, H, n_q, D = q.shape
    else:
        T, H, D = q.shape
        B, n_q = rows.batch, rows.n
        assert T == rows.rows
    assert (Bk, Dk) == (B, D) and v.shape == k.shape and q.dtype == k.dtype == v.dtype
    assert (prepared.batch, prepared.n_q, prepared.kv_len) == (B, n_q, kv_len), "mask/plan mismatch"
    if q.stride(-1) != 1:
        q = q.contiguous()
    if k.stride(3) != 1:
        k = k.contiguous()
    if v.stride(3) != 1:
        v = v.contiguous()
    if rows is None:
        out = torch.empty((B, n_q, H, D), dtype=q.dtype, device=q.device)
        q_strides = _strides3(q)
        o_strides = _strides3(out.permute(0, 2, 1, 3))  # (B, H, n_q, D) strides
    else:
        out = torch.empty((rows.rows, H, D), dtype=q.dtype, device=q.device)
        q_strides = (C.c_int64 * 3)(0, q.stride(1), q.stride(0))
        o_strides = (C.c_int64 * 3)(0, out.stride(1), out.stride(0))
    lib = _hip.lib()
    ws_bytes = lib.rd_attention_workspace_bytes(B, H, n_q, kv_len, D)
    if prepared.workspace is None or prepared.workspace.numel() < ws_bytes:
        prepared.workspace = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=q.device)
    if shape_log is not None:
        shape_log.append((B, n_q, kv_len, B * n_q if rows is None else rows.total))
    _hip.check(
        lib.rd_verify_attention(
            _hip.ptr(q), q_strides, _hip.ptr(k), _strides3(k), _hip.ptr(v), _strides3(v),
            _hip.ptr(out), o_strides, _hip.dtype_code(q.dtype), B, H, Hkv, n_q, kv_len, D,
            float(scale if scale is not None else 1.0 / math.sqrt(D)), _hip.ptr(prepared.bits),
            _hip.ptr(prepared.plan), _hip.ptr(prepared.workspace), prepared.workspace.numel(),
            int(force_generic), _hip.ptr(rows.row_start) if rows is not None else None,
            _hip.stream(),
        )
    )
    return out.view(B, n_q, H * D) if rows is None else out.view(rows.rows, H * D)


def rope_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                   position_ids: torch.Tensor, past_key_value, prepared: PreparedMask,
                   rows: Optional[PackedRows] = None, fused: Optional[bool] = None) -> torch.Tensor:
    """Rotation of q and k by their positions, append of k and v to the cache, attention of q over
    the cache under `prepared`: modeling_llama.py:148-176 for the new tokens of one layer.

    q (B, n, heads*D), k, v (B, n, kv_heads*D) as the projections produce them (with `rows`:
    (rows.rows, ...)); cos/sin (positions, D); position_ids (B, n) int64; past_key_value the layer's
    (key view, value view) of a kv_cache.Cache.  Returns (B, n, heads*D) (or (rows.rows, heads*D)).

    bf16 with head_dim 128 and at most 256 new tokens per row runs as ONE kernel (rd_rope_verify_attention: the attention kernel rotates
    its query rows in registers and writes the new cache rows itself before it reads them; q stays
    as it was); anything else, or fused=False, runs kv_cache.rope_append (which rotates q in place)
    and masked_attention.  Both give the same bits in the output and in the cache."""
    from . import kv_cache  # (kv_cache does not import this module)

    key_view, value_view = past_key_value
    cache = key_view._cache
    _, _, batch, n_kv_heads, max_length, head_dim = cache.shape
    n_heads = q.shape[-1] // head_dim
    lib = _hip.lib()
    owner = key_view._owner
    in_place = owner is not None and owner.rows_in_place
    can_fuse = bool(lib.rd_rope_verify_attention_eligible(_hip.dtype_code(q.dtype), n_heads, head_dim,
                                                          prepared.n_q)) and prepared.shifted == in_place
    if fused is None:
        fused = can_fuse
    assert can_fuse or not fused, "no fused kernel for this dtype / head_dim / cache layout"
    if not fused:
        q_heads, keys, values = kv_cache.rope_append(q, k, v, cos, sin, position_ids, past_key_value, rows)
        return masked_attention(q_heads, keys, values, prepared, rows=rows)

    if rows is None:
        n_new = q.shape[1]
        lead = (batch, n_new)
        new_strides = lambda t: (C.c_int64 * 2)(t.stride(0), t.stride(1))
        out = torch.empty((batch, n_new, n_heads, head_dim), dtype=q.dtype, device=q.device)
        q_strides = (C.c_int64 * 3)(q.stride(0), head_dim, q.stride(1))  # batch, head, token
        o_strides = (C.c_int64 * 3)(out.stride(0), out.stride(2), out.stride(1))
    else:
        assert rows.batch == batch
        n_new = rows.n
        lead = (rows.rows,)
        new_strides = lambda t: (C.c_int64 * 2)(0, t.stride(0))
        out = torch.empty((rows.rows, n_heads, head_dim), dtype=q.dtype, device=q.device)
        q_strides = (C.c_int64 * 3)(0, head_dim, q.stride(0))
        o_strides = (C.c_int64 * 3)(0, out.stride(1), out.stride(0))
    assert q.shape == (*lead, n_heads * head_dim) and q.stride(-1) == 1
    assert k.shape == (*lead, n_kv_heads * head_dim) and k.stride(-1) == 1
    assert v.shape == k.shape and v.stride(-1) == 1
    assert q.dtype == k.dtype == v.dtype == cache.dtype == cos.dtype == sin.dtype
    assert cos.shape == sin.shape and cos.shape[1] == head_dim and cos.is_contiguous() and sin.is_contiguous()
    assert position_ids.shape == (batch, n_new) and position_ids.dtype == torch.long and position_ids.stride(1) == 1
    assert key_view.length == value_view.length and key_view.length + n_new <= max_length
    assert value_view._cache is cache and key_view._layer == value_view._layer
    kv_len = key_view.length + n_new
    assert (prepared.batch, prepared.n_q, prepared.kv_len) == (batch, n_new, kv_len), "mask/plan mismatch"
    k_slab = cache[key_view._layer, 0]
    v_slab = cache[key_view._layer, 1]
    ws_bytes = lib.rd_attention_workspace_bytes(batch, n_heads, n_new, kv_len, head_dim)
    if prepared.workspace is None or prepared.workspace.numel() < ws_bytes:
        prepared.workspace = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=q.device)
    if shape_log is not None:
        shape_log.append((batch, n_new, kv_len, batch * n_new if rows is None else rows.total))
    _hip.check(
        lib.rd_rope_verify_attention(
            _hip.ptr(q), q_strides, _hip.ptr(k), new_strides(k), _hip.ptr(v), new_strides(v),
            _hip.ptr(cos), _hip.ptr(sin), cos.shape[0], _hip.ptr(position_ids), position_ids.stride(0),
            _hip.ptr(k_slab), _hip.ptr(v_slab),
            (C.c_int64 * 3)(k_slab.stride(0), k_slab.stride(1), k_slab.stride(2)), max_length,
            _hip.ptr(out), o_strides, _hip.dtype_code(q.dtype), batch, n_heads, n_kv_heads, n_new, kv_len,
            head_dim, 1.0 / math.sqrt(head_dim), _hip.ptr(prepared.bits), _hip.ptr(prepared.plan),
            _hip.ptr(prepared.workspace), prepared.workspace.numel(),
            _hip.ptr(rows.row_start) if rows is not None else None, _hip.stream(),
        )
    )
    key_view.length += n_new
    value_view.length += n_new
    return out.view(batch, n_new, n_heads * head_dim) if rows is None else out.view(rows.rows, n_heads * head_dim)
