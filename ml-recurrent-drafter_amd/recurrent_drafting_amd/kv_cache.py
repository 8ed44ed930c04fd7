"""Pre-allocated KV cache with the reference's View/Cache objects (recurrent_drafting/kv_cache.py).

One dense tensor (n_layers, 2, batch, n_heads, max_length, head_dim) lives in HBM for the whole
generation; `View.cat` appends in place and hands back a strided view, `Cache.unpack` and
`Cache.compact` move rows with the HIP kernels rd_kv_unpack / rd_kv_compact (in place, no clone).

Rows in place: the reference re-right-aligns the whole live cache after every step
(recurrent_drafting.py:200-209).  With `Cache.rows_in_place = True` (the decode loop of
`RecurrentDrafting` sets it) the cache rows never move: a per-row `Cache.shift` says that token
column c of row b lives in cache row c - shift[b]; the re-alignment adds the change of the left
padding to it, and `rope_append` and the attention subtract it.  `Cache.materialize()` moves the rows
once to the reference's layout; `View.cat`, `View.slice` and `Cache.unpack` call it first.
"""

from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import _hip
from .packed_rows import PackedRows


class View:
    """Key or value rows of one layer: cache[layer, kv, :, :, 0:length, :] (kv_cache.py:10-35)."""

    def __init__(self, cache: torch.Tensor, layer: int, kv: int, owner: Optional["Cache"] = None):
        self._cache = cache
        self._layer = layer
        self._kv = kv  # 0 = key, 1 = value
        self._owner = owner
        self.length = 0

    @property
    def shape(self) -> Tuple[int, int, int, int]:
        _, _, batch_size, n_heads, _, head_dim = self._cache.shape
        return (batch_size, n_heads, self.length, head_dim)

    def cat(self, new_kv: torch.Tensor) -> torch.Tensor:
        """Appends (batch, n_heads, n_new, head_dim) rows in place and returns rows [0, length)."""
        _, _, batch_size, n_heads, max_length, head_dim = self._cache.shape
        n_new = new_kv.shape[2]
        assert new_kv.shape == (batch_size, n_heads, n_new, head_dim)
        assert self.length + n_new <= max_length
        if self._owner is not None:
            self._owner.materialize()
        slab = self._cache[self._layer, self._kv]
        slab[:, :, self.length : self.length + n_new, :] = new_kv
        self.length += n_new
        return slab[:, :, : self.length, :]

    def slice(self, prev: int) -> torch.Tensor:
        """Rows [prev, length)."""
        if self._owner is not None:
            self._owner.materialize()
        return self._cache[self._layer, self._kv, :, :, prev : self.length, :]


def rope_append(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                position_ids: torch.Tensor, past_key_value: Tuple[View, View],
                rows: Optional[PackedRows] = None):
    """Rotates q and k by their positions and appends the rotated k and v to the cache, one kernel.

    q (B, n, heads*D) and k, v (B, n, kv_heads*D) as the projections produce them (token rows may be
    strided, e.g. slices of one fused projection); cos/sin (positions, D) tables in q's dtype;
    position_ids (B, n) int64.  q is rotated in place.  Returns (q as (B, heads, n, D) view, keys,
    values) with keys/values the (B, kv_heads, length, D) views `View.cat` would return
    (modeling_llama.py:148-159, apply_rotary_pos_emb :87-110).

    With `rows`, q, k and v are (total, heads*D) / (total, kv_heads*D): only the slots that exist.
    The cache still grows by n rows per batch row (the slots that do not exist keep what the
    cache held), and q comes back as a (total, heads, D) view."""
    key_view, value_view = past_key_value
    cache = key_view._cache
    _, _, batch, n_kv_heads, max_length, head_dim = cache.shape
    if rows is None:
        n_new = q.shape[1]
        lead = (batch, n_new)
        strides = lambda t: (ctypes.c_int64 * 2)(t.stride(0), t.stride(1))
    else:
        assert rows.batch == batch
        n_new = rows.n
        lead = (rows.rows,)
        strides = lambda t: (ctypes.c_int64 * 2)(0, t.stride(0))
    n_heads = q.shape[-1] // head_dim
    assert q.shape == (*lead, n_heads * head_dim) and q.stride(-1) == 1
    assert k.shape == (*lead, n_kv_heads * head_dim) and k.stride(-1) == 1
    assert v.shape == k.shape and v.stride(-1) == 1
    assert q.dtype == k.dtype == v.dtype == cache.dtype == cos.dtype == sin.dtype
    assert cos.shape == sin.shape and cos.shape[1] == head_dim and cos.is_contiguous() and sin.is_contiguous()
    assert position_ids.shape == (batch, n_new) and position_ids.dtype == torch.long and position_ids.stride(1) == 1
    assert key_view.length == value_view.length and key_view.length + n_new <= max_length
    assert value_view._cache is cache and key_view._layer == value_view._layer
    k_slab = cache[key_view._layer, 0]
    v_slab = cache[key_view._layer, 1]
    owner = key_view._owner
    shift = owner.shift if owner is not None and owner.rows_in_place else None
    _hip.check(
        _hip.lib().rd_rope_append(
            _hip.ptr(q), strides(q), _hip.ptr(k), strides(k), _hip.ptr(v), strides(v),
            _hip.dtype_code(q.dtype), batch, n_new, n_heads,
            n_kv_heads, head_dim, _hip.ptr(cos), _hip.ptr(sin), cos.shape[0], _hip.ptr(position_ids),
            position_ids.stride(0), _hip.ptr(q), strides(q), _hip.ptr(k_slab), _hip.ptr(v_slab),
            (ctypes.c_int64 * 3)(k_slab.stride(0), k_slab.stride(1), k_slab.stride(2)), key_view.length,
            max_length, _hip.ptr(rows.row_start) if rows is not None else None, _hip.ptr(shift), _hip.stream(),
        )
    )
    key_view.length += n_new
    value_view.length += n_new
    if rows is None:
        q_heads = q.unflatten(2, (n_heads, head_dim)).transpose(1, 2)
    else:
        q_heads = q.unflatten(1, (n_heads, head_dim))
    return q_heads, k_slab[:, :, : key_view.length, :], v_slab[:, :, : value_view.length, :]


class Cache:
    def __init__(
        self,
        batch_size: int,
        max_length: int,
        n_layers: int,
        n_heads: int,
        head_dim: int,
        dtype: torch.dtype,
        device: torch.device,
    ) -> None:
        # (the attention reads only the cache rows of keys that somebody attends to, so nothing is
        # asked of the memory around a row's live rows; zeros as upstream, kv_cache.py:49-53)
        self._storage = torch.zeros([n_layers, 2, batch_size, n_heads, max_length, head_dim], dtype=dtype, device=device)
        self._cache = self._storage
        self.sliced = tuple(
            (View(self._cache, layer, 0, self), View(self._cache, layer, 1, self)) for layer in range(n_layers)
        )
        # token column c of batch row b lives in cache row c - shift[b] (all zero: the reference's layout)
        self.shift = torch.zeros(batch_size, dtype=torch.int32, device=device)
        self._rows_in_place = False
        self._shifted = False  # host-side: a re-alignment may have left non-zero shifts

    @property
    def rows_in_place(self) -> bool:
        """True: re-alignments leave the cache rows where they are and update `shift` instead."""
        return self._rows_in_place

    @rows_in_place.setter
    def rows_in_place(self, value: bool) -> None:
        if not value:
            self.materialize()  # nobody would follow the shifts any more
        self._rows_in_place = bool(value)

    # -- geometry handed to the C ABI ---------------------------------------------------------
    def _geometry(self):
        n_layers, _, batch, n_heads, max_len, head_dim = self._cache.shape
        return n_layers, batch, n_heads, max_len, head_dim * self._cache.element_size()

    def materialize(self) -> None:
        """Moves the rows to the layout in which column and cache row agree (no-op unless a
        re-alignment with rows in place has happened since the last call)."""
        if not self._shifted:
            return
        n_layers, batch, n_heads, max_len, row_bytes = self._geometry()
        lib = _hip.lib()
        plan = torch.empty(lib.rd_kv_materialize_plan_ints(batch), dtype=torch.int32, device=self._cache.device)
        _hip.check(
            lib.rd_kv_materialize(
                _hip.ptr(self._cache), n_layers, batch, n_heads, max_len, row_bytes,
                self.sliced[0][0].length, _hip.ptr(self.shift), _hip.ptr(plan), _hip.stream(),
            )
        )
        self._shifted = False

    def set_length(self, length: int) -> None:
        for key, value in self.sliced:
            key.length = value.length = length

    def unpack(self, prompt_length: int, tree_attn_index: torch.Tensor) -> None:
        """Every candidate position (beam, k) gets its own cache row behind the prompt:
        row prompt_length + beam*L + k takes the packed row prompt_length + tree_attn_index[b,beam,k]
        (kv_cache.py:58-98)."""
        batch, width, length = tree_attn_index.shape
        n_layers, cb, n_heads, max_len, row_bytes = self._geometry()
        assert cb == batch
        self.materialize()
        n_out = width * length
        n_src = self.sliced[0][0].length - prompt_length
        assert n_src > 0, "no packed rows behind the prompt"
        assert prompt_length + n_out <= max_len
        index = tree_attn_index.contiguous()
        assert index.dtype == torch.long
        _hip.check(
            _hip.lib().rd_kv_unpack(
                _hip.ptr(self._cache), n_layers, batch, n_heads, max_len, row_bytes, prompt_length,
                _hip.ptr(index), n_out, n_src, _hip.stream(),
            )
        )
        self.set_length(prompt_length + n_out)

    def compact(self, prev: int, beam_length: int, plan: torch.Tensor, new_length: int) -> None:
        """Follows a plan written by rd_realign_plan: accepted rows kept, rows re-right-aligned."""
        n_layers, batch, n_heads, max_len, row_bytes = self._geometry()
        assert plan.dtype == torch.int32
        _hip.check(
            _hip.lib().rd_kv_compact(
                _hip.ptr(self._cache), n_layers, batch, n_heads, max_len, row_bytes, prev,
                beam_length, _hip.ptr(plan), _hip.stream(),
            )
        )
        self.set_length(new_length)
