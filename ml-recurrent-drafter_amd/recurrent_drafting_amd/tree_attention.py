"""Tree attention on the GPU: draft beams -> prefix tree -> packed tokens, mask and unpacker.

Same call surface as the reference's recurrent_drafting/tree_attention.py (`pack`, `unpack` and the
underscore helpers its tests use); the work is done by the HIP kernels behind rd_tree_build,
rd_tree_mask and rd_unpack_rows.  One device-to-host read (the packed length) per `pack`, where the
reference has two (tree_attention.py:78 and :99).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import _hip
from .packed_rows import PackedRows, round_up_rows


@dataclass
class PackedTree:
    """Everything one `pack` produces; `pack()` returns the reference's 4-tuple view of it."""

    packed_beams: torch.Tensor  # (B, n) int64
    unpacker: torch.Tensor  # (B, W, L) int64
    packed_token_indices: torch.Tensor  # (B, n) int64, flat index beam*L+pos of each packed slot
    position_offsets: torch.Tensor  # (B, n) int64
    prefix_tree: torch.Tensor  # (B, W, L) int64
    counts: torch.Tensor  # (B+2,) int32 on device: per-row count, max, total
    n: int  # packed length (max over rows), host value
    total: int  # sum of the rows' counts, host value
    row_start: torch.Tensor  # (B+1,) int32: slots that exist in the rows before each row
    row_slots: torch.Tensor  # (total rounded up,) int64: slot b*n+t of every slot that exists, row after row, then zeros
    row_tokens: Optional[torch.Tensor] = None  # (total rounded up,) int64: the tokens of those slots, then zeros

    def rows(self) -> PackedRows:
        """The slots that exist (slot t of row b exists iff t < counts[b])."""
        return PackedRows(self.row_start, self.row_slots, self.total, self.unpacker.shape[0], self.n,
                          self.row_slots.shape[0], self.row_tokens)


def _check_beams(beams: torch.Tensor) -> Tuple[int, int, int]:
    assert beams.dim() == 3, f"beams must be (batch, beam_width, beam_length), got {tuple(beams.shape)}"
    assert beams.dtype == torch.long, f"beams.dtype {beams.dtype} is not long"
    return tuple(beams.shape)  # type: ignore[return-value]


@dataclass
class PendingTree:
    """The launches of `build_tree` are queued; the packed length and the total (two int32 at
    `sizes`, on the device) still have to reach the host before the outputs can be shaped."""

    slab: torch.Tensor  # (7, B*W*L) int64
    counts: torch.Tensor  # (2B+3 or more,) int32: counts (B), max, total, row_start (B+1)
    shape: Tuple[int, int, int]

    def __post_init__(self):
        # every view that does not depend on the sizes is cut now: `finish` runs between the step's
        # one read and the first launch of the verify forward, with the GPU waiting
        B, W, L = self.shape
        self._rows = self.slab.unbind(0)
        self._unpacker = self._rows[1].view(B, W, L)
        self._prefix_tree = self._rows[0].view(B, W, L)
        self._counts = self.counts[: B + 2]
        self._row_start = self.counts[B + 2 : 2 * B + 3]
        self._sizes = self.counts[B : B + 2]

    @property
    def sizes(self) -> torch.Tensor:
        return self._sizes

    def finish(self, n: int, total: int) -> PackedTree:
        B, W, L = self.shape
        rows = self._rows
        padded = round_up_rows(total, B * W * L)
        return PackedTree(
            packed_beams=rows[2].as_strided((B, n), (n, 1)),
            unpacker=self._unpacker,
            packed_token_indices=rows[3].as_strided((B, n), (n, 1)),
            position_offsets=rows[4].as_strided((B, n), (n, 1)),
            prefix_tree=self._prefix_tree,
            counts=self._counts,
            n=n,
            total=total,
            row_start=self._row_start,
            row_slots=rows[5][:padded],
            row_tokens=rows[6][:padded],
        )


def build_tree_enqueue(beams: torch.Tensor, counts: Optional[torch.Tensor] = None) -> PendingTree:
    """Dedup + unpacker + pack + position offsets in two launches (tree_attention.py:331-335);
    nothing is read back.  counts: an int32 device buffer of at least 2B+3 elements to write the
    counts into (a caller that reads the sizes together with other numbers owns a longer one)."""
    B, W, L = _check_beams(beams)
    beams = beams.contiguous()
    dev = beams.device
    n_tok = B * W * L
    slab = torch.empty((7, n_tok), dtype=torch.long, device=dev)
    if counts is None:
        counts = torch.empty(2 * B + 3, dtype=torch.int32, device=dev)  # counts (B+2), then row_start (B+1)
    assert counts.dtype == torch.int32 and counts.numel() >= 2 * B + 3 and counts.is_contiguous()
    lib = _hip.lib()
    ws_bytes = lib.rd_tree_workspace_bytes(B, W, L)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    _hip.check(
        lib.rd_tree_build(
            _hip.ptr(beams), B, W, L,
            _hip.ptr(slab[0]), _hip.ptr(slab[1]), _hip.ptr(slab[2]), _hip.ptr(slab[3]),
            _hip.ptr(slab[4]), _hip.ptr(counts), _hip.ptr(counts[B + 2 :]), _hip.ptr(slab[5]),
            _hip.ptr(slab[6]), _hip.ptr(ws), ws_bytes, _hip.stream(),
        )
    )
    return PendingTree(slab, counts, (B, W, L))


def build_tree(beams: torch.Tensor) -> PackedTree:
    """`build_tree_enqueue` and the one host read that the output shapes depend on."""
    pending = build_tree_enqueue(beams)
    n, total = pending.sizes.tolist()
    return pending.finish(n, total)


def build_mask(tree: PackedTree, padding_mask: torch.Tensor, pad_value: int = 0) -> torch.Tensor:
    """(B, n, prev+n) bool mask of the packed rows (tree_attention.py:336-337).  An element of
    padding_mask equal to pad_value is padding: a 0/1 mask with the default, or the token ids
    themselves with the pad token id."""
    B, W, L = tree.unpacker.shape
    assert padding_mask.dim() == 2 and padding_mask.shape[0] == B
    assert padding_mask.dtype in (torch.int32, torch.int64, torch.bool, torch.uint8)
    prev = padding_mask.shape[1]
    if prev > 0 and padding_mask.stride(1) != 1:
        padding_mask = padding_mask.contiguous()
    n = tree.n
    out = torch.empty((B, n, prev + n), dtype=torch.bool, device=tree.unpacker.device)
    _hip.check(
        _hip.lib().rd_tree_mask(
            _hip.ptr(tree.unpacker), _hip.ptr(tree.packed_token_indices), _hip.ptr(tree.counts),
            _hip.ptr(padding_mask) if prev > 0 else None, padding_mask.element_size(),
            padding_mask.stride(0) if prev > 0 else 0, int(pad_value), prev, B, W, L, _hip.ptr(out), _hip.stream(),
        )
    )
    return out


def prepare_attention(tree: PackedTree, padding_mask: torch.Tensor, pad_value: int = 0, n_heads: int = 32,
                      kv_shift: Optional[torch.Tensor] = None):
    """For a caller that goes straight to the HIP attention: the tree mask as bits plus the work
    plan (an `attention.PreparedMask`, what `attention.prepare(build_mask(...))` gives, bit for
    bit), the position ids (B, n) of the packed tokens (recurrent_drafting.py:449-458) and the
    leading pad count of every row (B,) int32 -- one launch, no (B, n, prev+n) byte mask.
    padding_mask / pad_value as for `build_mask`; n_heads sizes the work items; kv_shift as for
    `attention.prepare`."""
    from . import attention

    B, W, L = tree.unpacker.shape
    assert padding_mask.dim() == 2 and padding_mask.shape[0] == B
    assert padding_mask.dtype in (torch.int32, torch.int64, torch.bool, torch.uint8)
    prev = padding_mask.shape[1]
    if prev > 0 and padding_mask.stride(1) != 1:
        padding_mask = padding_mask.contiguous()
    assert kv_shift is None or (kv_shift.shape == (B,) and kv_shift.dtype == torch.int32 and kv_shift.is_contiguous())
    n, kv_len = tree.n, prev + tree.n
    lib = _hip.lib()
    dev = tree.unpacker.device
    bits = torch.empty(lib.rd_attn_bits_words(B, n, kv_len), dtype=torch.int64, device=dev)
    plan = torch.empty(lib.rd_attn_plan_ints(B, n, kv_len), dtype=torch.int32, device=dev)
    position_ids = torch.empty((B, n), dtype=torch.long, device=dev)
    left_pads = torch.empty(B, dtype=torch.int32, device=dev)
    _hip.check(
        lib.rd_tree_attn_prepare(
            _hip.ptr(tree.unpacker), _hip.ptr(tree.packed_token_indices), _hip.ptr(tree.counts),
            _hip.ptr(padding_mask) if prev > 0 else None, padding_mask.element_size(),
            padding_mask.stride(0) if prev > 0 else 0, int(pad_value), prev, B, W, L, n, int(n_heads),
            _hip.ptr(bits), _hip.ptr(plan), _hip.ptr(position_ids), _hip.ptr(left_pads), _hip.ptr(kv_shift),
            _hip.stream(),
        )
    )
    return attention.PreparedMask(bits.view(B, n, -1), plan, B, n, kv_len, shifted=kv_shift is not None), position_ids, left_pads


def pack(
    beams: torch.Tensor, padding_mask: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(packed_beams (B,n), unpacker (B,W,L), causal_mask (B,n,prev+n) bool, position_offsets (B,n)).

    Drop-in for tree_attention.pack (tree_attention.py:301-338)."""
    tree = build_tree(beams)
    mask = build_mask(tree, padding_mask)
    return tree.packed_beams, tree.unpacker, mask, tree.position_offsets


# The reference's tests call these helpers directly; they are thin views of the fused kernels.
def _dedup_prefix(beams: torch.Tensor) -> torch.Tensor:
    return build_tree(beams).prefix_tree


def _get_unpacker(beams: torch.Tensor, prefix_tree: Optional[torch.Tensor] = None) -> torch.Tensor:
    return build_tree(beams).unpacker


def _pack_beams(
    beams: torch.Tensor, prefix_tree: Optional[torch.Tensor] = None
) -> Tuple[torch.Tensor, torch.Tensor]:
    t = build_tree(beams)
    return t.packed_beams, t.packed_token_indices


def gather_rows(
    packed: torch.Tensor, index: torch.Tensor, out: Optional[torch.Tensor] = None,
    rows: Optional[PackedRows] = None,
) -> torch.Tensor:
    """out[b, t, :] = packed[b, index[b, t], :] for packed (B, n, F) and index (B, T) int64.

    `out`, if given, is a (B, T, F) view whose last dimension is contiguous (any row/batch stride),
    e.g. one time slice of a (B, T, steps, F) history.  With `rows`, packed is (rows.rows, F), the
    slots that exist batch row after batch row, and index[b, t] is a slot of batch row b."""
    assert index.dim() == 2 and index.dtype == torch.long
    if rows is not None:
        assert packed.dim() == 2 and packed.shape[0] == rows.rows and index.shape[0] == rows.batch
        packed = packed.unsqueeze(0)  # (1, rows, F): the batch stride is not used
        B, n_src, F = rows.batch, rows.n, packed.shape[2]
    else:
        assert packed.dim() == 3
        B, n_src, F = packed.shape
    T = index.shape[1]
    assert index.shape[0] == B
    if packed.stride(2) != 1 or packed.stride(1) != F:
        packed = packed.contiguous()
    index = index.contiguous()
    if out is None:
        out = torch.empty((B, T, F), dtype=packed.dtype, device=packed.device)
    assert out.shape == (B, T, F) and out.dtype == packed.dtype and out.stride(2) == 1
    es = packed.element_size()
    _hip.check(
        _hip.lib().rd_unpack_rows(
            _hip.ptr(packed), packed.stride(0) * es, F * es, _hip.ptr(index), T, B, T, n_src,
            _hip.ptr(out), out.stride(0) * es, out.stride(1) * es,
            _hip.ptr(rows.row_start) if rows is not None else None, _hip.stream(),
        )
    )
    return out


def unpack(packed_tensor: torch.Tensor, unpacker: torch.Tensor) -> torch.Tensor:
    """(B, n, F) packed rows -> (B, W, L, F) as if every beam had been verified on its own.

    Drop-in for tree_attention.unpack (tree_attention.py:341-387)."""
    assert len(packed_tensor.shape) == 3
    B, W, L = unpacker.shape
    out = gather_rows(packed_tensor, unpacker.reshape(B, W * L))
    return out.view(B, W, L, packed_tensor.shape[2])
