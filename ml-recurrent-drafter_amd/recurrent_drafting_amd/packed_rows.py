"""Token rows of a packed tree without the padding slots.

`tree_attention.pack` returns (batch, n) slots, n = the largest tree of the batch; a row's slots
past its own tree are filled with other rows' tokens (tree_attention.py:70-122) and nothing reads
what the model computes for them.  The fused decode step therefore runs the model's dense layers
on the T = sum of the tree sizes rows that exist: `PackedRows` carries the bookkeeping, and the
kernels that need the (batch row, slot) structure (rotary embedding + cache append, attention)
take `row_start`.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass
class PackedRows:
    row_start: torch.Tensor  # (batch + 1,) int32 on the device: first packed row of each batch row
    index: torch.Tensor  # (total,) int64 on the device: slot b * n + t of every packed row
    total: int  # packed rows, host value
    batch: int
    n: int  # slots per batch row in the padded layout

    @staticmethod
    def from_counts(counts: torch.Tensor, total: int, n: int) -> "PackedRows":
        """counts: (batch,) integer tensor on the device, the tree size of every batch row."""
        batch = counts.shape[0]
        row_start = torch.zeros(batch + 1, dtype=torch.int32, device=counts.device)
        torch.cumsum(counts, 0, dtype=torch.int32, out=row_start[1:])
        first = row_start[:-1].long()
        # packed row r of batch row b is slot b * n + (r - row_start[b])
        shift = torch.arange(batch, device=counts.device) * n - first
        index = torch.repeat_interleave(shift, counts.long(), output_size=total)
        index += torch.arange(total, device=counts.device)
        return PackedRows(row_start, index, total, batch, n)

    def take(self, padded: torch.Tensor) -> torch.Tensor:
        """(batch, n, ...) -> (total, ...): the slots that exist."""
        assert padded.shape[:2] == (self.batch, self.n)
        return padded.flatten(0, 1).index_select(0, self.index)

    def scatter(self, rows: torch.Tensor, fill=0) -> torch.Tensor:
        """(total, ...) -> (batch, n, ...), `fill` in the slots that do not exist."""
        assert rows.shape[0] == self.total
        out = rows.new_full((self.batch * self.n, *rows.shape[1:]), fill)
        out.index_copy_(0, self.index, rows)
        return out.view(self.batch, self.n, *rows.shape[1:])

    def row_of(self, slot: torch.Tensor) -> torch.Tensor:
        """(batch,) slot numbers -> their packed rows."""
        return self.row_start[:-1].long() + slot
