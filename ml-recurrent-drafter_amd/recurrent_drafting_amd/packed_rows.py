"""Token rows of a packed tree without the padding slots.

`tree_attention.pack` returns (batch, n) slots, n = the largest tree of the batch; a row's slots
past its own tree are filled with other rows' tokens (tree_attention.py:70-122) and nothing reads
what the model computes for them.  The fused decode step therefore runs the model's dense layers
on the T = sum of the tree sizes rows that exist: `PackedRows` carries the bookkeeping, and the
kernels that need the (batch row, slot) structure (rotary embedding + cache append, attention)
take `row_start`.

The row count handed to the dense layers is rounded up to a multiple of `PAD` (`rows`): the GEMM
library picks its kernel per problem size and pays for every size it has not seen (about 80 us of
host time per call, measured), and T changes with every step; rounded, a handful of sizes repeat.
The extra rows are copies of slot 0 on the way in and are dropped on the way out.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch


PAD = 32


def round_up_rows(total: int, capacity: Optional[int] = None) -> int:
    rows = (total + PAD - 1) // PAD * PAD
    return rows if capacity is None else min(rows, capacity)


@dataclass
class PackedRows:
    row_start: torch.Tensor  # (batch + 1,) int32 on the device: first packed row of each batch row
    index: torch.Tensor  # (rows,) int64 on the device: slot b * n + t of every packed row, then zeros
    total: int  # packed rows that exist, host value
    batch: int
    n: int  # slots per batch row in the padded layout
    rows: int  # rows handed to the dense layers: total rounded up (the extra rows are copies of slot 0)
    # (rows,) int64 or None: the token ids of the packed rows when whoever built the rows knows them
    # (rd_tree_build does), zeros in the extra rows; `take_tokens` then needs no gather
    tokens: Optional[torch.Tensor] = None

    @staticmethod
    def from_counts(counts: torch.Tensor, total: int, n: int,
                    capacity: Optional[int] = None) -> "PackedRows":
        """counts: (batch,) integer tensor on the device, the tree size of every batch row;
        capacity: an upper limit for the rounded row count."""
        batch = counts.shape[0]
        row_start = torch.zeros(batch + 1, dtype=torch.int32, device=counts.device)
        torch.cumsum(counts, 0, dtype=torch.int32, out=row_start[1:])
        first = row_start[:-1].long()
        # packed row r of batch row b is slot b * n + (r - row_start[b])
        shift = torch.arange(batch, device=counts.device) * n - first
        index = torch.repeat_interleave(shift, counts.long(), output_size=total)
        index += torch.arange(total, device=counts.device)
        rows = round_up_rows(total, capacity)
        index = torch.cat((index, index.new_zeros(rows - total)))
        return PackedRows(row_start, index, total, batch, n, rows)

    def take(self, padded: torch.Tensor) -> torch.Tensor:
        """(batch, n, ...) -> (rows, ...): the slots that exist, then the stand-in rows."""
        assert padded.shape[:2] == (self.batch, self.n)
        return padded.flatten(0, 1).index_select(0, self.index)

    def take_tokens(self, padded_ids: torch.Tensor) -> torch.Tensor:
        """`take` for the token ids of the model's input: uses the list the tree build left, if any
        (its extra rows hold token 0 instead of a copy of slot 0; those rows are dropped anyway)."""
        if self.tokens is not None:
            assert padded_ids.shape == (self.batch, self.n)
            return self.tokens
        return self.take(padded_ids)

    def scatter(self, rows: torch.Tensor, fill=0) -> torch.Tensor:
        """(rows, ...) -> (batch, n, ...), `fill` in the slots that do not exist."""
        assert rows.shape[0] == self.rows
        out = rows.new_full((self.batch * self.n, *rows.shape[1:]), fill)
        out.index_copy_(0, self.index[: self.total], rows[: self.total])
        return out.view(self.batch, self.n, *rows.shape[1:])

    def spread(self, rows: torch.Tensor) -> torch.Tensor:
        """(rows, ...) -> (batch, n, ...) with a copy of packed row 0 in the slots that do not
        exist: ordinary values for code that goes on to process every slot (a constant fill would
        hand it rows of equal numbers, the worst case of the top-k selection kernels)."""
        assert rows.shape[0] == self.rows
        where = torch.zeros(self.batch * self.n, dtype=torch.long, device=rows.device)
        where.index_copy_(0, self.index[: self.total],
                          torch.arange(self.total, dtype=torch.long, device=rows.device))
        return rows.index_select(0, where).view(self.batch, self.n, *rows.shape[1:])

    def row_of(self, slot: torch.Tensor) -> torch.Tensor:
        """(batch,) slot numbers -> their packed rows."""
        return self.row_start[:-1].long() + slot
