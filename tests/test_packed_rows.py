"""PackedRows bookkeeping (host logic; runs on the CPU)."""
import torch

from recurrent_drafting_amd.packed_rows import PackedRows


def test_index_take_scatter_roundtrip():
    counts = torch.tensor([3, 1, 4, 2], dtype=torch.int32)
    n = 4
    rows = PackedRows.from_counts(counts, int(counts.sum()), n)
    assert rows.row_start.tolist() == [0, 3, 4, 8, 10] and rows.row_start.dtype == torch.int32
    assert rows.rows == 32 and rows.total == 10
    assert rows.index.tolist() == [0, 1, 2, 4, 8, 9, 10, 11, 12, 13] + [0] * 22
    padded = torch.arange(4 * 4 * 2).view(4, 4, 2)
    taken = rows.take(padded)
    assert taken.shape == (32, 2) and torch.equal(taken[3], padded[1, 0]) and torch.equal(taken[9], padded[3, 1])
    back = rows.scatter(taken, fill=-1)
    for b, c in enumerate(counts.tolist()):
        assert torch.equal(back[b, :c], padded[b, :c]) and (back[b, c:] == -1).all()
    assert rows.row_of(torch.tensor([2, 0, 3, 1])).tolist() == [2, 3, 7, 9]
    spread = rows.spread(taken)
    for b, c in enumerate(counts.tolist()):
        assert torch.equal(spread[b, :c], padded[b, :c]) and (spread[b, c:] == padded[0, 0]).all()


def test_full_rows_are_the_identity():
    counts = torch.full((3,), 5, dtype=torch.int32)
    rows = PackedRows.from_counts(counts, 15, 5)
    assert rows.index.tolist() == list(range(15)) + [0] * 17
    x = torch.randn(3, 5, 7)
    assert torch.equal(rows.scatter(rows.take(x)), x)
