"""Packed token rows: the kernels and the model that take `row_start` against the same call on
the padded (batch, n) layout.  The arithmetic per row is the same code, so attention and the
rotary embedding must agree bit for bit on every slot that exists; slots that do not exist must
not be touched."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _rows(counts, n):
    from recurrent_drafting_amd.packed_rows import PackedRows

    c = torch.tensor(counts, dtype=torch.int32, device="cuda")
    return PackedRows.from_counts(c, int(sum(counts)), n)


@pytest.mark.parametrize("dtype,H,D,n,counts,kv_prev,generic", [
    (torch.bfloat16, 4, 128, 100, [100, 37, 64, 1], 300, False),     # two waves per row block
    (torch.bfloat16, 2, 128, 200, [130, 200, 33], 500, False),       # one wave per row block
    (torch.bfloat16, 2, 128, 150, [150, 20, 97], 260, False),        # two full row blocks, three split ones
    (torch.bfloat16, 2, 128, 180, [64, 180, 161], 333, False),       # four full row blocks, two split ones
    (torch.bfloat16, 1, 128, 300, [290, 10], 700, False),            # two query tiles; a tile with no rows
    (torch.bfloat16, 2, 128, 90, [90, 45], 2400, False),             # long rows: keys split over work items
    (torch.float32, 3, 64, 20, [20, 7, 1], 50, True),
    (torch.float16, 2, 32, 9, [3, 9], 11, True),
])
def test_attention_packed_equals_padded(dtype, H, D, n, counts, kv_prev, generic):
    from recurrent_drafting_amd import attention

    B = len(counts)
    rows = _rows(counts, n)
    g = torch.Generator(device="cuda").manual_seed(n + H)
    kv = kv_prev + n
    q = torch.randn(B, n, H, D, generator=g, device="cuda").to(dtype)
    k = torch.randn(B, H, kv, D, generator=g, device="cuda").to(dtype)
    v = torch.randn(B, H, kv, D, generator=g, device="cuda").to(dtype)
    mask = torch.rand(B, n, kv, generator=g, device="cuda") > 0.3
    mask[:, :, : kv_prev // 3] &= torch.rand(B, 1, kv_prev // 3, generator=g, device="cuda") > 0.5
    prep = attention.prepare(mask, n_heads=H)
    padded = attention.masked_attention(q.transpose(1, 2), k, v, prep, force_generic=generic)  # (B, n, H*D)
    q_packed = rows.take(q)  # (T, H, D)
    packed = attention.masked_attention(q_packed, k, v, prep, force_generic=generic, rows=rows)
    assert packed.shape == (rows.rows, H * D) and rows.rows % 32 == 0 and rows.rows >= rows.total
    assert torch.equal(packed[: rows.total], rows.take(padded)[: rows.total])
    # the packed call writes nothing outside its rows: run it into a poisoned neighbourhood
    again = attention.masked_attention(q_packed, k, v, prep, force_generic=generic, rows=rows)
    assert torch.equal(again[: rows.total], packed[: rows.total])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_rope_append_packed_equals_padded(dtype):
    from recurrent_drafting_amd import kv_cache
    from oracle import torch_path

    B, n, heads, kv_heads, dim, prev, max_len = 3, 11, 4, 2, 32, 5, 24
    counts = [11, 4, 1]
    rows = _rows(counts, n)
    g = torch.Generator().manual_seed(7)
    hidden = (heads + 2 * kv_heads) * dim
    qkv = torch.randn(B, n, hidden, generator=g).to(dtype).cuda()
    pos = torch.randint(0, prev + n, (B, n), generator=g).cuda()
    old = torch.randn(2, B, kv_heads, max_len, dim, generator=g).to(dtype).cuda()
    cos, sin = torch_path._rope_tables(dim, 10000.0, prev + n, "cpu", dtype)
    cos, sin = cos.cuda(), sin.cuda()
    nq, nk = heads * dim, kv_heads * dim

    def run(packed):
        cache = kv_cache.Cache(B, max_len, 1, kv_heads, dim, dtype, torch.device("cuda"))
        cache._cache[0] = old
        cache.sliced[0][0].length = cache.sliced[0][1].length = prev
        x = rows.take(qkv).clone() if packed else qkv.clone()
        q, k, v = x[..., :nq], x[..., nq : nq + nk], x[..., nq + nk :]
        got_q, keys, values = kv_cache.rope_append(q, k, v, cos, sin, pos, cache.sliced[0],
                                                   rows if packed else None)
        assert cache.sliced[0][0].length == prev + n and keys.shape[2] == prev + n
        return got_q, cache._cache[0].clone()

    q_pad, cache_pad = run(False)   # (B, heads, n, dim)
    q_pack, cache_pack = run(True)  # (T, heads, dim)
    assert q_pack.shape == (rows.rows, heads, dim)
    assert torch.equal(q_pack[: rows.total], rows.take(q_pad.transpose(1, 2))[: rows.total])
    # the stand-in rows behind the last row that exists are not rotated
    assert torch.equal(q_pack[rows.total :], rows.take(qkv)[rows.total :, :nq].view(-1, heads, dim))
    for b, c in enumerate(counts):
        assert torch.equal(cache_pack[:, b, :, : prev + c], cache_pad[:, b, :, : prev + c])
        assert torch.equal(cache_pack[:, b, :, prev + c :], old[:, b, :, prev + c :])  # untouched


def test_model_on_packed_rows_matches_padded():
    """Decoder stack on the slots that exist against the same stack on all (batch, n) slots: the
    GEMMs see a different number of rows, so float32 here and a tolerance of a few ulps."""
    from recurrent_drafting_amd import kv_cache, modeling_llama
    from transformers.models.llama.configuration_llama import LlamaConfig

    torch.manual_seed(0)
    cfg = LlamaConfig(vocab_size=97, hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                      num_attention_heads=4, num_key_value_heads=4, max_position_embeddings=64)
    llm = modeling_llama.LlamaForCausalLM(cfg).cuda().float().eval()
    B, n, prev = 3, 9, 6
    counts = [9, 5, 2]
    rows = _rows(counts, n)
    ids = torch.randint(1, 97, (B, n), device="cuda")
    pos = (prev + torch.arange(n, device="cuda")).expand(B, n).contiguous()
    mask = torch.ones(B, n, prev + n, dtype=torch.bool, device="cuda").tril(prev)
    outs = []
    for packed in (False, True):
        cache = kv_cache.Cache(B, prev + n, 2, 4, 16, torch.float32, torch.device("cuda"))
        g = torch.Generator(device="cuda").manual_seed(1)
        cache._cache[:, :, :, :, :prev] = torch.randn(2, 2, B, 4, prev, 16, generator=g, device="cuda")
        for kv in cache.sliced:
            kv[0].length = kv[1].length = prev
        with torch.inference_mode():
            outs.append(llm.hidden_states(ids, mask, pos, cache.sliced, rows if packed else None))
    padded, packed = outs
    assert packed.shape == (rows.rows, 64)
    # a slot that exists attends only to slots that exist (causal within the row), so the values
    # of the padding slots cannot reach it
    torch.testing.assert_close(packed[: rows.total], rows.take(padded)[: rows.total], rtol=2e-5, atol=2e-5)


def test_tree_build_lists_the_slots_that_exist():
    from oracle import tree_oracle as T
    from recurrent_drafting_amd import tree_attention
    from recurrent_drafting_amd.packed_rows import PackedRows

    for B, W, L, seed in ((1, 1, 1, 0), (3, 4, 3, 1), (8, 45, 5, 2), (16, 64, 5, 3)):
        beams = torch.tensor(T.synthetic_beams(B, W, L, vocab=50, seed=seed), device="cuda")
        tree = tree_attention.build_tree(beams)
        counts = tree.counts[:B]
        assert tree.total == int(counts.sum()) and tree.n == int(counts.max())
        want = PackedRows.from_counts(counts, tree.total, tree.n, capacity=B * W * L)
        got = tree.rows()
        assert torch.equal(got.row_start, want.row_start) and got.row_start.dtype == torch.int32
        assert torch.equal(got.index, want.index) and got.index.dtype == torch.long
        assert (got.total, got.batch, got.n, got.rows) == (want.total, B, tree.n, want.rows)
        # the tokens of those rows, as the embedding lookup takes them: the existing slots' tokens, then zeros
        taken = want.take(tree.packed_beams)
        assert got.tokens is not None and got.tokens.shape == taken.shape
        assert torch.equal(got.tokens[: got.total], taken[: got.total]) and not got.tokens[got.total :].any()
        assert got.take_tokens(tree.packed_beams) is got.tokens


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_argmax_of_packed_rows_lands_at_the_slots(dtype):
    """rd_argmax_rows with an output index: the argmax of every packed row at its (batch, slot) place,
    equal to the plain argmax scattered by torch; the stand-in rows behind the last packed row are
    not run."""
    from recurrent_drafting_amd import acceptance

    counts, n, V = [9, 1, 14, 6], 14, 777
    rows = _rows(counts, n)
    g = torch.Generator(device="cuda").manual_seed(3)
    logits = torch.randn(rows.rows, V, generator=g, device="cuda").to(dtype)
    plain = acceptance.argmax_rows(logits)
    assert torch.equal(plain, logits.float().argmax(dim=-1))
    placed = acceptance.argmax_rows(logits, rows)
    assert placed.shape == (len(counts), n)
    want = rows.scatter(plain, fill=-1)
    exists = want >= 0
    assert int(exists.sum()) == rows.total
    assert torch.equal(placed[exists], want[exists])


def test_gather_of_packed_rows_by_slot():
    """rd_unpack_rows with row_start: row (b, slot) of a (rows, F) tensor of packed rows; a slot a batch
    row does not have leaves its output row as it was."""
    from recurrent_drafting_amd import tree_attention

    counts, n, F = [9, 1, 14, 6], 14, 96
    rows = _rows(counts, n)
    g = torch.Generator(device="cuda").manual_seed(4)
    packed = torch.randn(rows.rows, F, generator=g, device="cuda").to(torch.bfloat16)
    slots = torch.tensor([[8, 0], [0, 0], [13, 5], [2, 5]], device="cuda")
    got = tree_attention.gather_rows(packed, slots, rows=rows)
    want = packed.index_select(0, (rows.row_start[:-1].long()[:, None] + slots).flatten()).view(4, 2, F)
    assert torch.equal(got, want)
    out = torch.full((4, 1, F), 7.0, dtype=torch.bfloat16, device="cuda")
    tree_attention.gather_rows(packed, torch.tensor([[9], [1], [14], [5]], device="cuda"), out=out, rows=rows)
    assert bool((out[:3] == 7.0).all())  # slots 9, 1 and 14 do not exist in rows 0, 1 and 2
    assert torch.equal(out[3, 0], packed[int(rows.row_start[3]) + 5])


def test_realign_reports_the_new_length_and_the_accepted_tokens():
    """rd_realign_plan's step_out: the new length M and the accepted tokens summed over the rows."""
    from recurrent_drafting_amd import acceptance, kv_cache, tree_attention

    torch.manual_seed(5)
    B, W, L, prev = 4, 5, 4, 9
    ids = torch.randint(1, 50, (B, prev), device="cuda")
    ids[1, :3] = 0
    ids[3, :1] = 0
    beams = torch.randint(1, 50, (B, W, L), device="cuda")
    beams[:, :, 0] = beams[:, :1, 0]
    tree = tree_attention.build_tree(beams)
    cache = kv_cache.Cache(B, prev + W * L + 4, 1, 2, 8, torch.float32, torch.device("cuda"))
    cache.set_length(prev + tree.n)
    n_tokens = torch.tensor([3, 0, 2, 1], device="cuda")
    seq = torch.tensor([1, 0, 4, 2], device="cuda")
    out = torch.full((2,), -1, dtype=torch.int32, device="cuda")
    pending = acceptance.realign_enqueue(ids, n_tokens, seq, beams, cache, 0, unpacker=tree.unpacker, step_out=out)
    new_len = int(pending.new_len.item())
    assert out.tolist() == [new_len, 6]
    assert new_len == max(prev - p + n + 1 for p, n in zip([0, 3, 0, 1], [3, 0, 2, 1]))
