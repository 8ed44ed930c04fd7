"""GPU parity: acceptance, row gathers, KV unpack and KV compaction vs the CPU oracle (bit-exact)."""
import numpy as np
import pytest
import torch

from oracle import accept_oracle as Acc
from oracle import tree_oracle as T

pytestmark = pytest.mark.gpu

A = lambda x: np.asarray(x, dtype=np.int64)  # noqa: E731


def _dev(x, dtype=torch.long):
    return torch.tensor(np.asarray(x), dtype=dtype, device="cuda")


def test_greedy_choose_literal(literals):
    from recurrent_drafting_amd import acceptance

    g = literals["greedy_choose"]
    n, s = acceptance._greedy_choose_from_candidates(_dev(g["beams_by_drafter"]), _dev(g["beams_by_llm"]))
    assert n.cpu().tolist() == g["n_tokens_in_seq"] and s.cpu().tolist() == g["seq_in_beam"]


@pytest.mark.parametrize("B,W,L,vocab", [(1, 1, 2, 2), (4, 4, 4, 2), (13, 13, 13, 2), (8, 45, 5, 3), (16, 64, 5, 2), (2, 700, 4, 2)])
def test_greedy_choose_random(B, W, L, vocab):
    from recurrent_drafting_amd import acceptance

    rng = np.random.default_rng(123 + W)
    d = rng.integers(0, vocab, size=(B, W, L))
    m = rng.integers(0, vocab, size=(B, W, L))
    n, s = acceptance._greedy_choose_from_candidates(_dev(d), _dev(m))
    on, os_ = Acc.greedy_choose(d, m)
    assert np.array_equal(n.cpu().numpy(), on) and np.array_equal(s.cpu().numpy(), os_)


def test_greedy_accept_on_packed_slots():
    """LLM tokens given per packed slot + unpacker == unpacked form; next token and slot too."""
    from recurrent_drafting_amd import acceptance, tree_attention

    beams = T.synthetic_beams(8, 45, 5, vocab=6, seed=5)
    tok, unp, _, _, _ = T.pack(beams, np.zeros((8, 0), dtype=np.int64))
    rng = np.random.default_rng(0)
    llm_packed = rng.integers(0, 6, size=tok.shape)
    llm_unpacked = np.take_along_axis(llm_packed, unp.reshape(8, -1), axis=1).reshape(beams.shape)
    on, os_ = Acc.greedy_choose(beams, llm_unpacked)
    n, s, nxt, slot = acceptance.greedy_accept(_dev(beams), _dev(llm_packed), _dev(unp))
    assert np.array_equal(n.cpu().numpy(), on) and np.array_equal(s.cpu().numpy(), os_)
    r = np.arange(8)
    assert np.array_equal(nxt.cpu().numpy(), llm_unpacked[r, os_, on])
    assert np.array_equal(slot.cpu().numpy(), unp[r, os_, on])
    n2, s2, nxt2, slot2 = acceptance.greedy_accept(_dev(beams), _dev(llm_unpacked))
    assert torch.equal(n2, n) and torch.equal(s2, s) and torch.equal(nxt2, nxt)
    assert np.array_equal(slot2.cpu().numpy(), os_ * 5 + on)


def test_greedy_prepare_next_input_property():
    from recurrent_drafting_amd import acceptance

    torch.manual_seed(123)
    B, W, L, H = 3, 4, 5, 32
    llm = torch.randint(high=128, size=(B, W, L), device="cuda")
    hid = torch.rand(B, W, L, H, device="cuda")
    s = torch.randint(high=W, size=(B,), device="cuda")
    n = torch.randint(high=L - 1, size=(B,), device="cuda")
    state, tok = acceptance._greedy_prepare_next_input(llm, hid, s, n)
    for b in range(B):
        assert tok[b] == llm[b][s[b]][n[b]]
        assert torch.equal(state[b], hid[b][s[b]][n[b]])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,V", [(7, 1000), (33, 32000), (5, 32003), (3, 17)])
def test_argmax_rows(dtype, rows, V):
    from recurrent_drafting_amd import acceptance

    torch.manual_seed(rows * V)
    x = torch.randn(rows, V, device="cuda").to(dtype)
    x[0, V // 2] = x[0].max()  # an exact tie: the first index must win
    x[1, :] = 0.5
    got = acceptance.argmax_rows(x)
    want = np.argmax(x.float().cpu().numpy(), axis=-1)
    assert np.array_equal(got.cpu().numpy(), want)
    # non-contiguous rows (a column slice) take the strided path
    y = torch.randn(rows, V + 5, device="cuda").to(dtype)[:, 1 : V + 1]
    assert np.array_equal(acceptance.argmax_rows(y).cpu().numpy(), np.argmax(y.float().cpu().numpy(), axis=-1))


def test_argmax_rows_nan_and_inf():
    from recurrent_drafting_amd import acceptance

    x = torch.zeros(3, 100, device="cuda")
    x[0, 40] = float("nan"); x[0, 70] = float("nan"); x[0, 10] = float("inf")
    x[1, :] = float("-inf")
    x[2, 99] = 1.0
    assert acceptance.argmax_rows(x).cpu().tolist() == torch.argmax(x.cpu(), dim=-1).tolist() == [40, 0, 99]


@pytest.mark.parametrize("dtype,F", [(torch.float32, 8), (torch.bfloat16, 4096), (torch.float32, 32000), (torch.bfloat16, 7), (torch.float16, 10)])
def test_unpack_rows(dtype, F):
    from recurrent_drafting_amd import tree_attention

    beams = T.synthetic_beams(4, 9, 5, vocab=5, seed=F)
    tok, unp, _, _, _ = T.pack(beams, np.zeros((4, 0), dtype=np.int64))
    torch.manual_seed(0)
    packed = torch.rand(4, tok.shape[1], F, device="cuda").to(dtype)
    got = tree_attention.unpack(packed, _dev(unp))
    want = T.unpack_rows(packed.float().cpu().numpy(), unp)
    assert got.shape == (4, 9, 5, F) and np.array_equal(got.float().cpu().numpy(), want)


def test_unpack_reference_shapes(literals):
    from recurrent_drafting_amd import tree_attention

    for case in literals["unpack_shapes"]["cases"]:
        unp = _dev(case["unpacker"])
        packed = torch.rand((unp.shape[0], case["packed_len"], 8), device="cuda")
        out = tree_attention.unpack(packed, unp)
        assert out.shape[:3] == unp.shape
        for b, beam in enumerate(unp.cpu().tolist()):
            for i, cand in enumerate(beam):
                for k, slot in enumerate(cand):
                    assert torch.equal(out[b][i][k], packed[b][slot])


def test_count_left_paddings():
    from recurrent_drafting_amd import acceptance

    rng = np.random.default_rng(123)
    for shape in [(1, 4), (3, 17), (8, 2548), (5, 700)]:
        x = rng.integers(0, 2, size=shape)
        x[0, :] = 0
        if shape[0] > 2:
            x[2, : shape[1] - 1] = 0; x[2, -1] = 1
        got = acceptance._count_left_paddings(_dev(x), 0)
        assert np.array_equal(got.cpu().numpy(), T.count_left_paddings(x, 0))


def test_tree_position_ids_equal_the_op_chain():
    """position_ids = (prev - left pads) + position offsets (recurrent_drafting.py:449-458), with
    all-pad rows, rows without pads, an empty prefix, a strided offsets view and a pad id that is not 0."""
    from recurrent_drafting_amd import acceptance

    rng = np.random.default_rng(5)
    for (B, prev, n), pad in [((1, 4, 1), 0), ((3, 17, 9), 0), ((8, 2548, 181), 0), ((5, 700, 33), 7), ((2, 0, 5), 0)]:
        x = rng.integers(0, 9, size=(B, prev))
        for b in range(B):
            x[b, : rng.integers(0, prev + 1)] = pad
        if B > 2 and prev:
            x[0, :] = pad
            x[1, 0] = pad + 1
        off = rng.integers(0, 5, size=(B, n + 3))
        offsets = _dev(off)[:, :n]  # row stride n + 3
        got = acceptance.tree_position_ids(_dev(x), pad, offsets)
        want = (prev - T.count_left_paddings(x, pad))[:, None] + off[:, :n]
        assert got.dtype == torch.long and np.array_equal(got.cpu().numpy(), want)


def test_cache_object(literals):
    """The reference's test_cache, on the GPU object."""
    from recurrent_drafting_amd import kv_cache

    B, ML, NL, H, D = 7, 11, 3, 5, 2
    cache = kv_cache.Cache(B, ML, NL, H, D, torch.float32, torch.device("cuda"))
    assert cache._cache.shape == (NL, 2, B, H, ML, D) and len(cache.sliced) == NL
    assert all(cache.sliced[i][j].shape == (B, H, 0, D) for i in range(NL) for j in range(2))
    new_kv = torch.ones([B, H, 2, D], device="cuda")
    assert torch.all(cache.sliced[0][0].cat(new_kv) == new_kv) and cache.sliced[0][0].length == 2
    assert torch.all(cache.sliced[0][0].cat(new_kv) == torch.cat([new_kv, new_kv], dim=2))
    assert cache.sliced[0][0].length == 4 and torch.all(cache.sliced[0][0].slice(2) == new_kv)
    with pytest.raises(AssertionError):
        cache.sliced[0][0].cat(torch.ones([B, H, 8, D], device="cuda"))


def test_kv_unpack_docstring_example(literals):
    from recurrent_drafting_amd import kv_cache

    k = literals["kv_unpack"]
    P, B, ML, NL, H, D = (k[x] for x in ("prompt_length", "batch_size", "max_length", "n_layers", "n_heads", "head_dim"))
    cache = kv_cache.Cache(B, ML, NL, H, D, torch.float32, torch.device("cuda"))
    vals = [k["packed_values_key"], k["packed_values_value"]]
    for layer in range(NL):
        for kv in range(2):
            row = torch.tensor([k["prompt_value"]] * P + vals[kv], device="cuda")
            cache.sliced[layer][kv].cat(row[None, None, :, None].expand(B, H, -1, D))
    cache.unpack(P, _dev(k["tree_attn_index"]).expand(B, -1, -1))
    for layer in range(NL):
        for kv in range(2):
            want = torch.tensor([k["prompt_value"]] * P + [vals[kv][j] for j in k["expected_order"]], device="cuda")
            assert cache.sliced[layer][kv].length == P + 6
            assert torch.all(cache.sliced[layer][kv].slice(0) == want[None, None, :, None].expand(B, H, -1, D))


def test_kv_update_reference_vectors(ref_vectors):
    """Cache.unpack then _update_kv_cache_and_input_ids on the reference's own ragged cases.

    The vectors use head_dim 2 (8-byte rows); the C ABI moves 16-byte lanes, so every value is
    repeated 4x along head_dim, which commutes with row movement."""
    from recurrent_drafting_amd import acceptance, kv_cache

    for c in ref_vectors["kv_update"]:
        sh = c["shape"]
        shape = (sh["layers"], 2, sh["B"], sh["H"], sh["max_len"], sh["D"])
        wide = lambda key: np.repeat(np.array(c[key], dtype=np.float32).reshape(shape), 4, axis=-1)  # noqa: E731
        cache = kv_cache.Cache(sh["B"], sh["max_len"], sh["layers"], sh["H"], sh["D"] * 4, torch.float32, torch.device("cuda"))
        cache._cache.copy_(torch.tensor(wide("cache_before")))
        n_sel = int(np.max(c["unpacker"])) + 1
        cache.set_length(sh["prev"] + n_sel)
        cache.unpack(sh["prev"], _dev(c["unpacker"]))
        assert np.array_equal(cache._cache.cpu().numpy(), wide("cache_after_unpack"))
        ids = acceptance._update_kv_cache_and_input_ids(
            _dev(c["input_ids"]), _dev(c["n_tokens_in_seq"]), _dev(c["seq_in_beam"]), _dev(c["beams"]), cache, 0)
        assert ids.cpu().tolist() == c["new_ids"] and cache.sliced[0][0].length == c["new_length"]
        want = wide("cache_after_update")
        got = cache._cache.cpu().numpy()
        new_pads = T.count_left_paddings(A(c["new_ids"]), 0)
        for b in range(sh["B"]):
            lo, hi = int(new_pads[b]), c["new_length"]
            assert np.array_equal(got[:, :, b, :, lo:hi], want[:, :, b, :, lo:hi])


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_kv_unpack_and_compact_random(seed, dtype):
    """Ragged acceptance, left pads, shifts in both directions; packed-source and unpacked-source
    forms; live region bit-exact against the oracle, ids exact."""
    from recurrent_drafting_amd import acceptance, kv_cache

    rng = np.random.default_rng(seed)
    B, W, L = [(3, 3, 4), (4, 2, 3), (2, 4, 5), (5, 3, 3), (8, 45, 5), (6, 7, 6)][seed]
    NL, H, D = 2, 3, 8
    prev = int(rng.integers(3, 300 if seed >= 4 else 9))
    pads = rng.integers(0, 3 if seed < 4 else prev // 2, size=B)
    pads[rng.integers(0, B)] = 0
    ids = rng.integers(1, 50, size=(B, prev))
    for b in range(B):
        ids[b, : pads[b]] = 0
    beams = T.synthetic_beams(B, W, L, vocab=6, seed=seed) + 1
    tok, unp, _, _, _ = T.pack(beams, (ids != 0).astype(np.int64))
    n_sel = tok.shape[1]
    max_len = prev + W * L + 3
    vals = rng.integers(-120, 120, size=(NL, 2, B, H, max_len, D)).astype(np.float32)
    n_tok = rng.integers(0, L, size=B)
    s_beam = rng.integers(0, W, size=B)

    # oracle: unpack, then update (unpacked layout)
    o_cache = vals.copy()
    Acc.kv_unpack(o_cache, prev, unp)
    o_unpacked = o_cache.copy()
    o_ids, M = Acc.update_kv_and_ids(ids, n_tok, s_beam, beams, o_cache, 0)
    new_pads = T.count_left_paddings(o_ids, 0)

    def fresh():
        c = kv_cache.Cache(B, max_len, NL, H, D, dtype, torch.device("cuda"))
        c._cache.copy_(torch.tensor(vals).to(dtype))
        c.set_length(prev + n_sel)
        return c

    def live_equal(c):
        got = c._cache.float().cpu().numpy()
        for b in range(B):
            assert np.array_equal(got[:, :, b, :, new_pads[b] : M], o_cache[:, :, b, :, new_pads[b] : M]), b
        assert c.sliced[0][0].length == M and c.sliced[-1][1].length == M

    # drop-in sequence: Cache.unpack + _update_kv_cache_and_input_ids
    c1 = fresh()
    c1.unpack(prev, _dev(unp))
    assert np.array_equal(c1._cache.float().cpu().numpy(), o_unpacked)
    assert c1.sliced[0][0].length == prev + W * L
    g_ids = acceptance._update_kv_cache_and_input_ids(_dev(ids), _dev(n_tok), _dev(s_beam), _dev(beams), c1, 0)
    assert np.array_equal(g_ids.cpu().numpy(), o_ids)
    live_equal(c1)

    # fused sequence: accepted rows straight from the packed slots
    c2 = fresh()
    g_ids2 = acceptance.realign(_dev(ids), _dev(n_tok), _dev(s_beam), _dev(beams), c2, 0, unpacker=_dev(unp))
    assert np.array_equal(g_ids2.cpu().numpy(), o_ids)
    live_equal(c2)


def test_update_ids_doc_example(literals):
    from recurrent_drafting_amd import acceptance, kv_cache

    e = literals["update_ids_doc_example"]
    beams = _dev(e["selected_beams"])[:, None, :]
    cache = kv_cache.Cache(2, 12, 1, 1, 8, torch.float32, torch.device("cuda"))
    cache._cache.copy_(torch.arange(cache._cache.numel(), device="cuda").view_as(cache._cache))
    before = cache._cache.clone()
    cache.set_length(2 + 5)
    ids = acceptance._update_kv_cache_and_input_ids(_dev(e["input_ids"]), _dev(e["n_tokens_in_seq"]), _dev([0, 0]), beams, cache, 0)
    assert ids.cpu().tolist() == e["expected_ids"] and cache.sliced[0][0].length == e["max_seq_len"]
    assert torch.equal(cache._cache[:, :, 0, :, 1:6], before[:, :, 0, :, 0:5])
    assert torch.equal(cache._cache[:, :, 1, :, 0:6], before[:, :, 1, :, 1:7])


def test_kv_unpack_and_realign_at_the_full_configuration_size():
    """Configuration 4's cache (32 layers x 2 x batch 8 x 32 heads x 128, bf16, 1500 cached tokens,
    beam 45 x 5: 7 GB) through Cache.unpack + the re-alignment, and through the fused re-alignment
    with the rows moved and with the rows kept in place.  Moving rows is the same permutation in
    every layer, head and column, so the oracle runs on a one-column cache whose values are row
    numbers, and tells where every live row of the result came from; the full-size result must
    hold exactly those rows of the full-size input."""
    from recurrent_drafting_amd import acceptance, kv_cache

    rng = np.random.default_rng(11)
    B, W, L, NL, H, D, prev = 8, 45, 5, 32, 32, 128, 1500
    pads = rng.integers(0, 400, size=B)
    pads[3] = 0
    ids = rng.integers(1, 32000, size=(B, prev))
    for b in range(B):
        ids[b, : pads[b]] = 0
    beams = T.synthetic_beams(B, W, L, vocab=32000, seed=11) + 1
    tok, unp, _, _, _ = T.pack(beams, (ids != 0).astype(np.int64))
    n_sel = tok.shape[1]
    max_len = prev + W * L + 3
    n_tok = np.array([4, 0, 1, 2, 3, 0, 1, 2])
    s_beam = rng.integers(0, W, size=B)

    rows = np.broadcast_to(np.arange(max_len, dtype=np.float32)[None, None, None, None, :, None], (1, 2, B, 1, max_len, 1)).copy()
    Acc.kv_unpack(rows, prev, unp)
    unpacked_from = rows[0, 0, :, 0, :, 0].astype(np.int64).copy()  # (B, max_len): source row of every row
    o_ids, M = Acc.update_kv_and_ids(ids, n_tok, s_beam, beams, rows, 0)
    final_from = rows[0, 0, :, 0, :, 0].astype(np.int64)
    new_pads = T.count_left_paddings(o_ids, 0)

    dev = torch.device("cuda")
    g = torch.Generator(device="cuda").manual_seed(3)
    before = torch.empty((NL, 2, B, H, max_len, D), dtype=torch.bfloat16, device=dev)
    before.view(torch.int16).random_(-30000, 30000, generator=g)  # arbitrary bit patterns, made finite below
    before.nan_to_num_(nan=1.0, posinf=2.0, neginf=-2.0)

    def fresh():
        c = kv_cache.Cache(B, max_len, NL, H, D, torch.bfloat16, dev)
        c._cache.copy_(before)
        c.set_length(prev + n_sel)
        return c

    def same_rows(c, source, lo_of, hi):
        for b in range(B):
            lo = int(lo_of[b])
            src = torch.tensor(source[b, lo:hi], device=dev)
            want = before[:, :, b, :, :, :].index_select(3, src)
            assert torch.equal(c._cache[:, :, b, :, lo:hi, :].view(torch.int16), want.view(torch.int16)), b

    zeros = np.zeros(B, dtype=np.int64)
    # drop-in sequence
    c = fresh()
    c.unpack(prev, _dev(unp))
    same_rows(c, unpacked_from, zeros, prev + W * L)
    g_ids = acceptance._update_kv_cache_and_input_ids(_dev(ids), _dev(n_tok), _dev(s_beam), _dev(beams), c, 0)
    assert np.array_equal(g_ids.cpu().numpy(), o_ids) and c.sliced[0][0].length == M
    same_rows(c, final_from, new_pads, M)
    del c
    # fused: accepted rows straight from their packed slots, rows moved
    c = fresh()
    g_ids = acceptance.realign(_dev(ids), _dev(n_tok), _dev(s_beam), _dev(beams), c, 0, unpacker=_dev(unp))
    assert np.array_equal(g_ids.cpu().numpy(), o_ids)
    same_rows(c, final_from, new_pads, M)
    del c
    # fused, rows kept in place; materialize() then gives the reference's layout
    c = fresh()
    c.rows_in_place = True
    g_ids = acceptance.realign(_dev(ids), _dev(n_tok), _dev(s_beam), _dev(beams), c, 0, unpacker=_dev(unp))
    assert np.array_equal(g_ids.cpu().numpy(), o_ids)
    assert c.shift.cpu().tolist() == [int(new_pads[b] - pads[b]) for b in range(B)]
    c.materialize()
    same_rows(c, final_from, new_pads, M)
