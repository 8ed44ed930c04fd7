"""Pins oracle/accept_oracle.py: reference literals, injected-uniform brute force, KV examples."""
import numpy as np
import pytest

from oracle import accept_oracle as Acc
from oracle import tree_oracle as T

A = lambda x: np.asarray(x, dtype=np.int64)  # noqa: E731


def test_greedy_choose_literal(literals):
    g = literals["greedy_choose"]
    n, s = Acc.greedy_choose(A(g["beams_by_drafter"]), A(g["beams_by_llm"]))
    assert n.tolist() == g["n_tokens_in_seq"] and s.tolist() == g["seq_in_beam"]


@pytest.mark.parametrize("B,W,L", [(1, 1, 2), (4, 4, 4), (13, 13, 13)])
def test_greedy_choose_maximality(B, W, L):
    rng = np.random.default_rng(123)
    d = rng.integers(0, 2, size=(B, W, L))
    m = rng.integers(0, 2, size=(B, W, L))
    n, s = Acc.greedy_choose(d, m)
    cmp = (d[:, :, 1:] == m[:, :, :-1]).astype(np.int64)
    per_beam = np.cumprod(cmp, axis=-1).sum(-1)
    assert np.array_equal(n, per_beam.max(-1))
    assert np.array_equal(s, per_beam.argmax(-1))  # first maximal beam
    for b in range(B):
        assert np.array_equal(d[b, s[b], 1 : n[b] + 1], m[b, s[b], : n[b]])


def test_greedy_next_input_property():
    rng = np.random.default_rng(123)
    B, W, L, H = 3, 4, 5, 32
    llm = rng.integers(0, 128, size=(B, W, L))
    hid = rng.random((B, W, L, H))
    s = rng.integers(0, W, size=B)
    n = rng.integers(0, L - 1, size=B)
    ctx, tok = Acc.greedy_next_input(llm, hid, s, n)
    for b in range(B):
        assert tok[b] == llm[b, s[b], n[b]]
        assert np.array_equal(ctx[b], hid[b, s[b], n[b]])


@pytest.mark.parametrize("B,W,L", [(1, 1, 2), (4, 4, 4), (13, 13, 13)])
def test_sample_choose_injected_uniforms(B, W, L):
    rng = np.random.default_rng(123)
    V = 2
    beams = rng.integers(0, V, size=(B, W, L))
    lp = rng.uniform(-10, 0, size=(B, W, L, V))
    lq = rng.uniform(-10, 0, size=(B, W, L - 1, V))
    u = rng.random((B, W, L - 1))
    n, s = Acc.sample_choose(beams, lp, lq, u)
    tok = beams[:, :, 1:, None]
    p = np.take_along_axis(lp[:, :, :-1], tok, -1)[..., 0]
    q = np.take_along_axis(lq, tok, -1)[..., 0]
    acc = (u < np.exp(p - q)).astype(np.int64)
    run = (np.cumsum(acc, -1) == np.arange(1, L)).sum(-1)  # cumsum==arange+1 form of the reference
    assert np.array_equal(n, run.max(-1)) and np.array_equal(s, run.argmax(-1))


def test_sample_choose_always_accept_when_p_ge_q():
    rng = np.random.default_rng(5)
    B, W, L, V = 3, 4, 5, 6
    beams = rng.integers(0, V, size=(B, W, L))
    lq = rng.uniform(-5, -1, size=(B, W, L - 1, V))
    lp = np.concatenate([lq + 0.5, rng.uniform(-5, 0, size=(B, W, 1, V))], axis=2)
    n, s = Acc.sample_choose(beams, lp, lq, rng.random((B, W, L - 1)))
    assert n.tolist() == [L - 1] * B and s.tolist() == [0] * B


def test_residual_probs_one_hot():
    rng = np.random.default_rng(123)
    B, W, L, V = 4, 3, 4, 10
    lq = rng.uniform(-50000.0, 0, size=(B, W, L - 1, V))
    lp = np.full((B, W, L, V), -50000.0)
    hot = rng.integers(0, V, size=(B, W, L))
    np.put_along_axis(lp, hot[..., None], 0.0, axis=-1)
    s = rng.integers(0, W, size=B)
    n = rng.integers(0, L, size=B)
    probs = Acc.residual_probs(lq, lp, s, n)
    for b in range(B):
        nz = np.nonzero(probs[b])[0]
        k = n[b]
        if k == L - 1 or lq[b, s[b], k, hot[b, s[b], k]] < 0:
            assert nz.tolist() == [hot[b, s[b], k]]


def test_kv_unpack_docstring_example(literals):
    k = literals["kv_unpack"]
    P, B, ML, NL, H, D = (k[x] for x in ("prompt_length", "batch_size", "max_length", "n_layers", "n_heads", "head_dim"))
    cache = np.zeros((NL, 2, B, H, ML, D), dtype=np.float32)
    vals = [k["packed_values_key"], k["packed_values_value"]]
    for kv in range(2):
        row = np.array([k["prompt_value"]] * P + vals[kv], dtype=np.float32)
        cache[:, kv, :, :, : len(row), :] = row[None, None, None, :, None]
    unp = np.broadcast_to(A(k["tree_attn_index"]), (B, 2, 3))
    Acc.kv_unpack(cache, P, unp)
    for kv in range(2):
        want = np.array([k["prompt_value"]] * P + [vals[kv][j] for j in k["expected_order"]], dtype=np.float32)
        assert np.array_equal(cache[:, kv, :, :, : len(want), :], np.broadcast_to(want[None, None, None, :, None], (NL, B, H, len(want), D)))


def test_update_ids_doc_example(literals):
    e = literals["update_ids_doc_example"]
    ids = A(e["input_ids"])
    beams = A(e["selected_beams"])[:, None, :]  # one beam per row
    B, W, L = beams.shape
    cache = np.arange(1 * 2 * B * 1 * 12 * 1, dtype=np.float32).reshape(1, 2, B, 1, 12, 1)
    before = cache.copy()
    new_ids, M = Acc.update_kv_and_ids(ids, A(e["n_tokens_in_seq"]), A([0, 0]), beams, cache, 0)
    assert M == e["max_seq_len"] and new_ids.tolist() == e["expected_ids"]
    # live region of row 0: old [0,2) + 3 accepted rows, right-aligned behind one pad
    assert np.array_equal(cache[:, :, 0, :, 1:6], before[:, :, 0, :, 0:5])
    assert np.array_equal(cache[:, :, 1, :, 0:6], before[:, :, 1, :, 1:7])


def test_update_kv_reference_vectors(ref_vectors):
    """B>1, ragged acceptance, shifts in both directions: the reference's own outputs."""
    for c in ref_vectors["kv_update"]:
        sh = c["shape"]
        shape = (sh["layers"], 2, sh["B"], sh["H"], sh["max_len"], sh["D"])
        cache = np.array(c["cache_before"], dtype=np.float32).reshape(shape)
        unp = A(c["unpacker"])
        Acc.kv_unpack(cache, sh["prev"], unp)
        assert np.array_equal(cache, np.array(c["cache_after_unpack"], dtype=np.float32).reshape(shape))
        ids, M = Acc.update_kv_and_ids(A(c["input_ids"]), A(c["n_tokens_in_seq"]), A(c["seq_in_beam"]),
                                       A(c["beams"]), cache, 0)
        assert ids.tolist() == c["new_ids"] and M == c["new_length"]
        assert np.array_equal(cache, np.array(c["cache_after_update"], dtype=np.float32).reshape(shape))
        # the packed-source form gives the same live region without the unpack step
        cache2 = np.array(c["cache_before"], dtype=np.float32).reshape(shape)
        ids2, M2 = Acc.update_kv_and_ids(A(c["input_ids"]), A(c["n_tokens_in_seq"]), A(c["seq_in_beam"]),
                                         A(c["beams"]), cache2, 0, unpacked=False, unpack=unp)
        assert ids2.tolist() == c["new_ids"]
        pads = T.count_left_paddings(ids2, 0)
        for b in range(sh["B"]):
            assert np.array_equal(cache2[:, :, b, :, pads[b] : M], cache[:, :, b, :, pads[b] : M])
