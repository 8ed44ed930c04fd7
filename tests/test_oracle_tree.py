"""Pins oracle/tree_oracle.py: reference literals, brute force, exhaustive tiny beams, invariants."""
import itertools

import numpy as np
import pytest

from oracle import tree_oracle as T

A = lambda x: np.asarray(x, dtype=np.int64)  # noqa: E731


def test_dedup_literals(literals):
    t = literals["tree"]
    assert np.array_equal(T.dedup_prefix(A(t["beams"])), A(t["prefix_tree"]))
    assert np.array_equal(T.dedup_prefix_loops(A(t["beams"])), A(t["prefix_tree"]))
    d = literals["doc_beam_to_prefix_tree"]
    assert np.array_equal(T.dedup_prefix(A(d["beams"])), A(d["prefix_tree"]))


def test_unpacker_literals(literals):
    t = literals["tree"]
    for fn in (T.unpacker, T.unpacker_loops, T.unpacker_closed_form):
        assert np.array_equal(fn(A(t["prefix_tree"])), A(t["unpacker"]))
    d = literals["doc_beam_to_prefix_tree"]
    assert np.array_equal(T.unpacker(A(d["prefix_tree"])), A(d["unpacker"]))


def test_pack_beams_literals(literals):
    t = literals["tree"]
    for fn in (T.pack_beams, T.pack_beams_loops):
        tok, idx, n = fn(A(t["beams"]), A(t["prefix_tree"]))
        assert np.array_equal(tok, A(t["packed_beams"]))
        assert np.array_equal(idx, A(t["packed_token_indices"]))
        assert n.tolist() == [7, 9]
    d = literals["doc_beam_to_prefix_tree"]
    _, idx, _ = T.pack_beams(A(d["beams"]), A(d["prefix_tree"]))
    assert np.array_equal(idx, A(d["packed_token_indices"]))


def test_pack_literal_masks(literals):
    t = literals["tree"]
    for case in literals["pack_masks"]["cases"]:
        tok, unp, mask, off, _ = T.pack(A(t["beams"]), A(case["padding_mask"]))
        assert np.array_equal(tok, A(t["packed_beams"]))
        assert np.array_equal(unp, A(t["unpacker"]))
        assert np.array_equal(mask, A(case["mask"]).astype(bool))
        assert np.array_equal(off, A(t["position_offsets"]))


def test_full_mask_literals(literals):
    t = literals["tree"]
    for case in literals["full_masks"]["cases"]:
        m = T.full_mask(A(case["padding_mask"]), A(t["unpacker"]), A(t["packed_token_indices"]))
        assert np.array_equal(m, A(case["mask"]).astype(bool))


def test_no_common_prefix_literals(literals):
    c = literals["no_common_prefix"]
    for case in c["cases"]:
        pm = np.ones((1, case["prompt_len"]), dtype=np.int64)
        tok, unp, mask, off, _ = T.pack(A(c["beams"]), pm)
        assert np.array_equal(mask, A(case["mask"]).astype(bool))
        assert tok.shape[1] == 12 and np.array_equal(off[0], np.tile(np.arange(4), 3))


def test_attention_mask_literals(literals):
    for case in literals["causal_mask"]["cases"]:
        m = T.causal_mask(A(case["padding_mask"]), case["query_len"])
        assert np.array_equal(m, A(case["mask"]).astype(bool))
    for case in literals["fully_masked_rows"]["cases"]:
        assert np.array_equal(T.fully_masked_rows_to_true(A(case["mask"])), A(case["expected"]).astype(bool))
    nf = np.finfo(np.float32).min
    for case in literals["bias"]["cases"]:
        b = T.bias(A(case["mask"]), np.float32)
        assert np.array_equal(b, np.where(A(case["mask"]) != 0, np.float32(0), nf))


def test_reference_vectors_pack(ref_vectors):
    """Spill-over padding with >= 3 rows and the last-row clamp, as the reference computes them."""
    for c in ref_vectors["pack"]:
        beams = A(c["beams"])
        tree = T.dedup_prefix(beams)
        assert np.array_equal(tree, A(c["prefix_tree"]))
        tok, idx, _ = T.pack_beams(beams, tree)
        assert np.array_equal(tok, A(c["packed_beams"]))
        assert np.array_equal(idx, A(c["packed_token_indices"]))
        pm = A(c["padding_mask"]).reshape(beams.shape[0], -1)
        tok, unp, mask, off, _ = T.pack(beams, pm)
        assert np.array_equal(unp, A(c["unpacker"]))
        assert np.array_equal(mask, A(c["mask"]).astype(bool).reshape(mask.shape))
        assert np.array_equal(off, A(c["position_offsets"]))


def test_exhaustive_small_beams():
    """Every beam set with W<=3, L<=3 over a 2-token vocabulary: array code == brute force."""
    for W, L in itertools.product((1, 2, 3), (1, 2, 3)):
        n = W * L
        all_beams = np.array(list(itertools.product((0, 1), repeat=n)), dtype=np.int64).reshape(-1, W, L)
        tree = T.dedup_prefix(all_beams)
        assert np.array_equal(tree, T.dedup_prefix_loops(all_beams))
        assert np.array_equal(T.unpacker(tree), T.unpacker_loops(tree))
        assert np.array_equal(T.unpacker(tree), T.unpacker_closed_form(tree))
        a = T.pack_beams(all_beams, tree)
        b = T.pack_beams_loops(all_beams, tree)
        for x, y in zip(a, b):
            assert np.array_equal(x, y)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_invariants_random(seed):
    rng = np.random.default_rng(seed)
    B, W, L = 4, 7, 5
    beams = rng.integers(0, 3, size=(B, W, L))
    tree = T.dedup_prefix(beams)
    assert np.array_equal(tree, T.dedup_prefix_loops(beams))
    assert (tree <= np.arange(W)[None, :, None]).all()
    unp = T.unpacker(tree)
    assert np.array_equal(unp, T.unpacker_closed_form(tree))
    tok, idx, n_sel = T.pack_beams(beams, tree)
    for b in range(B):
        # packed[unpacker] == beams, and the count equals the number of distinct prefixes
        assert np.array_equal(tok[b][unp[b]], beams[b])
        prefixes = {tuple(beams[b, i, : k + 1]) for i in range(W) for k in range(L)}
        assert n_sel[b] == len(prefixes)
    m = T.tree_mask_of_packed(unp, idx)
    for b in range(B):
        for n in range(int(n_sel[b])):
            i, k = divmod(int(idx[b, n]), L)
            assert set(np.nonzero(m[b, n])[0]) == {int(unp[b, i, k2]) for k2 in range(k + 1)}
            assert m[b, n, n]  # every real slot attends to itself


def test_synthetic_beams_generator():
    beams = T.synthetic_beams(8, 45, 5)
    assert beams.shape == (8, 45, 5) and beams.dtype == np.int64
    assert beams[:, :, 0].max() < 4 and beams.max() < 32000
    assert np.array_equal(beams, T.synthetic_beams(8, 45, 5))
    _, _, n = T.pack_beams(beams, T.dedup_prefix(beams))
    assert (n <= 225).all() and (n >= 5).all()


def test_count_left_paddings():
    x = A([[0, 0, 5, 0, 3], [4, 0, 0, 1, 1], [0, 0, 0, 0, 0]])
    assert T.count_left_paddings(x, 0).tolist() == [2, 0, 5]
