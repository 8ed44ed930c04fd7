"""GPU parity: rd_tree_build / rd_tree_mask / rd_tree_attn_prepare through the C ABI vs the CPU
oracle (bit-exact)."""
import numpy as np
import pytest
import torch

from oracle import tree_oracle as T

pytestmark = pytest.mark.gpu

A = lambda x: np.asarray(x, dtype=np.int64)  # noqa: E731


def _dev(x, dtype=torch.long):
    return torch.tensor(np.asarray(x), dtype=dtype, device="cuda")


def _check_against_oracle(beams, padding_mask):
    from recurrent_drafting_amd import tree_attention

    tok, unp, mask, off, idx = T.pack(beams, padding_mask)
    tree = tree_attention.build_tree(_dev(beams))
    assert np.array_equal(tree.prefix_tree.cpu().numpy(), T.dedup_prefix(beams))
    assert tree.n == tok.shape[1]
    assert np.array_equal(tree.packed_beams.cpu().numpy(), tok)
    assert np.array_equal(tree.packed_token_indices.cpu().numpy(), idx)
    assert np.array_equal(tree.unpacker.cpu().numpy(), unp)
    assert np.array_equal(tree.position_offsets.cpu().numpy(), off)
    for dt in (torch.long, torch.int32, torch.bool):
        g_tok, g_unp, g_mask, g_off = tree_attention.pack(_dev(beams), _dev(padding_mask, dt))
        assert g_mask.dtype == torch.bool and g_mask.shape == mask.shape
        assert np.array_equal(g_mask.cpu().numpy(), mask)
        assert np.array_equal(g_tok.cpu().numpy(), tok) and np.array_equal(g_off.cpu().numpy(), off)
        _check_prepare_attention(tree, _dev(padding_mask, dt), mask, off)


def bits_to_mask(bits, kv_len):
    """(B, n, words) int64 holding uint64 words -> (B, n, kv_len) bool; bits past kv_len must be zero."""
    words = bits.cpu().numpy().view(np.uint64)
    B, n, nw = words.shape
    flat = np.unpackbits(words.reshape(B, n, nw, 1).view(np.uint8), axis=-1, bitorder="little").reshape(B, n, nw * 64)
    assert not flat[:, :, kv_len:].any()
    return flat[:, :, :kv_len].astype(bool)


def _check_prepare_attention(tree, padding_mask, want_mask, want_offsets, pad_value=0, n_heads=3, shift=None):
    """rd_tree_attn_prepare against the oracle's mask and against the two-step path
    (rd_tree_mask -> rd_attn_prepare), bit for bit: mask bits, plan records, position ids, pad counts."""
    from recurrent_drafting_amd import acceptance, attention, tree_attention

    B, n, kv_len = want_mask.shape
    prev = kv_len - n
    prepared, pos, pads = tree_attention.prepare_attention(tree, padding_mask, pad_value, n_heads, shift)
    assert np.array_equal(bits_to_mask(prepared.bits, kv_len), want_mask)
    pm = padding_mask.cpu().numpy()
    want_pads = np.array([next((j for j in range(prev) if pm[b, j] != pad_value), prev) for b in range(B)])
    assert np.array_equal(pads.cpu().numpy(), want_pads)
    assert np.array_equal(pos.cpu().numpy(), (prev - want_pads)[:, None] + want_offsets)
    two_step = attention.prepare(tree_attention.build_mask(tree, padding_mask, pad_value), fix_empty_rows=True,
                                 n_heads=n_heads, kv_shift=shift)
    assert torch.equal(prepared.bits, two_step.bits)
    a, b = prepared.plan.cpu().numpy(), two_step.plan.cpu().numpy()
    n_items = int(b[0])
    used = 8 + 4 * B + 8 * n_items  # header, per-row records, work items (what the attention reads)
    assert np.array_equal(a[:used], b[:used])


def test_reference_literals(literals):
    t = literals["tree"]
    for case in literals["pack_masks"]["cases"]:
        _check_against_oracle(A(t["beams"]), A(case["padding_mask"]))
    c = literals["no_common_prefix"]
    for case in c["cases"]:
        _check_against_oracle(A(c["beams"]), np.ones((1, case["prompt_len"]), dtype=np.int64))


def test_reference_literal_values_directly(literals):
    """Reads like the reference's test_pack: outputs equal the literals, no oracle in between."""
    from recurrent_drafting_amd import tree_attention

    t = literals["tree"]
    for case in literals["pack_masks"]["cases"]:
        tok, unp, mask, off = tree_attention.pack(_dev(t["beams"]), _dev(case["padding_mask"]))
        assert tok.cpu().tolist() == t["packed_beams"]
        assert unp.cpu().tolist() == t["unpacker"]
        assert mask.cpu().to(torch.long).tolist() == case["mask"]
        assert off.cpu().tolist() == t["position_offsets"]
    p, i = tree_attention._pack_beams(_dev(t["beams"]))
    assert p.cpu().tolist() == t["packed_beams"] and i.cpu().tolist() == t["packed_token_indices"]
    assert tree_attention._dedup_prefix(_dev(t["beams"])).cpu().tolist() == t["prefix_tree"]


def test_reference_vectors(ref_vectors):
    for c in ref_vectors["pack"]:
        beams = A(c["beams"])
        _check_against_oracle(beams, A(c["padding_mask"]).reshape(beams.shape[0], -1))


@pytest.mark.parametrize("B,W,L,vocab,prev", [
    (1, 1, 2, 3, 0), (2, 3, 4, 2, 5), (4, 7, 5, 3, 17), (8, 45, 5, 4, 33), (3, 64, 5, 5, 100),
    (5, 13, 13, 2, 1), (16, 64, 5, 6, 64), (2, 128, 32, 2, 7),
])
def test_random_shapes(B, W, L, vocab, prev):
    rng = np.random.default_rng(B * 1000 + W * 10 + L)
    beams = rng.integers(0, vocab, size=(B, W, L))
    pm = (rng.random((B, prev)) > 0.2).astype(np.int64)
    _check_against_oracle(beams, pm)


def test_benchmark_config_full_size():
    """Config 2: (8,45,5) beams with shared prefixes, prev 0 and prev 2548."""
    beams = T.synthetic_beams(8, 45, 5, seed=123)
    _check_against_oracle(beams, np.zeros((8, 0), dtype=np.int64))
    rng = np.random.default_rng(1)
    pm = np.ones((8, 2548), dtype=np.int64)
    for b in range(8):
        pm[b, : rng.integers(0, 2048)] = 0
    pm[rng.random(pm.shape) < 0.001] = 0  # a few pad-valued tokens inside the live region
    _check_against_oracle(beams, pm)


def test_replicated_batch_invariants():
    """x64 replicated batch (512 rows): packed[unpacker] == beams, counts == distinct prefixes."""
    from recurrent_drafting_amd import tree_attention

    beams = np.concatenate([T.synthetic_beams(8, 45, 5, seed=s) for s in range(64)], axis=0)
    tree = tree_attention.build_tree(_dev(beams))
    packed = tree.packed_beams.cpu().numpy()
    unp = tree.unpacker.cpu().numpy()
    assert np.array_equal(np.take_along_axis(packed, unp.reshape(512, -1), axis=1).reshape(beams.shape), beams)
    counts = tree.counts.cpu().numpy()
    tok, _, n_sel = T.pack_beams(beams, T.dedup_prefix(beams))
    assert np.array_equal(counts[:512], n_sel) and counts[512] == n_sel.max() and counts[513] == n_sel.sum()
    assert np.array_equal(packed, tok)


def test_limits_raise():
    from recurrent_drafting_amd import tree_attention

    with pytest.raises(RuntimeError, match="width"):
        tree_attention.build_tree(torch.zeros((1, 2048, 2), dtype=torch.long, device="cuda"))
    with pytest.raises(AssertionError):
        tree_attention.build_tree(torch.zeros((1, 4, 2), dtype=torch.int32, device="cuda"))


def test_mask_from_token_ids_equals_mask_from_the_comparison():
    """rd_tree_mask takes the token ids with the pad id in place of a 0/1 padding mask."""
    from recurrent_drafting_amd import tree_attention

    rng = np.random.default_rng(11)
    for B, W, L, prev, pad in ((2, 3, 4, 9, 0), (8, 45, 5, 600, 0), (3, 5, 3, 40, 7)):
        beams = torch.tensor(T.synthetic_beams(B, W, L, vocab=50, seed=prev), device="cuda")
        ids = rng.integers(0, 12, size=(B, prev))
        for b in range(B):
            ids[b, : rng.integers(0, prev // 2)] = pad
        ids = torch.tensor(ids, device="cuda")
        tree = tree_attention.build_tree(beams)
        want = tree_attention.build_mask(tree, ids != pad)
        got = tree_attention.build_mask(tree, ids, pad_value=pad)
        assert torch.equal(got, want)


@pytest.mark.parametrize("seed", range(4))
def test_prepare_attention_from_token_ids_with_pads_by_value_and_row_shifts(seed):
    """The fused loop's call: the token ids stand in for the padding mask (pad id by value, also in
    the middle of a row), rows with nothing but padding, and a per-row cache shift in the plan."""
    from recurrent_drafting_amd import tree_attention

    rng = np.random.default_rng(seed)
    B, W, L = [(3, 5, 4), (8, 45, 5), (2, 64, 5), (5, 7, 6)][seed]
    prev = [9, 700, 64, 130][seed]
    beams = T.synthetic_beams(B, W, L, vocab=40, seed=seed) + 1
    ids = rng.integers(1, 50, size=(B, prev))
    pad = 7
    ids[ids == pad] = 8
    for b in range(B):
        ids[b, : rng.integers(0, prev // 2)] = pad
    ids[0, prev // 2 + 1] = pad  # a generated token that equals the pad id is masked as a key
    ids[B - 1, :] = pad          # nothing but padding: the tree rows still attend to themselves
    tok, unp, mask, off, idx = T.pack(beams, (ids != pad).astype(np.int64))
    tree = tree_attention.build_tree(_dev(beams))
    shift = torch.tensor(rng.integers(-3, 4, size=B), dtype=torch.int32, device="cuda")
    _check_prepare_attention(tree, _dev(ids), mask, off, pad_value=pad, n_heads=32, shift=shift)
    _check_prepare_attention(tree, _dev(ids), mask, off, pad_value=pad, n_heads=1)
