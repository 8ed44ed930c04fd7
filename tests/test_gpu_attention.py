"""GPU parity: mask compression, causal mask and the verification attention (MFMA + generic)
against the float64 oracle.  Tolerances: bf16 2e-2 of the output scale, fp32 1e-5."""
import numpy as np
import pytest
import torch

from oracle import fp_oracle as O
from oracle import tree_oracle as T

pytestmark = pytest.mark.gpu


def _dev(x, dtype):
    return torch.tensor(np.asarray(x), dtype=dtype, device="cuda")


def test_causal_mask_literals(literals):
    from recurrent_drafting_amd import attention

    for case in literals["causal_mask"]["cases"]:
        for dt in (torch.long, torch.int32, torch.bool):
            m = attention.causal_mask(_dev(case["padding_mask"], dt), case["query_len"], torch.device("cuda"))
            assert m.dtype == torch.bool and m.cpu().to(torch.long).tolist() == case["mask"]
    for case in literals["fully_masked_rows"]["cases"]:
        got = attention.set_sdpa_fully_masked_rows(_dev(case["mask"], torch.long))
        assert got.cpu().tolist() == case["expected"]
    nf = torch.finfo(torch.float32).min
    for case in literals["bias"]["cases"]:
        m = _dev(case["mask"], torch.long)
        b = attention.bias(m, torch.float32)
        assert torch.equal(b, torch.where(m != 0, 0.0, nf).to(torch.float32))


def test_causal_mask_random():
    from recurrent_drafting_amd import attention

    rng = np.random.default_rng(0)
    pm = (rng.random((5, 300)) > 0.3).astype(np.int64)
    for ql in (1, 7, 300):
        got = attention.causal_mask(_dev(pm, torch.long), ql, torch.device("cuda"))
        assert np.array_equal(got.cpu().numpy(), T.causal_mask(pm, ql))


def test_mask_bits_and_plan():
    from recurrent_drafting_amd import attention

    rng = np.random.default_rng(1)
    B, nq, kv = 3, 10, 1500
    mask = rng.random((B, nq, kv)) > 0.5
    mask[0, :, :700] = False  # row 0: first attended key >= 700 -> begin 640
    mask[1, 3, :] = False  # an empty row gets all keys
    mask[2, :, :64] = False
    mask[2, 5, 70] = True
    prep = attention.prepare(_dev(mask, torch.bool), n_heads=1)  # one head: minimum-size items
    words = prep.bits.cpu().numpy().view(np.uint64)
    fixed = T.fully_masked_rows_to_true(mask)
    for b in range(B):
        for q in range(nq):
            bits = np.unpackbits(words[b, q].view(np.uint8), bitorder="little")[:kv].astype(bool)
            assert np.array_equal(bits, fixed[b, q]), (b, q)
            assert not np.unpackbits(words[b, q].view(np.uint8), bitorder="little")[kv:].any()
    plan = prep.plan.cpu().numpy()
    n_items, max_splits = plan[0], plan[4]
    assert plan[1] == nq and plan[2] == kv and plan[3] == (kv + 63) // 64
    per_row = plan[8 : 8 + 4 * B].reshape(B, 4)
    attended = [np.flatnonzero(fixed[b].any(axis=0)) for b in range(B)]
    key_min, key_end = [int(a[0]) for a in attended], [int(a[-1]) + 1 for a in attended]
    firsts = [m // 64 * 64 for m in key_min]
    assert per_row[:, 0].tolist() == firsts
    items = plan[8 + 4 * B : 8 + 4 * B + 8 * n_items].reshape(n_items, 8)
    assert n_items == per_row[:, 1].sum() and per_row[:, 1].max() <= max_splits
    lens = items[:, 2] - items[:, 1]
    assert (np.diff(lens) <= 0).all()  # longest first
    for b in range(B):  # the items of a row tile [begin, last attended key] without gaps or overlap
        mine = sorted((lo, hi, s) for bb, lo, hi, s, *_ in items.tolist() if bb == b)
        assert mine[0][0] == firsts[b] and mine[-1][1] == key_end[b]
        assert all(a[1] == c[0] for a, c in zip(mine, mine[1:]))
        assert all(lo % 64 == 0 for lo, _, _ in mine)
        assert [s for _, _, s in mine] == list(range(len(mine)))
        for bb, lo, hi, s, shift, kmin, n_splits, kend in items.tolist():
            if bb == b:
                assert (shift, kmin, n_splits, kend) == (0, key_min[b], per_row[b, 1], key_end[b])


def test_mfma_kernel_reads_only_the_rows_of_attended_keys():
    """Left padding in front of a row's first key, tree slots that do not exist behind its last one
    and the tail of the cache hold NaN here (a cache made with torch.empty may hold anything): keys
    that nobody attends to must not reach the arithmetic, not even with a zero weight."""
    from recurrent_drafting_amd import attention

    rng = np.random.default_rng(5)
    prev_lens = [700, 333, 1, 640]
    mask = _tree_case(4, 8, 5, prev_lens, seed=2).copy()
    B, nq, kv = mask.shape
    prev = kv - nq
    counts = [nq - 5, nq, nq - 17, nq - 1]  # tree slots that exist per row; the rest attends to nothing
    for b, c in enumerate(counts):
        mask[b, c:, :] = False
        mask[b, :, prev + c:] = False
    H, D = 3, 128
    q = torch.tensor(rng.standard_normal((B, H, nq, D)), dtype=torch.bfloat16, device="cuda")
    k = torch.tensor(rng.standard_normal((B, H, kv + 90, D)), dtype=torch.bfloat16, device="cuda")
    v = torch.tensor(rng.standard_normal((B, H, kv + 90, D)), dtype=torch.bfloat16, device="cuda")
    clean_k, clean_v = k.clone(), v.clone()
    for b in range(B):
        for t in (k, v):
            t[b, :, : prev - prev_lens[b]] = float("nan")
            t[b, :, prev + counts[b]:] = float("nan")
    tq = q.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    for heads_for_plan in (H, 1):  # whole rows, and rows split over several work items
        prep = attention.prepare(_dev(mask, torch.bool), fix_empty_rows=False, n_heads=heads_for_plan)
        got = attention.masked_attention(tq, k[:, :, :kv], v[:, :, :kv], prep)
        prep2 = attention.prepare(_dev(mask, torch.bool), fix_empty_rows=False, n_heads=heads_for_plan)
        want = attention.masked_attention(tq, clean_k[:, :, :kv], clean_v[:, :, :kv], prep2)
        assert torch.isfinite(got).all()
        assert torch.equal(got, want)
        for b, c in enumerate(counts):  # queries that attend to nothing give zeros
            assert not got[b, c:].any()


def _run(q, k, v, mask, dtype, force_generic, cache_like=False, n_heads_for_plan=None):
    from recurrent_drafting_amd import attention

    tq, tk, tv = (_dev(x, torch.float32).to(dtype) for x in (q, k, v))
    B, H, nq, D = tq.shape
    # q arrives as the transpose view of (B, nq, H, D), as in the model
    tq = tq.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    if cache_like:  # K/V as views into a longer pre-allocated cache
        kv = tk.shape[2]
        big_k = torch.zeros(B, tk.shape[1], kv + 37, D, dtype=dtype, device="cuda")
        big_v = torch.full_like(big_k, 3.0)
        big_k[:, :, :kv] = tk; big_v[:, :, :kv] = tv
        tk, tv = big_k[:, :, :kv], big_v[:, :, :kv]
    prep = attention.prepare(_dev(mask, torch.bool), n_heads=n_heads_for_plan or H)
    out = attention.masked_attention(tq, tk, tv, prep, force_generic=force_generic)
    torch.cuda.synchronize()
    ref_in = [x.float().cpu().numpy() for x in (tq, tk, tv)]  # the oracle sees the rounded inputs
    # on a GPU the reference first turns empty rows into all-True rows (modeling_llama.py:264-265),
    # so such a row attends to every key with its real scores
    ref = O.masked_attention(*ref_in, T.fully_masked_rows_to_true(mask))
    return out.float().cpu().numpy().reshape(B, nq, H, D).transpose(0, 2, 1, 3), ref


def _assert_close(got, ref, dtype):
    scale = np.abs(ref).max()
    tol = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-3}[dtype]
    err = np.abs(got - ref).max()
    assert err <= tol * scale, f"max err {err:.3e} vs scale {scale:.3e} ({dtype})"


def _tree_case(B, W, L, prev_lens, seed):
    beams = T.synthetic_beams(B, W, L, vocab=50, seed=seed)
    S = max(prev_lens)
    pm = np.zeros((B, S), dtype=np.int64)
    for b, n in enumerate(prev_lens):
        pm[b, S - n :] = 1
    _, _, mask, _, _ = T.pack(beams, pm)
    return mask


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("H,Hkv,D", [(4, 4, 32), (4, 2, 64), (2, 1, 128), (3, 3, 80)])
def test_generic_kernel_small(dtype, H, Hkv, D):
    mask = _tree_case(2, 4, 3, [5, 9], seed=D)
    rng = np.random.default_rng(D)
    B, nq, kv = mask.shape
    q = rng.standard_normal((B, H, nq, D)); k = rng.standard_normal((B, Hkv, kv, D)); v = rng.standard_normal((B, Hkv, kv, D))
    got, ref = _run(q, k, v, mask, dtype, force_generic=True, cache_like=True)
    _assert_close(got, ref, dtype)


def test_generic_kernel_random_mask_with_empty_rows():
    rng = np.random.default_rng(7)
    B, H, nq, kv, D = 2, 2, 6, 700, 32
    mask = rng.random((B, nq, kv)) > 0.7
    mask[0, 2] = False
    mask[1, :, :300] = False
    q = rng.standard_normal((B, H, nq, D)); k = rng.standard_normal((B, H, kv, D)); v = rng.standard_normal((B, H, kv, D))
    got, ref = _run(q, k, v, mask, torch.float32, force_generic=True)
    _assert_close(got, ref, torch.float32)


@pytest.mark.parametrize("B,H,Hkv,W,L,prev_lens", [
    (1, 1, 1, 2, 3, [40]),            # one tile, one item
    (2, 2, 2, 8, 5, [100, 37]),       # ragged prefix, < 64 queries
    (2, 2, 2, 24, 5, [300, 150]),     # 64..128 queries: four row blocks, keys of a tile split over wave pairs
    (2, 4, 2, 45, 5, [700, 1300]),    # > 32 queries per wave, split keys, GQA
    (1, 2, 2, 64, 5, [64]),           # > 256 queries: two query tiles
    (3, 2, 2, 16, 4, [2000, 5, 900]),  # several splits and a nearly empty prefix
])
def test_mfma_kernel(B, H, Hkv, W, L, prev_lens):
    mask = _tree_case(B, W, L, prev_lens, seed=W)
    rng = np.random.default_rng(W * 7 + L)
    _, nq, kv = mask.shape
    D = 128
    q = rng.standard_normal((B, H, nq, D)); k = rng.standard_normal((B, Hkv, kv, D)); v = rng.standard_normal((B, Hkv, kv, D))
    got, ref = _run(q, k, v, mask, torch.bfloat16, force_generic=False, cache_like=True)
    _assert_close(got, ref, torch.bfloat16)
    # (with few heads the plan above cuts long rows into minimum-size items and merges partials)
    # a plan made for many heads leaves every row whole: one work item per row, no partials
    got3, _ = _run(q, k, v, mask, torch.bfloat16, force_generic=False, cache_like=True, n_heads_for_plan=4096)
    _assert_close(got3, ref, torch.bfloat16)
    got2, _ = _run(q, k, v, mask, torch.bfloat16, force_generic=True, cache_like=True)
    _assert_close(got2, ref, torch.bfloat16)


@pytest.mark.parametrize("nq", [127, 128, 129, 150, 160, 161, 192, 193, 256, 257])
def test_mfma_kernel_every_wave_layout(nq):
    """Query counts on both sides of every boundary between the ways the waves of a workgroup share
    rows and keys (128, 160, 192, 256 rows per workgroup), odd and even numbers of key tiles."""
    rng = np.random.default_rng(nq)
    B, H = 2, 2
    for kv_prev in (70, 200):
        kv = kv_prev + nq
        mask = rng.random((B, nq, kv)) > 0.35
        mask[:, :, kv_prev:] &= np.tril(np.ones((nq, nq), dtype=bool))  # causal over the new tokens
        mask[0, :, : kv_prev // 2] = False  # row 0 starts later: its first tiles are skipped
        mask[1, nq // 2, :] = False  # a query with no key at all
        q = rng.standard_normal((B, H, nq, 128)); k = rng.standard_normal((B, H, kv, 128)); v = rng.standard_normal((B, H, kv, 128))
        got, ref = _run(q, k, v, mask, torch.bfloat16, force_generic=False, cache_like=True)
        _assert_close(got, ref, torch.bfloat16)


@pytest.mark.parametrize("nq,kv_prev", [(300, 1500), (150, 2100), (96, 1300)])
def test_mfma_kernel_split_rows_in_every_layout_against_the_oracle(nq, kv_prev):
    """Long rows with few heads: the plan cuts every row into 512-key items, so several work items
    (and, at 300 queries, two query tiles each) meet at the arrival counters and one of them merges."""
    from recurrent_drafting_amd import attention

    rng = np.random.default_rng(nq + kv_prev)
    B, H = 2, 2
    kv = kv_prev + nq
    mask = rng.random((B, nq, kv)) > 0.5
    mask[1, :, : kv_prev - 200] = False  # a row that starts late: fewer items than row 0
    q = rng.standard_normal((B, H, nq, 128)); k = rng.standard_normal((B, H, kv, 128)); v = rng.standard_normal((B, H, kv, 128))
    prep = attention.prepare(_dev(mask, torch.bool), n_heads=H)
    assert int(prep.plan[0]) >= 4  # split
    got, ref = _run(q, k, v, mask, torch.bfloat16, force_generic=False, cache_like=True)
    _assert_close(got, ref, torch.bfloat16)


def test_split_rows_merge_is_repeatable_on_one_plan():
    """Every row split into many work items (a plan made for one head: minimum-size items): the item
    that arrives last merges the partials.  Launch after launch on the same plan (one per layer in
    the model) must give the same bits, equal to the unsplit result up to the rounding of the
    merge, and the plan itself is only read."""
    from recurrent_drafting_amd import attention

    torch.manual_seed(3)
    B, H, D, nq, kv = 3, 6, 128, 150, 1900
    q = torch.randn(B, nq, H, D, device="cuda", dtype=torch.bfloat16).permute(0, 2, 1, 3)
    k = torch.randn(B, H, kv, D, device="cuda", dtype=torch.bfloat16)
    v = torch.randn(B, H, kv, D, device="cuda", dtype=torch.bfloat16)
    mask = torch.rand(B, nq, kv, device="cuda") > 0.4
    whole_plan = attention.prepare(mask, n_heads=4096)  # a share of many heads: nothing is split
    assert int(whole_plan.plan[0]) == B
    whole = attention.masked_attention(q, k, v, whole_plan)
    prep = attention.prepare(mask, n_heads=1)
    assert int(prep.plan[0]) >= 3 * B  # really split
    plan_before = prep.plan.clone()
    first = attention.masked_attention(q, k, v, prep).clone()
    for _ in range(40):
        again = attention.masked_attention(q, k, v, prep)
        assert torch.equal(again, first)
    assert torch.equal(prep.plan, plan_before)
    assert (first.float() - whole.float()).abs().max() <= 2e-2 * whole.float().abs().max()


def test_split_rows_merge_when_the_arrival_counters_come_round_again():
    """The arrival counters are a ring of 2^18 that launches take slabs of in turn: enough launches
    to go round it more than once (every launch of the second lap counts on counters that another
    launch used before it), one result throughout."""
    from recurrent_drafting_amd import attention

    torch.manual_seed(5)
    B, H, D, nq, kv = 3, 128, 128, 8, 1900
    q = torch.randn(B, nq, H, D, device="cuda", dtype=torch.bfloat16).permute(0, 2, 1, 3)
    k = torch.randn(B, 1, kv, D, device="cuda", dtype=torch.bfloat16)
    v = torch.randn(B, 1, kv, D, device="cuda", dtype=torch.bfloat16)
    mask = torch.rand(B, nq, kv, device="cuda") > 0.3
    prep = attention.prepare(mask, n_heads=1)
    assert int(prep.plan[0]) >= 3 * B
    first = attention.masked_attention(q, k, v, prep).clone()
    per_launch = B * H
    laps = 2 * (1 << 18) // per_launch + 3
    for i in range(laps):
        again = attention.masked_attention(q, k, v, prep)
        if i % 16 == 0 or i >= laps - 3:
            assert torch.equal(again, first), i


def test_two_streams_share_one_plan():
    """Bits and plan are only read and every launch counts arrivals on counters of its own, so two
    streams may run split rows on one plan at the same time (each with its own workspace)."""
    import dataclasses

    from recurrent_drafting_amd import attention

    torch.manual_seed(9)
    B, H, D, nq, kv = 4, 16, 128, 60, 2300
    q = torch.randn(B, nq, H, D, device="cuda", dtype=torch.bfloat16).permute(0, 2, 1, 3)
    k = torch.randn(B, 2, kv, D, device="cuda", dtype=torch.bfloat16)
    v = torch.randn(B, 2, kv, D, device="cuda", dtype=torch.bfloat16)
    mask = torch.rand(B, nq, kv, device="cuda") > 0.5
    prep_a = attention.prepare(mask, n_heads=1)
    prep_b = dataclasses.replace(prep_a, workspace=None)
    assert int(prep_a.plan[0]) >= 3 * B
    want = attention.masked_attention(q, k, v, prep_a).clone()
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[], []]
    for _ in range(30):
        for i, (st, prep) in enumerate(zip(streams, (prep_a, prep_b))):
            with torch.cuda.stream(st):
                outs[i].append(attention.masked_attention(q, k, v, prep))
    torch.cuda.synchronize()
    for side in outs:
        for got in side:
            assert torch.equal(got, want)


def test_mfma_kernel_pad_tokens_inside_the_prefix_and_empty_rows():
    """Keys masked by VALUE in the middle of the prefix, and a query row with no key at all."""
    rng = np.random.default_rng(11)
    mask = _tree_case(2, 6, 4, [333, 200], seed=3).copy()
    mask[:, :, rng.integers(150, 300, size=20)] = False
    mask[1, 4, :] = False
    B, nq, kv = mask.shape
    q = rng.standard_normal((B, 2, nq, 128)); k = rng.standard_normal((B, 2, kv, 128)); v = rng.standard_normal((B, 2, kv, 128))
    got, ref = _run(q, k, v, mask, torch.bfloat16, force_generic=False)
    _assert_close(got, ref, torch.bfloat16)


def test_verify_attention_benchmark_shape():
    """Config 3: 32 heads x 128, batch 8, cached length U[500,2548], tree from the config-2 beams.
    Full size against a float32 torch reference on the GPU; two heads against the float64 oracle."""
    from recurrent_drafting_amd import attention

    rng = np.random.default_rng(123)
    B, H, D = 8, 32, 128
    lens = rng.integers(500, 2549, size=B)
    beams = T.synthetic_beams(B, 45, 5, seed=123)
    S = int(lens.max())
    pm = np.zeros((B, S), dtype=np.int64)
    for b in range(B):
        pm[b, S - lens[b] :] = 1
    _, _, mask, _, _ = T.pack(beams, pm)
    _, nq, kv = mask.shape
    torch.manual_seed(0)
    cache = torch.randn(2, B, H, kv + 64, D, device="cuda", dtype=torch.bfloat16)
    k, v = cache[0, :, :, :kv], cache[1, :, :, :kv]
    q = torch.randn(B, nq, H, D, device="cuda", dtype=torch.bfloat16).permute(0, 2, 1, 3)
    tmask = _dev(mask, torch.bool)
    prep = attention.prepare(tmask, n_heads=H)
    out = attention.masked_attention(q, k, v, prep).view(B, nq, H, D).permute(0, 2, 1, 3).float()
    s = torch.einsum("bhqd,bhkd->bhqk", q.float(), k.float()) / D ** 0.5
    s = s.masked_fill(~tmask[:, None], float("-inf"))
    ref = torch.einsum("bhqk,bhkd->bhqd", torch.softmax(s, dim=-1), v.float())
    err = (out - ref).abs().max().item()
    assert err <= 2e-2 * ref.abs().max().item(), err
    heads = [0, 17]
    ref64 = O.masked_attention(q[:, heads].float().cpu().numpy(), k[:, heads].float().cpu().numpy(),
                               v[:, heads].float().cpu().numpy(), mask)
    _assert_close(out[:, heads].cpu().numpy(), ref64, torch.bfloat16)


def test_argument_errors():
    from recurrent_drafting_amd import attention

    mask = torch.ones(1, 2, 5, dtype=torch.bool, device="cuda")
    prep = attention.prepare(mask)
    q = torch.zeros(1, 2, 2, 16, device="cuda"); k = torch.zeros(1, 2, 6, 16, device="cuda")
    with pytest.raises(AssertionError, match="mismatch"):
        attention.masked_attention(q, k, k, prep)
    k = torch.zeros(1, 3, 5, 16, device="cuda")
    with pytest.raises(RuntimeError, match="multiple"):
        attention.masked_attention(q, k, k, prep)


def _fused_case(B, H, Hkv, n_new, prev_lens, seed, shifted, packed, max_len=None):
    """One layer's new tokens through kv_cache.rope_append + attention.masked_attention and through
    attention.rope_attention(fused=True), on two caches with the same contents."""
    import recurrent_drafting_amd as rd
    from recurrent_drafting_amd import attention, kv_cache
    from recurrent_drafting_amd.packed_rows import PackedRows

    D = 128
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(seed)
    prev = max(prev_lens)
    max_len = max_len or prev + n_new + 7
    kv_len = prev + n_new
    caches = []
    filler = torch.randn((1, 2, B, Hkv, max_len, D), generator=g).to(torch.bfloat16)
    shift = torch.tensor([prev - p if shifted else 0 for p in prev_lens], dtype=torch.int32)
    for _ in range(2):
        c = kv_cache.Cache(B, max_len, 1, Hkv, D, torch.bfloat16, dev)
        c._cache.copy_(filler.to(dev))
        c.rows_in_place = shifted
        c.shift.copy_(shift.to(dev))
        for view in c.sliced[0]:
            view.length = prev
        caches.append(c)
    # columns [prev - len_b, prev) hold row b's context (left-padded); with shifts they live at the
    # front of the slab.  The new tokens see their context and a random lower-triangular tree.
    mask = torch.zeros((B, n_new, kv_len), dtype=torch.bool)
    tree = torch.rand((B, n_new, n_new), generator=g) < 0.4
    tree = torch.tril(tree) | torch.eye(n_new, dtype=torch.bool)
    counts = torch.randint(max(1, n_new // 2), n_new + 1, (B,), generator=g) if packed else torch.full((B,), n_new)
    counts[0] = n_new
    for b in range(B):
        mask[b, :, prev - prev_lens[b]:prev] = True
        mask[b, :, prev:] = tree[b]
        mask[b, :, prev + int(counts[b]):] = False
    mask = mask.to(dev)
    nq, nk = H * D, Hkv * D
    rows = None
    if packed:
        total = int(counts.sum())
        rows = PackedRows.from_counts(counts.to(dev), total, n_new)
        qkv = torch.randn((rows.rows, nq + 2 * nk), generator=g).to(torch.bfloat16).to(dev)
    else:
        qkv = torch.randn((B, n_new, nq + 2 * nk), generator=g).to(torch.bfloat16).to(dev)
    position_ids = (torch.tensor(prev_lens).view(B, 1) + torch.randint(0, 5, (B, n_new), generator=g)).to(dev)
    table = torch.randn((max(prev_lens) + 8, 2, D), generator=g).to(torch.bfloat16).to(dev)
    cos, sin = table[:, 0].contiguous(), table[:, 1].contiguous()
    outs = []
    for c, fused in zip(caches, (False, True)):
        x = qkv.clone()
        q, k, v = x[..., :nq], x[..., nq:nq + nk], x[..., nq + nk:]
        prepared = attention.prepare(mask, n_heads=H, kv_shift=c.shift if shifted else None)
        outs.append(attention.rope_attention(q, k, v, cos, sin, position_ids, c.sliced[0], prepared,
                                             rows=rows, fused=fused))
        assert c.sliced[0][0].length == kv_len and c.sliced[0][1].length == kv_len
    torch.cuda.synchronize()
    live = outs[0].shape[0] if rows is None else rows.total
    return outs[0][:live], outs[1][:live], caches[0]._cache, caches[1]._cache


@pytest.mark.gpu
@pytest.mark.parametrize("B,H,Hkv,n_new,prev_lens,shifted,packed", [
    (2, 4, 4, 23, [200, 131], False, False),
    (3, 4, 2, 37, [300, 17, 150], True, False),
    (3, 8, 2, 40, [1, 64, 129], True, True),
    (2, 4, 4, 130, [500, 420], True, True),       # five row blocks
    (2, 2, 2, 256, [90, 64], False, False),       # the largest fused query count
    (4, 32, 32, 26, [2500, 300, 1800, 64], True, True),  # rows cut into several items
])
def test_rope_attention_one_kernel_equals_two(B, H, Hkv, n_new, prev_lens, shifted, packed):
    two, one, cache_two, cache_one = _fused_case(B, H, Hkv, n_new, prev_lens, 11, shifted, packed)
    assert torch.equal(one.view(torch.int16), two.view(torch.int16))
    assert torch.equal(cache_one.view(torch.int16), cache_two.view(torch.int16))


@pytest.mark.gpu
def test_rope_attention_on_a_slab_that_ends_behind_the_new_tokens():
    two, one, cache_two, cache_one = _fused_case(2, 4, 4, 20, [100, 40], 5, True, False, max_len=120)
    assert torch.equal(one.view(torch.int16), two.view(torch.int16))
    assert torch.equal(cache_one.view(torch.int16), cache_two.view(torch.int16))


@pytest.mark.gpu
def test_rope_attention_refuses_what_the_fused_kernel_does_not_cover():
    import ctypes as C
    from recurrent_drafting_amd import _hip
    lib = _hip.lib()
    assert lib.rd_rope_verify_attention_eligible(_hip.dtype_code(torch.bfloat16), 32, 128, 26) == 1
    assert lib.rd_rope_verify_attention_eligible(_hip.dtype_code(torch.bfloat16), 32, 128, 257) == 0
    assert lib.rd_rope_verify_attention_eligible(_hip.dtype_code(torch.bfloat16), 32, 64, 26) == 0
    assert lib.rd_rope_verify_attention_eligible(_hip.dtype_code(torch.float16), 32, 128, 26) == 0
    t = torch.zeros(4096, dtype=torch.bfloat16, device="cuda")
    s3, s2 = (C.c_int64 * 3)(0, 64, 64), (C.c_int64 * 2)(0, 64)
    rc = lib.rd_rope_verify_attention(
        _hip.ptr(t), s3, _hip.ptr(t), s2, _hip.ptr(t), s2, _hip.ptr(t), _hip.ptr(t), 4,
        _hip.ptr(torch.zeros(4, dtype=torch.long, device="cuda")), 1, _hip.ptr(t), _hip.ptr(t), s3, 8,
        _hip.ptr(t), s3, _hip.dtype_code(torch.bfloat16), 1, 1, 1, 1, 8, 64, 1.0,
        _hip.ptr(t), _hip.ptr(t.view(torch.int32)), None, 0, None, None)
    assert rc == -2 and b"rd_rope_verify_attention" in lib.rd_last_error()
