"""KV cache rows kept in place across re-alignments (kv_cache.Cache.rows_in_place).

The reference moves the whole live cache whenever the accepted lengths differ between rows
(recurrent_drafting.py:200-209).  With rows in place only a per-row shift changes; these tests
pin that the two ways agree: bit-exact cache contents after materialize(), identical attention
output, identical token streams."""
import os
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "golden"))
import tiny_models as tm  # noqa: E402

pytestmark = pytest.mark.gpu


def _pair(B, max_len, layers=2, heads=3, D=16, dtype=torch.float32):
    from recurrent_drafting_amd import kv_cache

    a = kv_cache.Cache(B, max_len, layers, heads, D, dtype, torch.device("cuda"))
    b = kv_cache.Cache(B, max_len, layers, heads, D, dtype, torch.device("cuda"))
    a._cache.normal_(generator=torch.Generator(device="cuda").manual_seed(1))
    b._cache.copy_(a._cache)
    a.rows_in_place = True
    return a, b


@pytest.mark.parametrize("seed,switch_off", [(0, False), (1, False), (2, True)])
def test_successive_realignments_then_materialize_equal_the_moved_cache(seed, switch_off):
    """Three re-alignments with random accepted lengths and ragged left padding; between them the
    tree rows of the next step are written through rope_append's cache rows (here: plain copies)."""
    from recurrent_drafting_amd import acceptance

    rng = np.random.default_rng(seed)
    B, W, L, prev0 = 4, 5, 4, 23
    pads = rng.integers(0, 9, size=B)
    pads[rng.integers(0, B)] = 0
    ids = torch.from_numpy(rng.integers(1, 50, size=(B, prev0))).cuda()
    for r in range(B):
        ids[r, : pads[r]] = 0
    max_len = prev0 + 3 * L + W * L + int(pads.max()) + 8
    in_place, moved = _pair(B, max_len)
    ids_a, ids_b = ids.clone(), ids.clone()
    for step in range(3):
        prev = ids_a.shape[1]
        beams = torch.from_numpy(rng.integers(1, 50, size=(B, W, L))).cuda()
        n_tok = torch.from_numpy(rng.integers(0, L, size=B)).cuda()
        seq = torch.from_numpy(rng.integers(0, W, size=B)).cuda()
        # the rows a verification step would have appended: identical values for both caches, written
        # where each cache keeps column prev + t
        new_rows = torch.randn(in_place._cache.shape[:4] + (W * L, in_place._cache.shape[5]), device="cuda")
        moved._cache[:, :, :, :, prev : prev + W * L, :] = new_rows
        shift = in_place.shift.cpu().tolist()
        for r in range(B):
            in_place._cache[:, :, r, :, prev - shift[r] : prev - shift[r] + W * L, :] = new_rows[:, :, r]
        in_place.set_length(prev + W * L)
        moved.set_length(prev + W * L)
        ids_a = acceptance.realign(ids_a, n_tok, seq, beams, in_place, 0)
        ids_b = acceptance.realign(ids_b, n_tok, seq, beams, moved, 0)
        assert torch.equal(ids_a, ids_b)
    assert in_place._shifted and in_place.shift.abs().sum() > 0, "the case never shifted a row"
    length = ids_a.shape[1]
    if switch_off:
        in_place.rows_in_place = False  # switching the mode off brings the rows home first
    else:
        in_place.materialize()
    assert not in_place._shifted and int(in_place.shift.abs().sum()) == 0
    new_pads = (ids_a == 0).long().cumprod(1).sum(1).cpu().tolist()
    for r in range(B):
        got = in_place._cache[:, :, r, :, new_pads[r] : length, :]
        want = moved._cache[:, :, r, :, new_pads[r] : length, :]
        assert torch.equal(got, want), f"row {r}"


@pytest.mark.parametrize("dtype,prev", [(torch.float32, 70), (torch.bfloat16, 70), (torch.bfloat16, 1400)])
def test_attention_and_rope_append_follow_the_shift(dtype, prev):
    """rope_append writes and the attention reads cache row c - shift[b]: same output as the same
    data laid out without a shift.  (1400 cached keys: the rows are cut into several work items, so
    the shift also travels with split rows and their merge.)"""
    from recurrent_drafting_amd import attention, kv_cache

    torch.manual_seed(3)
    B, H, D, n = 3, 4, 128, 9
    max_len = prev + n + 40
    shift = torch.tensor([5, 0, -3], dtype=torch.int32, device="cuda")  # row 2 sits 3 rows further right
    plain = kv_cache.Cache(B, max_len, 1, H, D, dtype, torch.device("cuda"))
    shifted = kv_cache.Cache(B, max_len, 1, H, D, dtype, torch.device("cuda"))
    live = torch.randn(2, B, H, prev, D, device="cuda").to(dtype)
    first = [8, 0, 2]  # left pads (columns) of each row; shift <= pads keeps cache rows >= 0
    for b in range(B):
        plain._cache[0, :, b, :, first[b] : prev] = live[:, b, :, first[b] :]
        s = int(shift[b])
        shifted._cache[0, :, b, :, first[b] - s : prev - s] = live[:, b, :, first[b] :]
    shifted.shift.copy_(shift)
    shifted.rows_in_place = True
    shifted._shifted = True
    plain.set_length(prev)
    shifted.set_length(prev)
    q = torch.randn(B, n, H * D, device="cuda").to(dtype)
    k = torch.randn(B, n, H * D, device="cuda").to(dtype)
    v = torch.randn(B, n, H * D, device="cuda").to(dtype)
    cos = torch.randn(prev + n + 8, D, device="cuda").to(dtype)
    sin = torch.randn(prev + n + 8, D, device="cuda").to(dtype)
    pos = (prev + torch.arange(n, device="cuda")).repeat(B, 1)
    mask = torch.ones(B, n, prev + n, dtype=torch.bool, device="cuda").tril(prev)
    for b in range(B):
        mask[b, :, : first[b]] = False
    outs = []
    for cache in (plain, shifted):
        qq, keys, values = kv_cache.rope_append(q.clone(), k, v, cos, sin, pos, cache.sliced[0])
        prepared = attention.prepare(mask, n_heads=H, kv_shift=cache.shift if cache.rows_in_place else None)
        outs.append(attention.masked_attention(qq, keys, values, prepared))
        if prev > 1000:
            assert int(prepared.plan[0]) > B, "the rows were not split"
    assert torch.equal(outs[0], outs[1])
    shifted.materialize()
    for b in range(B):
        assert torch.equal(shifted._cache[0, :, b, :, first[b] : prev + n], plain._cache[0, :, b, :, first[b] : prev + n])


def _streams(in_place, seed, batch, prompt_len, left_pads, new_tokens, W, L, sampling=False):
    import recurrent_drafting_amd as rd
    from transformers.models.llama.configuration_llama import LlamaConfig

    llama_sd, drafter_sd = tm.markov(seed)
    # the toy pair has its attention switched off; switch it back on at half strength, so that the
    # tokens depend on what the attention reads from the cache while the drafter still often agrees
    drawn = tm.draw(tm.llama_shapes(), seed)
    for name in llama_sd:
        if name.endswith("o_proj.weight"):
            llama_sd[name] = drawn[name] * 0.5
    llm = rd.modeling_llama.LlamaForCausalLM(LlamaConfig(**tm.LLAMA))
    drafter = rd.modeling_drafter.Drafter(rd.configuration_drafter.DrafterConfig(**tm.DRAFTER))
    llm.load_state_dict(llama_sd, strict=False)
    drafter.load_state_dict(drafter_sd)
    model = rd.RecurrentDrafting(llm.cuda().eval(), drafter.cuda().eval())
    model.kv_rows_in_place = in_place
    ids = tm.prompt(batch, prompt_len, tm.LLAMA["vocab_size"], seed, left_pads)
    torch.manual_seed(7)
    ledger = rd.stats.Ledger()
    steps = [t.cpu().tolist() for t in model.generate(
        ledger, ids.cuda(), prompt_len + new_tokens, rd.BeamShape(W, L), rd.SamplingArgs(1.0, not sampling),
        rd.SpecialTokens(0, None))]
    return steps, ledger.records[0]["avg_num_accepted"]


@pytest.mark.parametrize("sampling", [False, True])
def test_generate_is_the_same_with_rows_in_place_and_with_moved_rows(sampling):
    """Markov-chain models accept several tokens per step, differently per row, so the rows shift
    against each other on most steps; ragged left padding on top."""
    args = dict(seed=21, batch=4, prompt_len=12, left_pads=[0, 3, 7, 1], new_tokens=40, W=6, L=4, sampling=sampling)
    a, acc = _streams(True, **args)
    b, _ = _streams(False, **args)
    assert a == b
    assert max(acc) > 0.2, "nothing was accepted: the rows never shifted"


def test_rope_append_drops_rows_that_a_shift_would_put_outside_the_cache():
    """A shift that leaves the slab is never followed: q is still rotated, k and v of that row are
    dropped, nothing outside the row's slab is written."""
    from recurrent_drafting_amd import kv_cache

    torch.manual_seed(5)
    dtype, B, H, D, prev, n, max_len = torch.float32, 2, 2, 32, 6, 4, 12
    cache = kv_cache.Cache(B, max_len, 1, H, D, dtype, torch.device("cuda"))
    cache._cache.fill_(7.0)
    cache.shift.copy_(torch.tensor([-5, 9], dtype=torch.int32))  # row 0: rows 11..14 (12+ outside); row 1: rows -3..0
    cache.rows_in_place = True
    cache._shifted = True
    cache.set_length(prev)
    q = torch.randn(B, n, H * D, device="cuda")
    k = torch.randn(B, n, H * D, device="cuda")
    v = torch.randn(B, n, H * D, device="cuda")
    cos = torch.ones(prev + n, D, device="cuda")
    sin = torch.zeros(prev + n, D, device="cuda")
    pos = (prev + torch.arange(n, device="cuda")).repeat(B, 1)
    qq, _, _ = kv_cache.rope_append(q.clone(), k, v, cos, sin, pos, cache.sliced[0])
    assert torch.equal(qq.transpose(1, 2).reshape(B, n, H * D), q)  # identity rotation, every row
    raw = cache._cache[0]  # (2, B, H, max_len, D)
    kk = k.view(B, n, H, D).transpose(1, 2)
    # row 0: token 0 lands in cache row 11, tokens 1..3 would be rows 12..14: dropped
    assert torch.equal(raw[0, 0, :, 11], kk[0, :, 0]) and (raw[0, 0, :, :11] == 7).all()
    # row 1: tokens 0..2 would be rows -3..-1: dropped; token 3 lands in row 0
    assert torch.equal(raw[0, 1, :, 0], kk[1, :, 3]) and (raw[0, 1, :, 1:] == 7).all()


def test_timing_sample_times_every_nth_launch():
    from recurrent_drafting_amd import _hip, acceptance

    x = torch.randn(4, 1000, device="cuda")
    try:
        _hip.timing_select("argmax_rows_kernel")
        _hip.timing_sample(3)
        _hip.timing_enable(True)
        for _ in range(10):
            acceptance.argmax_rows(x)
        torch.cuda.synchronize()
        got = _hip.timing_collect()
        assert got["argmax_rows_kernel"][0] == 4  # launches 0, 3, 6, 9
    finally:
        _hip.timing_enable(False)
        _hip.timing_select(None)
        _hip.timing_sample(1)


def test_stream_tiles_probe_reads_what_it_is_given_and_refuses_the_rest():
    """The memory-side yardstick of the attention (bench_stream_tiles of the bench-only library that
    kernel_bench.py loads): every depth folds the same tiles into the same checksum, a slab shorter
    than its tiles is refused before anything runs."""
    import os
    import sys

    import numpy as np
    from recurrent_drafting_amd import _hip

    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import kernel_bench

    lib = kernel_bench.bench_library()

    slabs, tiles, rows = 6, 8, 8 * 64 + 7  # (a whole number of rounds for every depth: the probe repeats its last tile otherwise)
    k = torch.randint(-2**31, 2**31 - 1, (slabs, rows, 64), dtype=torch.int32, device="cuda")  # 256-byte rows
    v = torch.randint(-2**31, 2**31 - 1, (slabs, rows, 64), dtype=torch.int32, device="cuda")
    words = np.concatenate([t[:, : tiles * 64].reshape(slabs, -1).cpu().numpy() for t in (k, v)], axis=1)
    want = np.bitwise_xor.reduce(words, axis=1)
    for depth in (1, 2, 4):
        sink = torch.zeros(slabs * 512, dtype=torch.int32, device="cuda")
        assert lib.bench_stream_tiles(_hip.ptr(k), _hip.ptr(v), rows * 256, slabs, tiles, depth, _hip.ptr(sink), 1, _hip.stream(), None) == 0
        torch.cuda.synchronize()
        got = np.bitwise_xor.reduce(sink.view(slabs, 512).cpu().numpy(), axis=1)
        assert np.array_equal(got, want), depth
    sink = torch.zeros(slabs * 512, dtype=torch.int32, device="cuda")
    assert lib.bench_stream_tiles(_hip.ptr(k), _hip.ptr(v), tiles * 64 * 256 - 16, slabs, tiles, 2, _hip.ptr(sink), 1, None, None) == -1
    assert lib.bench_stream_tiles(_hip.ptr(k), _hip.ptr(v), rows * 256, slabs, tiles, 3, _hip.ptr(sink), 1, None, None) == -2
    assert lib.bench_stream_tiles(None, _hip.ptr(v), rows * 256, slabs, tiles, 2, _hip.ptr(sink), 1, None, None) == -1
