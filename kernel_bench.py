"""Per-kernel micro-benchmarks of libredrafter_hip.so on one MI355X.

    python kernel_bench.py [--only NAME[,NAME]] [--reps N] [--json]

Each case runs one entry point on the benchmark shapes (batch 8, beam 45x5, vocabulary 32000,
32 heads x 128, 32 layers; cached length U[500, 2548] for the attention), times the kernels with
the library's HIP-event timing (`rd_timing_enable`), and prices the ALGORITHMIC bytes or FLOPs of
one launch against the MI355X peaks (HBM 8 TB/s, bf16 MFMA 2.5 PFLOP/s).  Inputs are synthetic and
seeded; nothing here checks results (tests/ does).
"""

from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "ml-recurrent-drafter_amd"))

import recurrent_drafting_amd as rd  # noqa: E402
from recurrent_drafting_amd import _hip, acceptance, attention, kv_cache, modeling_drafter, tree_attention  # noqa: E402

HBM, MFMA = 8000.0, 2500.0  # GB/s, TFLOP/s
B, W, L, V, H, D, LAYERS = 8, 45, 5, 32000, 32, 128, 32


def synthetic_beams(batch, width, length, vocab=32000, seed=123, p_copy=0.6, zipf_s=1.1, n_first=4):
    """Beams with shared prefixes: token 0 from 4 values, later positions copy beam i-1 with p=0.6,
    else Zipf(1.1) over the vocabulary (benchmark configuration 2)."""
    rng = np.random.default_rng(seed)
    pz = np.arange(1, vocab + 1, dtype=np.float64) ** (-zipf_s)
    pz /= pz.sum()
    beams = np.zeros((batch, width, length), dtype=np.int64)
    beams[:, :, 0] = rng.integers(0, n_first, size=(batch, width))
    draws = rng.choice(vocab, size=(batch, width, length), p=pz)
    copy = rng.random((batch, width, length)) < p_copy
    for i in range(width):
        for k in range(1, length):
            beams[:, i, k] = np.where(copy[:, i, k] & (i > 0), beams[:, i - 1, k] if i > 0 else 0, draws[:, i, k])
    return beams


def timed(fn, reps, warm=3):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    _hip.timing_enable(True)
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    out = _hip.timing_collect()
    _hip.timing_enable(False)
    return {k: (n // reps, ms * 1e3 / n) for k, (n, ms) in out.items()}  # launches per call, avg us


def report(rows, name, kernels, work, unit, note=""):
    """work: {kernel: algorithmic bytes (unit GB/s) or FLOPs (unit TFLOP/s) per launch}."""
    for k, (per_call, us) in sorted(kernels.items()):
        w = work.get(k)
        rate = frac = None
        if w is not None:
            if unit[k] == "GB/s":
                rate = w / (us * 1e-6) / 1e9
                frac = rate / HBM
            else:
                rate = w / (us * 1e-6) / 1e12
                frac = rate / MFMA
        rows.append(dict(case=name, kernel=k, launches_per_call=per_call, avg_us=round(us, 2),
                         algorithmic_work=w, achieved=None if rate is None else round(rate, 1),
                         unit=unit.get(k), frac_of_peak=None if frac is None else round(frac, 4), note=note))


def case_tree(rows, reps, replicate=1):
    beams = torch.tensor(np.concatenate([synthetic_beams(B, W, L, seed=123 + r) for r in range(replicate)]), device="cuda")
    nb = beams.shape[0]
    for prev in (0, 2548):
        pm = torch.ones((nb, prev), dtype=torch.bool, device="cuda")
        tree = tree_attention.build_tree(beams)
        n = tree.n
        k = timed(lambda: tree_attention.pack(beams, pm), reps)
        io = nb * W * L * 8 * 2 + 3 * nb * n * 8
        work = {"tree_rows_kernel": nb * W * L * 8 * 3, "tree_fill_kernel": 3 * nb * n * 8 + nb * n * 12,
                "tree_mask_kernel": nb * n * (prev + n) + nb * prev}
        report(rows, f"tree_pack batch {nb} prev {prev} (n={n})", k, work,
               {x: "GB/s" for x in work}, note=f"whole pack moves {io + work['tree_mask_kernel']} algorithmic bytes")


def attention_case(seed=123, full_len=None, p_copy=0.6):
    rng = np.random.default_rng(seed)
    lens = rng.integers(500, 2549, size=B) if full_len is None else np.full(B, full_len)
    S = int(lens.max())
    beams = torch.tensor(synthetic_beams(B, W, L, seed=seed, p_copy=p_copy), device="cuda")
    ids_mask = torch.zeros((B, S), dtype=torch.bool, device="cuda")
    for b in range(B):
        ids_mask[b, S - int(lens[b]):] = True
    tree = tree_attention.build_tree(beams)
    mask = tree_attention.build_mask(tree, ids_mask)
    n, kv = tree.n, S + tree.n
    torch.manual_seed(seed)
    cache = torch.randn(2, B, H, kv + 64, D, device="cuda", dtype=torch.bfloat16)
    q = torch.randn(B, n, H, D, device="cuda", dtype=torch.bfloat16).permute(0, 2, 1, 3)
    return lens, n, kv, mask, q, cache[0, :, :, :kv], cache[1, :, :, :kv]


def case_attention(rows, reps):
    for label, full_len, p_copy in (("cached length U[500,2548]", None, 0.6), ("cached length 2548 for every row", 2548, 0.6),
                                    ("cached length 525 for every row", 525, 0.6),
                                    ("narrow tree, cached length U[500,2548]", None, 0.93),
                                    ("narrow tree, cached length 525 for every row", 525, 0.93)):
        lens, n, kv, mask, q, k_, v_ = attention_case(full_len=full_len, p_copy=p_copy)
        prep = attention.prepare(mask, n_heads=H)
        kt = timed(lambda: attention.masked_attention(q, k_, v_, prep), reps)
        kp = timed(lambda: attention.prepare(mask, n_heads=H), reps)
        keys = int(lens.sum()) + B * n
        flops = 4.0 * H * D * n * keys
        byts = 2.0 * H * D * 2 * keys + 2.0 * B * H * n * D * 2
        total_us = sum(us * c for c, us in kt.values())
        report(rows, f"verify_attention {label} (n_q={n}, sum keys={keys})", kt,
               {"attn_mfma_kernel": flops}, {"attn_mfma_kernel": "TFLOP/s"},
               note=f"{flops / 1e9:.1f} GFLOP, {byts / 1e6:.0f} MB algorithmic; {total_us:.1f} us = "
                    f"{flops / total_us / 1e6:.0f} TFLOP/s, {byts / total_us / 1e3:.0f} GB/s "
                    f"({byts / total_us / 1e3 / HBM:.3f} of HBM peak)")
        report(rows, f"attn_prepare {label}", kp, {"mask_bits_kernel": B * n * kv + B * n * ((kv + 63) // 64) * 8},
               {"mask_bits_kernel": "GB/s"})


def case_beam(rows, reps):
    torch.manual_seed(0)
    for dtype, want in ((torch.bfloat16, False), (torch.bfloat16, True), (torch.float32, False)):
        logits = (torch.randn(B, W, V, device="cuda") * 1.3).to(dtype)
        lpb = -torch.rand(B, W, device="cuda") * 3
        beams = torch.randint(0, V, (B, W, 3), device="cuda")
        k = timed(lambda: modeling_drafter.beam_topk_step(logits, lpb, beams, want), reps)
        rd_bytes = B * W * V * logits.element_size() + (B * W * V * 4 if want else 0)
        report(rows, f"beam_topk {str(dtype).split('.')[-1]} log_probs={want}", k, {"beam_row_kernel": rd_bytes},
               {"beam_row_kernel": "GB/s"})


def case_logits(rows, reps):
    torch.manual_seed(1)
    n = 181
    logits = torch.randn(B, n, V, device="cuda").to(torch.bfloat16)
    k = timed(lambda: acceptance.argmax_rows(logits), reps)
    report(rows, f"argmax packed bf16 logits (B*n={B * n})", k, {"argmax_rows_kernel": B * n * V * 2}, {"argmax_rows_kernel": "GB/s"})
    k = timed(lambda: acceptance.verify_row_stats(logits, 1.0), reps)
    report(rows, "verify_row_stats packed bf16 logits", k, {"row_stats_kernel": B * n * V * 2}, {"row_stats_kernel": "GB/s"})
    hidden = torch.randn(B, n, 4096, device="cuda").to(torch.bfloat16)
    unp = torch.randint(0, n, (B, W, L), device="cuda")
    k = timed(lambda: tree_attention.unpack(hidden, unp), reps)
    report(rows, "unpack hidden (B,n,4096) bf16", k, {"gather_rows_kernel": 2 * B * W * L * 4096 * 2}, {"gather_rows_kernel": "GB/s"})


def case_kv(rows, reps):
    prev, n = 1500, 181
    max_len = prev + W * L + 64
    cache = kv_cache.Cache(B, max_len, LAYERS, H, D, torch.bfloat16, torch.device("cuda"))
    cache._cache.normal_()
    beams = torch.tensor(synthetic_beams(B, W, L), device="cuda")
    tree = tree_attention.build_tree(beams)
    n = tree.n
    row = LAYERS * 2 * H * D * 2  # bytes of one token row over all slabs of one batch row

    def unpack():
        cache.set_length(prev + n)
        cache.unpack(prev, tree.unpacker)

    k = timed(unpack, reps)
    report(rows, f"Cache.unpack prev {prev} n {n}", k, {"kv_unpack_kernel": B * row * (n + W * L)}, {"kv_unpack_kernel": "GB/s"})

    # acceptance patterns: nothing shifts / every row but one shifts by 1..4 rows
    ids = torch.randint(1, V, (B, prev), device="cuda")
    for label, n_tok in (("no row shifts", [0] * B), ("7 of 8 rows shift", [4, 0, 1, 2, 3, 0, 1, 2])):
        nt = torch.tensor(n_tok, device="cuda")
        sb = torch.zeros(B, dtype=torch.long, device="cuda")

        def compact():
            cache.set_length(prev + n)
            acceptance.realign(ids, nt, sb, beams, cache, 0, unpacker=tree.unpacker)

        k = timed(compact, reps)
        m = max(n_tok) + 1
        moved = sum((t + 1) for t in n_tok) + sum(prev for t in n_tok if m - (t + 1) != 0)
        report(rows, f"realign + kv_compact prev {prev}, {label}", k, {"kv_compact_kernel": 2 * row * moved},
               {"kv_compact_kernel": "GB/s"})
    # the same re-alignment with the cache rows kept in place (what the decode loop does): only the
    # accepted rows are copied, the change of the left padding goes into the per-row shift
    cache.rows_in_place = True

    def compact_in_place():
        cache.set_length(prev + n)
        cache.shift.zero_()
        acceptance.realign(ids, nt, sb, beams, cache, 0, unpacker=tree.unpacker)

    k = timed(compact_in_place, reps)
    report(rows, f"realign + kv_compact prev {prev}, 7 of 8 rows shift, cache rows kept in place", k,
           {"kv_append_kernel": 2 * row * sum((t + 1) for t in n_tok)}, {"kv_append_kernel": "GB/s"})


def case_slope(rows, reps):
    """The small bandwidth-bound kernels at 1x, 2x and 4x the work of a decode step: the time of a
    launch is a fixed part (launch, the kernel's chain of dependent loads; an empty kernel between
    the same two events takes about 4 us) plus bytes over a marginal rate, and at the decode step's
    size the fixed part dominates.  `marginal` is (bytes(4x) - bytes(1x)) / (time(4x) - time(1x))."""
    torch.manual_seed(1)
    n = 181

    def series(label, kernel, make):
        pts = []
        for mult in (1, 2, 4):
            fn, nbytes = make(mult)
            k = timed(fn, reps)
            pts.append((nbytes, k[kernel][1]))
            report(rows, f"{label} x{mult}", {kernel: k[kernel]}, {kernel: nbytes}, {kernel: "GB/s"})
            del fn
            torch.cuda.empty_cache()
        (b1, t1), _, (b4, t4) = pts
        marginal = (b4 - b1) / ((t4 - t1) * 1e-6) / 1e9
        fixed = t1 - b1 / (marginal * 1e9) * 1e6
        rows.append(dict(case=f"{label}: marginal rate {marginal:.0f} GB/s ({marginal / HBM * 100:.0f}% of peak), "
                              f"fixed part {fixed:.1f} us of {t1:.1f} us at x1", kernel=kernel, launches_per_call=0, avg_us=0.0,
                         algorithmic_work=None, achieved=None, unit="", frac_of_peak=None, note=""))

    def logits_case(op):
        def make(mult):
            logits = torch.randn(B * mult, n, V, device="cuda").to(torch.bfloat16)
            return (lambda: op(logits)), B * mult * n * V * 2
        return make

    def beam(mult):
        # one beam-search iteration at 1x, 2x and 4x the decode step's batch (360, 720, 1440 rows of
        # 32000 logits): the row kernel reads every row once
        logits = (torch.randn(B * mult, W, V, device="cuda") * 2).to(torch.bfloat16)
        lpb = -torch.rand(B * mult, W, device="cuda") * 4
        beams = torch.randint(0, V, (B * mult, W, 2), device="cuda")
        return (lambda: modeling_drafter.beam_topk_step(logits, lpb, beams, False)), B * mult * W * V * 2

    series("beam_topk bf16 (batch x width rows of 32000)", "beam_row_kernel", beam)
    series("argmax packed bf16 logits", "argmax_rows_kernel", logits_case(acceptance.argmax_rows))
    series("verify_row_stats packed bf16 logits", "row_stats_kernel", logits_case(lambda x: acceptance.verify_row_stats(x, 1.0)))

    def gather(mult):
        hidden = torch.randn(B * mult, n, 4096, device="cuda").to(torch.bfloat16)
        unp = torch.randint(0, n, (B * mult, W, L), device="cuda")
        return (lambda: tree_attention.unpack(hidden, unp)), 2 * B * mult * W * L * 4096 * 2

    series("unpack hidden (B,n,4096) bf16", "gather_rows_kernel", gather)

    def append(mult):
        prev = 1500
        layers = 8 * mult  # (a quarter of the model's layers at x1: the series stays inside 32 layers' memory)
        cache = kv_cache.Cache(B, prev + W * L + 64, layers, H, D, torch.bfloat16, torch.device("cuda"))
        beams = torch.tensor(synthetic_beams(B, W, L), device="cuda")
        tree = tree_attention.build_tree(beams)
        ids = torch.randint(1, V, (B, prev), device="cuda")
        n_tok = [4, 0, 1, 2, 3, 0, 1, 2]
        nt = torch.tensor(n_tok, device="cuda")
        sb = torch.zeros(B, dtype=torch.long, device="cuda")
        cache.rows_in_place = True

        def run():
            cache.set_length(prev + tree.n)
            cache.shift.zero_()
            acceptance.realign(ids, nt, sb, beams, cache, 0, unpacker=tree.unpacker)

        return run, 2 * layers * 2 * H * D * 2 * sum(t + 1 for t in n_tok)

    series("kv_append, 8 layers x", "kv_append_kernel", append)


_bench_lib = None


def bench_library():
    """The bench-only shared object (ml-recurrent-drafter_amd/bench_csrc, built by build_hip.py beside
    the product library but not part of it or of its C ABI)."""
    global _bench_lib
    if _bench_lib is None:
        import ctypes as C

        path = os.path.join(HERE, "ml-recurrent-drafter_amd", "bench_csrc", "libredrafter_bench.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: build it with `python ml-recurrent-drafter_amd/build_hip.py`")
        lib = C.CDLL(path)
        lib.bench_stream_tiles.restype = C.c_int
        lib.bench_stream_tiles.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                           C.c_int, C.c_void_p, C.POINTER(C.c_float)]
        _bench_lib = lib
    return _bench_lib


def case_stream(rows, reps):
    """What the memory system delivers to the attention's access pattern (a K and a V slab per
    (batch row, head), 64-row tiles, one 512-thread workgroup per compute unit) when the tile loop
    does nothing but load, stage and meet at its barrier: bench_stream_tiles.  The slabs are those
    of a cache of 2560 + 128 rows, 690 MB together: more than the 256 MB memory-side cache."""
    import ctypes as C

    slabs, max_len = B * H, 2560 + 128
    k = torch.randn(slabs, max_len, D, device="cuda").to(torch.bfloat16)
    v = torch.randn(slabs, max_len, D, device="cuda").to(torch.bfloat16)
    sink = torch.empty(slabs * 512, dtype=torch.int32, device="cuda")
    lib = bench_library()
    for keys in (640, 1536, 2560):
        tiles = keys // 64
        for depth in (1, 2, 4):
            us = C.c_float(0.0)
            for n in (3, reps):  # warm-up, then the timed launches
                rc = lib.bench_stream_tiles(_hip.ptr(k), _hip.ptr(v), max_len * D * 2, slabs, tiles, depth, _hip.ptr(sink), n,
                                            _hip.stream(), C.byref(us))
                assert rc == 0, rc
            kk = {"stream_tiles_kernel": (1, float(us.value))}
            nbytes = 2 * slabs * tiles * 64 * D * 2
            report(rows, f"stream K/V tiles only, {keys} keys per row, {depth} tile(s) ahead", kk,
                   {"stream_tiles_kernel": nbytes}, {"stream_tiles_kernel": "GB/s"})


def case_rope(rows, reps):
    prev, n = 1500, 181
    cache = kv_cache.Cache(B, prev + n + 8, 1, H, D, torch.bfloat16, torch.device("cuda"))
    torch.manual_seed(2)
    q, k, v = (torch.randn(B, n, H * D, device="cuda").to(torch.bfloat16) for _ in range(3))
    ang = torch.outer(torch.arange(prev + n, device="cuda").float(),
                      1.0 / (10000.0 ** (torch.arange(0, D, 2, device="cuda").float() / D)))
    cos, sin = (torch.cat((f, f), -1).to(torch.bfloat16) for f in (ang.cos(), ang.sin()))
    pos = torch.randint(prev, prev + 5, (B, n), device="cuda")

    def step():
        cache.set_length(prev)
        kv_cache.rope_append(q, k, v, cos, sin, pos, cache.sliced[0])

    kt = timed(step, reps)
    report(rows, f"rope + append prev {prev} n {n}", kt, {"rope_append_kernel": 2 * 3 * B * n * H * D * 2},
           {"rope_append_kernel": "GB/s"})


def case_traffic(rows, reps):
    """For hardware-counter runs (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE): a plain copy of known size
    (256 MiB read, 256 MiB written: the yardstick the counters are scaled by), then the verify
    attention on the decode-bench shape (narrow tree, cached length 525) and on the ragged
    configuration-3 shape.  Nothing is timed here."""
    src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(reps):
        dst.copy_(src)
    for full_len, p_copy in ((525, 0.93), (None, 0.6)):
        lens, n, kv, mask, q, k_, v_ = attention_case(full_len=full_len, p_copy=p_copy)
        prep = attention.prepare(mask, n_heads=H)
        for _ in range(reps):
            attention.masked_attention(q, k_, v_, prep)
        keys = int(lens.sum()) + B * n
        rows.append(dict(case=f"traffic: attention n_q={n} sum keys={keys}", kernel="attn_mfma_kernel", launches_per_call=1,
                         avg_us=0.0, algorithmic_work=2.0 * H * D * 2 * keys + 2.0 * B * H * n * D * 2, achieved=None,
                         unit=None, frac_of_peak=None, note="algorithmic bytes per launch in algorithmic_work"))
    torch.cuda.synchronize()


CASES = dict(rope=case_rope, traffic=case_traffic, tree=case_tree, tree_x64=lambda r, n: case_tree(r, n, 64), attention=case_attention, beam=case_beam,
             logits=case_logits, kv=case_kv, slope=case_slope, stream=case_stream)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--only", default="")
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--json", action="store_true")
    args = ap.parse_args()
    names = [n for n in args.only.split(",") if n] or [n for n in CASES if n not in ("traffic", "slope", "stream")]
    rows = []
    for name in names:
        CASES[name](rows, args.reps)
    if args.json:
        print(json.dumps(rows))
        return
    for r in rows:
        if r["unit"] == "":
            print(r["case"])
            continue
        if r["unit"] is None and r["algorithmic_work"] is not None:
            print(f"{r['case']:<72} {r['kernel']:<22} algorithmic bytes per launch {r['algorithmic_work']:.0f}")
            continue
        rate = "" if r["achieved"] is None else f"{r['achieved']:>9.1f} {r['unit']:<8} {100 * r['frac_of_peak']:6.2f}% of peak"
        print(f"{r['case']:<72} {r['kernel']:<22} x{r['launches_per_call']:<3} {r['avg_us']:>9.2f} us  {rate}")
        if r["note"] and r["kernel"] in ("attn_mfma_kernel", "tree_mask_kernel"):
            print(f"    {r['note']}")


if __name__ == "__main__":
    main()
