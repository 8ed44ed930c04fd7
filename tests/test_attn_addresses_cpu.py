"""Every memory address of attn_mfma_kernel, checked on the host before the kernel runs anywhere.

The kernel forms its addresses with the integer functions of csrc/attn_addr.h and cuts rows into
work items with those of csrc/attn_plan.h.  tests/attn_address_check.cpp (built here with g++; no
GPU, no HIP) calls the same functions for every (work item, head, query tile, thread, tile) of a
launch and asserts that each address lies inside the tensor it belongs to: Q, output, the cache
rows of the span of attended keys (never a row outside it: such rows may hold anything), mask
words, partial results and arrival counters of split rows, the new rows of the fused rotation,
and every LDS offset (inside the allocation, aligned, staging writes disjoint, fragment reads only
of bytes that were staged).  For each launch every item size that the plan's search can choose is
walked, not only the one it would choose.

The launches are the shapes of the GPU tests of the attention (tests/test_gpu_attention.py), of the
decode loop with packed query rows and cache rows kept in place, of the prefill, and of the
benchmark configurations 3, 4 and 5.
"""
import ctypes as C
import os
import subprocess
import tempfile

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "ml-recurrent-drafter_amd", "csrc")
D = 128


class Launch(C.Structure):
    _fields_ = [
        ("B", C.c_int), ("H", C.c_int), ("Hkv", C.c_int), ("n_q", C.c_int), ("kv_len", C.c_int),
        ("n_heads_for_plan", C.c_int), ("n_cu", C.c_int),
        ("q_sb", C.c_int64), ("q_sh", C.c_int64), ("q_ss", C.c_int64), ("q_elems", C.c_int64),
        ("k_sb", C.c_int64), ("k_sh", C.c_int64), ("k_ss", C.c_int64),
        ("slab_rows", C.c_int64), ("kv_elems", C.c_int64),
        ("o_sb", C.c_int64), ("o_sh", C.c_int64), ("o_ss", C.c_int64), ("o_elems", C.c_int64),
        ("row_start", C.POINTER(C.c_int32)), ("key_min", C.POINTER(C.c_int32)),
        ("key_end", C.POINTER(C.c_int32)), ("kv_shift", C.POINTER(C.c_int32)),
        ("forced_chunk", C.c_int), ("rope", C.c_int),
        ("kn_sb", C.c_int64), ("kn_st", C.c_int64), ("kn_elems", C.c_int64),
        ("pos_sb", C.c_int64), ("pos_elems", C.c_int64), ("max_len", C.c_int64), ("table_rows", C.c_int64),
    ]


class Stats(C.Structure):
    _fields_ = [(n, C.c_longlong) for n in ("items", "workgroups", "tile_loads", "q_loads", "stores",
                                            "partial_rows", "new_rows", "chunks_tried")]


@pytest.fixture(scope="module")
def checker():
    out = os.path.join(tempfile.mkdtemp(prefix="attn_addr_"), "libattn_address_check.so")
    cmd = ["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-I", CSRC,
           os.path.join(ROOT, "tests", "attn_address_check.cpp"), "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    lib = C.CDLL(out)
    lib.attn_check_launch.argtypes = [C.POINTER(Launch), C.POINTER(Stats), C.c_char_p, C.c_int]
    lib.attn_check_lds.argtypes = [C.c_char_p, C.c_int]
    lib.attn_check_plan_sweep.argtypes = [C.c_int, C.c_char_p, C.c_int]
    return lib


def _i32(values):
    a = np.ascontiguousarray(values, dtype=np.int32)
    return a, a.ctypes.data_as(C.POINTER(C.c_int32))


def make(B, H, Hkv, n_q, prev, key_min, counts, plan_heads, *, slab_rows=None, packed=False, shift=None,
         rope=False, forced_chunk=0, n_cu=256, rows_rounded=32):
    """A launch as the package makes it: q/out (B, n_q, H, D) shown as (B, H, n_q, D) (or, packed,
    (rows, H, D) of the slots that exist, rounded up to 32 rows), K/V two slabs of one cache
    (B, Hkv, slab_rows, D).  key_min[b]: first attended key; counts[b]: tree slots of row b that exist
    (its last attended key is prev + counts[b] - 1)."""
    kv_len = prev + n_q
    slab_rows = slab_rows or kv_len
    keep = []
    L = Launch()
    L.B, L.H, L.Hkv, L.n_q, L.kv_len = B, H, Hkv, n_q, kv_len
    L.n_heads_for_plan, L.n_cu, L.forced_chunk = plan_heads, n_cu, forced_chunk
    if packed:
        total = int(np.sum(counts))
        rows = (total + rows_rounded - 1) // rows_rounded * rows_rounded
        L.q_sb, L.q_sh, L.q_ss, L.q_elems = 0, D, H * D, rows * H * D
        L.o_sb, L.o_sh, L.o_ss, L.o_elems = 0, D, H * D, rows * H * D
        a, p = _i32(np.concatenate([[0], np.cumsum(counts)]))
        keep.append(a)
        L.row_start = p
    else:
        L.q_sb, L.q_sh, L.q_ss, L.q_elems = n_q * H * D, D, H * D, B * n_q * H * D
        L.o_sb, L.o_sh, L.o_ss, L.o_elems = n_q * H * D, D, H * D, B * n_q * H * D
    L.k_sb, L.k_sh, L.k_ss = Hkv * slab_rows * D, slab_rows * D, D
    L.slab_rows, L.kv_elems = slab_rows, B * Hkv * slab_rows * D
    for name, vals in (("key_min", key_min), ("key_end", [prev + c for c in counts])):
        a, p = _i32(vals)
        keep.append(a)
        setattr(L, name, p)
    if shift is not None:
        a, p = _i32(shift)
        keep.append(a)
        L.kv_shift = p
    if rope:
        L.rope = 1
        L.max_len = slab_rows
        L.table_rows = kv_len + 8
        if packed:
            L.kn_sb, L.kn_st, L.kn_elems = 0, Hkv * D, L.q_elems // H * Hkv
        else:
            L.kn_sb, L.kn_st, L.kn_elems = n_q * Hkv * D, Hkv * D, B * n_q * Hkv * D
        L.pos_sb, L.pos_elems = n_q, B * n_q
    L._keep = keep
    return L


def run(checker, launch):
    msg = C.create_string_buffer(600)
    st = Stats()
    rc = checker.attn_check_launch(C.byref(launch), C.byref(st), msg, len(msg))
    return rc, msg.value.decode(), st


def ok(checker, launch):
    rc, msg, st = run(checker, launch)
    assert rc == 0, msg
    assert st.tile_loads > 0 and st.stores > 0 and st.workgroups > 0
    return st


def test_lds_offsets_of_every_thread_tile_and_fragment(checker):
    msg = C.create_string_buffer(600)
    assert checker.attn_check_lds(msg, len(msg)) == 0, msg.value.decode()


def test_plan_items_are_never_empty_and_tile_the_row(checker):
    """Every (live keys, item size): the items of a row hold keys, start on tile boundaries and cover
    [begin, end) without gap or overlap -- also where the tile rounding of the share needs fewer items
    than first counted (5121 keys at 512 per item: ten counted, nine of 576 cover the row)."""
    msg = C.create_string_buffer(600)
    assert checker.attn_check_plan_sweep(9000, msg, len(msg)) == 0, msg.value.decode()


# the shapes of tests/test_gpu_attention.py --------------------------------------------------------
def test_shapes_of_the_span_test(checker):
    prev_lens, n_q = [700, 333, 1, 640], 33
    prev = max(prev_lens)
    counts = [n_q - 5, n_q, n_q - 17, n_q - 1]
    for heads in (3, 1):
        st = ok(checker, make(4, 3, 3, n_q, prev, [prev - p for p in prev_lens], counts, heads, slab_rows=prev + n_q + 90))
    assert st.partial_rows > 0  # with one head for the plan the long rows are split


@pytest.mark.parametrize("B,H,Hkv,n_q,prev_lens", [
    (1, 1, 1, 5, [40]), (2, 2, 2, 30, [100, 37]), (2, 2, 2, 90, [300, 150]), (2, 4, 2, 170, [700, 1300]),
    (1, 2, 2, 300, [64]), (3, 2, 2, 50, [2000, 5, 900])])
def test_shapes_of_the_tree_cases(checker, B, H, Hkv, n_q, prev_lens):
    prev = max(prev_lens)
    for heads in (H, 4096, 1):
        ok(checker, make(B, H, Hkv, n_q, prev, [prev - p for p in prev_lens], [n_q] * B, heads, slab_rows=prev + n_q + 37))


@pytest.mark.parametrize("n_q", [1, 31, 32, 33, 64, 96, 97, 127, 128, 129, 150, 160, 161, 192, 193, 256, 257, 320, 513])
def test_every_wave_layout_and_row_count(checker, n_q):
    for prev in (70, 200):
        ok(checker, make(2, 2, 2, n_q, prev, [prev // 2, 0], [n_q, max(1, n_q // 2)], 2, slab_rows=prev + n_q + 37))


@pytest.mark.parametrize("n_q,prev", [(300, 1500), (150, 2100), (96, 1300), (150, 1750)])
def test_split_rows(checker, n_q, prev):
    for heads in (2, 1, 6):
        st = ok(checker, make(3, 6, 6, n_q, prev, [0, prev - 200, 17], [n_q] * 3, heads))
        assert st.partial_rows > 0


# decode loop and benchmark configurations -----------------------------------------------------------
def _ragged(rng, B, lo, hi):
    return [int(x) for x in rng.integers(lo, hi + 1, size=B)]


def test_configuration_3_ragged_cached_lengths(checker):
    rng = np.random.default_rng(123)
    B, H, n_q = 8, 32, 168
    lens = _ragged(rng, B, 500, 2548)
    prev = max(lens)
    counts = _ragged(rng, B, 100, n_q)
    counts[0] = n_q
    ok(checker, make(B, H, H, n_q, prev, [prev - n for n in lens], counts, H, slab_rows=prev + n_q + 64))


@pytest.mark.parametrize("prev", [500, 761, 1500, 2548])
def test_configuration_4_decode_step_packed_rows_cache_rows_in_place(checker, prev):
    """Batch 8 x 32 heads, beam 45 x 5: packed query rows, ragged left padding, and cache rows kept in
    place (column c of row b lives in cache row c - shift[b]; a row's cache rows begin where its prompt began)."""
    rng = np.random.default_rng(prev)
    B, H = 8, 32
    counts = _ragged(rng, B, 90, 125)
    n_q = max(counts)
    pads = [0] + _ragged(rng, B - 1, 0, min(400, prev - 1))
    # a row whose padding grew by s since its prompt was stored sits s rows to the left of its columns
    shift = [int(x) for x in rng.integers(-3, 4, size=B)]
    shift = [min(s, p) for s, p in zip(shift, pads)]  # (its first live column must stay inside the slab)
    slab_rows = 500 + 2048 + 225 + 400
    for rope in (False, True):
        ok(checker, make(B, H, H, n_q, prev, pads, counts, H, slab_rows=slab_rows, packed=True, shift=shift, rope=rope))


def test_configuration_5_batch_16_forty_heads_beam_64(checker):
    rng = np.random.default_rng(5)
    B, H = 16, 40
    counts = _ragged(rng, B, 150, 320)
    n_q = max(counts)
    for prev in (256, 1200):
        pads = _ragged(rng, B, 0, 100)
        ok(checker, make(B, H, H, n_q, prev, pads, counts, H, slab_rows=256 + 2048 + 320 + 100, packed=True,
                         shift=[0] * B))


@pytest.mark.parametrize("B,H,S,pads", [(4, 4, 300, [0, 131, 3, 250]), (8, 32, 500, [0] * 8),
                                        (8, 32, 1500, [0, 700, 13, 250, 999, 64, 1, 420])])
def test_prefill_square_causal_mask_with_left_padding(checker, B, H, S, pads):
    # queries are the whole prompt: n_q = kv_len = S, no cached keys in front
    ok(checker, make(B, H, H, S, 0, pads, [S] * B, H, slab_rows=S + 45 * 5 + 64))


@pytest.mark.parametrize("B,H,Hkv,n_new,prev_lens,shifted,packed", [
    (2, 4, 4, 23, [200, 131], False, False), (3, 4, 2, 37, [300, 17, 150], True, False),
    (3, 8, 2, 40, [1, 64, 129], True, True), (2, 4, 4, 130, [500, 420], True, True),
    (2, 2, 2, 256, [90, 64], False, False), (4, 32, 32, 26, [2500, 300, 1800, 64], True, True)])
def test_shapes_of_the_fused_rotation_cases(checker, B, H, Hkv, n_new, prev_lens, shifted, packed):
    prev = max(prev_lens)
    rng = np.random.default_rng(n_new)
    counts = [n_new] + (_ragged(rng, B - 1, max(1, n_new // 2), n_new) if packed else [n_new] * (B - 1))
    shift = [prev - p if shifted else 0 for p in prev_lens]
    st = ok(checker, make(B, H, Hkv, n_new, prev, [prev - p for p in prev_lens], counts, H, slab_rows=prev + n_new + 7,
                          packed=packed, shift=shift, rope=True))
    assert st.new_rows > 0


def test_fused_rotation_on_a_slab_that_ends_behind_the_new_tokens(checker):
    prev_lens, n_new = [100, 40], 20
    prev = max(prev_lens)
    ok(checker, make(2, 4, 4, n_new, prev, [prev - p for p in prev_lens], [n_new] * 2, 4, slab_rows=120,
                     shift=[prev - p for p in prev_lens], rope=True))


# the checker itself: launches that must NOT pass ------------------------------------------------------
def test_checker_refuses_a_slab_shorter_than_the_span(checker):
    rc, msg, _ = run(checker, make(2, 2, 2, 40, 700, [0, 100], [40, 40], 2, slab_rows=700))
    assert rc != 0 and "cache row" in msg


def test_checker_refuses_a_shift_that_leaves_the_slab(checker):
    rc, msg, _ = run(checker, make(2, 2, 2, 40, 700, [0, 100], [40, 40], 2, slab_rows=800, shift=[5, 0]))
    assert rc != 0 and "cache row" in msg


def test_checker_refuses_too_few_query_rows(checker):
    launch = make(2, 2, 2, 40, 100, [0, 0], [40, 40], 2)
    launch.q_elems -= 8
    rc, msg, _ = run(checker, launch)
    assert rc != 0 and "Q element" in msg
    launch = make(2, 2, 2, 40, 100, [0, 0], [40, 30], 2, packed=True)
    launch.o_elems = 69 * 2 * D  # the packed rows that exist are 70
    rc, msg, _ = run(checker, launch)
    assert rc != 0 and "output element" in msg
