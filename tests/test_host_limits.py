"""The compiled-in limits of the entry points are checked on the host and answered with an error
code instead of a launch.  Every call here passes null data pointers: whatever gets past the size
and limit checks stops at the null-pointer check, so nothing is ever launched (runs without a GPU)."""
import pytest

EINVAL, ELIMIT = -1, -2


@pytest.fixture(scope="module")
def lib():
    from recurrent_drafting_amd import _hip

    return _hip.lib()


def _beam_topk(lib, batch=8, width=45, vocab=32000, top_k=50):
    return lib.rd_beam_topk(None, 0, 0, 0, batch, width, vocab, None, top_k, 0.0, None, 0, None, None, None, None,
                            None, 0, None, 0, 0, None)


def test_beam_search_limits(lib):
    assert _beam_topk(lib) == EINVAL and b"null" in lib.rd_last_error()  # the shape itself is fine
    assert _beam_topk(lib, width=64) == EINVAL and _beam_topk(lib, width=65) == ELIMIT
    assert _beam_topk(lib, vocab=65536) == EINVAL and _beam_topk(lib, vocab=65537) == ELIMIT
    assert b"65536" in lib.rd_last_error()
    assert _beam_topk(lib, top_k=512) == EINVAL and _beam_topk(lib, top_k=513) == ELIMIT
    assert _beam_topk(lib, batch=0) == EINVAL and b"bad sizes" in lib.rd_last_error()


def test_beam_init_limits(lib):
    def init(batch=8, width=45, hidden_bytes=8192, state_rows=1, stride=None):
        stride = hidden_bytes if stride is None else stride
        return lib.rd_beam_init(None, stride, None, batch, width, hidden_bytes, -50000.0, None, None, None, 2 * stride,
                                None, state_rows, None)

    assert init() == EINVAL and b"null" in lib.rd_last_error()
    assert init(state_rows=46) == EINVAL and init(state_rows=0) == EINVAL and b"bad sizes" in lib.rd_last_error()
    assert init(batch=65536) == ELIMIT
    # (the alignment rules are checked behind the null pointers: covered on the GPU)


def test_attention_plan_limits(lib):
    def prepare(batch, n_q=168, kv_len=2716, heads=32):
        return lib.rd_attn_prepare(None, 0, 0, batch, n_q, kv_len, heads, 0, None, None, None, None)

    assert prepare(8) == EINVAL and b"null" in lib.rd_last_error()
    assert prepare(2048, kv_len=512) == EINVAL and prepare(2049, kv_len=512) == ELIMIT
    # rows times splits per row (512 keys each) share 32768 work item slots
    assert prepare(1024, kv_len=16384) == EINVAL and prepare(1025, kv_len=16384) == ELIMIT
    assert b"too large" in lib.rd_last_error()
    assert prepare(8, heads=0) == EINVAL and b"bad sizes" in lib.rd_last_error()

    def tree_prepare(batch=8, width=45, length=5, n=168, prev=2548, heads=32):
        return lib.rd_tree_attn_prepare(None, None, None, None, 8, 0, 0, prev, batch, width, length, n, heads, None,
                                        None, None, None, None, None)

    assert tree_prepare() == EINVAL and b"null" in lib.rd_last_error()
    assert tree_prepare(length=65, width=10, n=100) == ELIMIT           # beams of at most 64 tokens
    assert tree_prepare(n=45 * 5 + 1) == ELIMIT                           # more tree nodes than beam slots
    assert tree_prepare(batch=1024, prev=300) == EINVAL and tree_prepare(batch=1025, prev=300) == ELIMIT
    assert tree_prepare(prev=1 << 30) == ELIMIT and b"rd_tree_mask" in lib.rd_last_error()  # points to the two-call route
    assert tree_prepare(prev=-1) == EINVAL


def test_attention_arrival_counter_limit(lib):
    """The MFMA attention takes batch x heads x query tiles arrival counters of a ring of 2^18."""
    def attend(batch, heads, n_q, dtype, generic=0):
        return lib.rd_verify_attention(None, None, None, None, None, None, None, None, dtype, batch, heads, heads,
                                       n_q, 64, 128, 1.0, None, None, None, 0, generic, None, None)

    import torch

    from recurrent_drafting_amd import _hip

    bf16 = _hip.dtype_code(torch.bfloat16)
    assert attend(2048, 128, 256, bf16) == EINVAL and b"null" in lib.rd_last_error()   # exactly the ring
    assert attend(2048, 128, 257, bf16) == ELIMIT and b"arrival counters" in lib.rd_last_error()
    assert attend(2048, 128, 257, bf16, generic=1) == EINVAL                             # the generic kernel has none


def test_tree_limits(lib):
    def build(batch, width, length):
        return lib.rd_tree_build(None, batch, width, length, None, None, None, None, None, None, None, None, None,
                                 None, 0, None)

    assert build(8, 45, 5) == EINVAL and b"null" in lib.rd_last_error()
    assert build(8, 1024, 4) == EINVAL and build(8, 1025, 2) == ELIMIT      # width
    assert build(8, 64, 64) == EINVAL and build(8, 8, 65) == ELIMIT         # length
    assert build(8, 128, 33) == ELIMIT                                      # width * length > 4096
    assert build(65536, 45, 5) == ELIMIT


def test_rope_and_layer_kernel_limits(lib):
    def rope(dtype=0, batch=8, n_new=168, heads=32, kv_heads=32, head_dim=128):
        return lib.rd_rope_append(None, None, None, None, None, None, dtype, batch, n_new, heads, kv_heads, head_dim,
                                  None, None, 4096, None, 0, None, None, None, None, None, 0, 2773, None, None, None)

    assert rope() == EINVAL and b"null" in lib.rd_last_error()
    assert rope(head_dim=120) == ELIMIT and b"multiple of 16" in lib.rd_last_error()   # bf16: two 8-element vectors
    assert rope(dtype=2, head_dim=24) == EINVAL and rope(dtype=2, head_dim=20) == ELIMIT  # float32: two 4-element vectors
    assert rope(dtype=7) == EINVAL and b"dtype" in lib.rd_last_error()
    assert rope(batch=65536) == ELIMIT

    def norm(dtype, cols, rows=1448):
        return lib.rd_add_rms_norm(None, 0, None, 0, None, None, 0, None, 0, dtype, rows, cols, 1e-6, None)

    assert norm(0, 4096) == EINVAL and b"null" in lib.rd_last_error()
    assert norm(0, 16384) == EINVAL and norm(0, 16392) == ELIMIT      # 16-bit rows of at most 16384 columns
    assert norm(2, 8192) == EINVAL and norm(2, 8196) == ELIMIT        # float32 rows of at most 8192
    assert norm(0, 4100) == ELIMIT and norm(2, 4098) == ELIMIT        # whole 16-byte vectors only
    assert norm(0, 4096, rows=0) == EINVAL and b"bad sizes" in lib.rd_last_error()


def test_verification_and_acceptance_limits(lib):
    def stats(vocab=32000, top_k=50, rows=1448):
        return lib.rd_verify_row_stats(None, 0, vocab, rows, vocab, top_k, -1e4, 1.0, None, 0, None)

    assert stats() == EINVAL and b"null" in lib.rd_last_error()
    assert stats(vocab=65536) == EINVAL and stats(vocab=65537) == ELIMIT
    assert stats(top_k=512) == EINVAL and stats(top_k=513) == ELIMIT
    assert stats(rows=0) == EINVAL

    def greedy(batch=8, width=45, length=5):
        return lib.rd_accept_greedy(None, None, 0, None, batch, width, length, None, None, None, None, None)

    assert greedy() == EINVAL and b"null" in lib.rd_last_error()
    assert greedy(width=65535) == EINVAL and greedy(width=65536) == ELIMIT
    assert greedy(length=32767) == EINVAL and greedy(length=32768) == ELIMIT
    assert greedy(batch=0) == EINVAL

    def sample(batch=8, width=45, length=5, vocab=32000):
        return lib.rd_accept_sample(None, None, None, None, 0, None, None, 0, None, 1.0, None, None, None, batch, width,
                                    length, vocab, None, None, None)

    assert sample() == EINVAL and b"null" in lib.rd_last_error()
    assert sample(length=1) == EINVAL and b"null" not in lib.rd_last_error()   # nothing drafted: nothing to accept
    assert sample(width=65536) == ELIMIT

    def argmax(rows=1448, vocab=32000, stride=32000):
        return lib.rd_argmax_rows(None, 0, rows, vocab, stride, None, None, None)

    assert argmax() == EINVAL and b"null" in lib.rd_last_error()
    assert argmax(stride=31999) == EINVAL and b"null" not in lib.rd_last_error()
    assert argmax(rows=1 << 31) == ELIMIT


def test_mask_and_row_movement_limits(lib):
    def causal(batch=8, kv_len=500, query_len=500):
        return lib.rd_causal_mask(None, 8, kv_len, batch, kv_len, query_len, None, None)

    assert causal() == EINVAL and b"null" in lib.rd_last_error()
    assert causal(query_len=501) == EINVAL and b"null" not in lib.rd_last_error()   # more queries than keys
    assert causal(batch=65536) == ELIMIT

    def tree_mask(batch=8, width=45, length=5, prev=2548):
        return lib.rd_tree_mask(None, None, None, None, 8, prev, 0, prev, batch, width, length, None, None)

    assert tree_mask() == EINVAL and b"null" in lib.rd_last_error()
    assert tree_mask(length=65, width=8) == ELIMIT and tree_mask(width=1024, length=5) == ELIMIT
    assert tree_mask(batch=65536) == ELIMIT
    assert tree_mask(prev=-1) == EINVAL

    def unpack(batch=8, n_out=225, n_src=168, row_bytes=8192):
        return lib.rd_unpack_rows(None, n_src * row_bytes, row_bytes, None, n_out, batch, n_out, n_src, None,
                                  n_out * row_bytes, row_bytes, None, None)

    assert unpack() == EINVAL and b"null" in lib.rd_last_error()
    assert unpack(batch=65536) == ELIMIT
    assert unpack(row_bytes=0) == EINVAL and b"bad sizes" in lib.rd_last_error()

    def silu_mul(dtype=0, cols=11008, rows=1448):
        return lib.rd_silu_mul(None, None, 2 * cols, None, cols, dtype, rows, cols, None)

    assert silu_mul() == EINVAL and b"null" in lib.rd_last_error()
    assert silu_mul(cols=11004) == ELIMIT and silu_mul(dtype=2, cols=11006) == ELIMIT   # whole 16-byte vectors
    assert silu_mul(dtype=2, cols=11004) == EINVAL
    assert silu_mul(dtype=5) == EINVAL and b"dtype" in lib.rd_last_error()
