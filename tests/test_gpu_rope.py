"""rd_rope_append (rotation of q/k + in-place KV append) against the torch restatement of the
reference's op sequence (modeling_llama.py:87-110, 148-159), bit for bit in every dtype."""

import numpy as np
import pytest
import torch

from oracle import torch_path

pytestmark = pytest.mark.gpu


def _case(batch, n_new, heads, kv_heads, dim, prev, max_len, dtype, seed, fused_rows=False):
    from recurrent_drafting_amd import kv_cache

    g = torch.Generator().manual_seed(seed)
    hidden = (heads + 2 * kv_heads) * dim
    if fused_rows:  # q, k, v are column slices of one projection output: strided token rows
        qkv = torch.randn(batch, n_new, hidden, generator=g).to(dtype)
        q, k, v = qkv[..., : heads * dim], qkv[..., heads * dim : (heads + kv_heads) * dim], qkv[..., (heads + kv_heads) * dim :]
    else:
        q = torch.randn(batch, n_new, heads * dim, generator=g).to(dtype)
        k = torch.randn(batch, n_new, kv_heads * dim, generator=g).to(dtype)
        v = torch.randn(batch, n_new, kv_heads * dim, generator=g).to(dtype)
    position_ids = torch.randint(0, prev + n_new, (batch, n_new), generator=g)
    old = torch.randn(2, batch, kv_heads, max_len, dim, generator=g).to(dtype)
    cos, sin = torch_path._rope_tables(dim, 10000.0, prev + n_new, "cpu", dtype)

    # restatement on the CPU: rotate, then write rows [prev, prev + n_new)
    qh = q.reshape(batch, n_new, heads, dim).transpose(1, 2)
    kh = k.reshape(batch, n_new, kv_heads, dim).transpose(1, 2)
    vh = v.reshape(batch, n_new, kv_heads, dim).transpose(1, 2)
    c, s = cos[position_ids].unsqueeze(1), sin[position_ids].unsqueeze(1)
    want_q, want_k = torch_path._rope(qh, c, s), torch_path._rope(kh, c, s)
    want_cache = old.clone()
    want_cache[0, :, :, prev : prev + n_new] = want_k
    want_cache[1, :, :, prev : prev + n_new] = vh

    cache = kv_cache.Cache(batch, max_len, 3, kv_heads, dim, dtype, torch.device("cuda"))
    layer = 1
    cache._cache[layer] = old.cuda()
    cache.sliced[layer][0].length = cache.sliced[layer][1].length = prev
    if fused_rows:
        qkv_d = qkv.cuda()
        qd, kd, vd = (qkv_d[..., : heads * dim], qkv_d[..., heads * dim : (heads + kv_heads) * dim],
                      qkv_d[..., (heads + kv_heads) * dim :])
    else:
        qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    got_q, keys, values = kv_cache.rope_append(qd, kd, vd, cos.cuda(), sin.cuda(), position_ids.cuda(),
                                               cache.sliced[layer])
    assert cache.sliced[layer][0].length == prev + n_new == cache.sliced[layer][1].length
    assert got_q.shape == (batch, heads, n_new, dim) and keys.shape == (batch, kv_heads, prev + n_new, dim)
    assert torch.equal(got_q.cpu(), want_q)
    assert torch.equal(cache._cache[layer].cpu(), want_cache)  # rows outside the append untouched
    assert torch.equal(keys.cpu(), want_cache[0, :, :, : prev + n_new])
    assert torch.equal(values.cpu(), want_cache[1, :, :, : prev + n_new])
    assert not cache._cache[0].any() and not cache._cache[2].any()  # other layers untouched


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 1, 2, 2, 16, 0, 4), (2, 7, 4, 4, 32, 5, 16), (3, 5, 8, 2, 64, 9, 20),
                                   (2, 33, 32, 32, 128, 100, 160)])
def test_matches_restatement(shape, dtype):
    _case(*shape, dtype, seed=sum(shape))


def test_strided_token_rows():
    _case(2, 6, 4, 2, 32, 3, 12, torch.bfloat16, seed=5, fused_rows=True)


def test_benchmark_shape_bf16():
    _case(8, 181, 32, 32, 128, 1500, 1500 + 225 + 8, torch.bfloat16, seed=11)


def test_position_zero_is_identity_and_rotation_keeps_pair_norms():
    from recurrent_drafting_amd import kv_cache

    batch, n_new, heads, dim = 2, 9, 4, 64
    g = torch.Generator().manual_seed(3)
    q = torch.randn(batch, n_new, heads * dim, generator=g)
    k = torch.randn(batch, n_new, heads * dim, generator=g)
    v = torch.randn(batch, n_new, heads * dim, generator=g)
    cos, sin = torch_path._rope_tables(dim, 10000.0, 64, "cpu", torch.float32)
    for positions in (torch.zeros(batch, n_new, dtype=torch.long), torch.randint(1, 64, (batch, n_new), generator=g)):
        cache = kv_cache.Cache(batch, n_new, 1, heads, dim, torch.float32, torch.device("cuda"))
        got_q, keys, _ = kv_cache.rope_append(q.cuda(), k.cuda(), v.cuda(), cos.cuda(), sin.cuda(), positions.cuda(),
                                              cache.sliced[0])
        q4 = q.view(batch, n_new, heads, dim).transpose(1, 2)
        if not positions.any():
            assert torch.equal(got_q.cpu(), q4)
            assert torch.equal(keys.cpu(), k.view(batch, n_new, heads, dim).transpose(1, 2))
        pair = lambda x: (x[..., : dim // 2].double() ** 2 + x[..., dim // 2 :].double() ** 2)
        np.testing.assert_allclose(pair(got_q.cpu()).numpy(), pair(q4).numpy(), rtol=1e-5, atol=1e-6)


def test_argument_errors():
    from recurrent_drafting_amd import kv_cache

    cache = kv_cache.Cache(1, 4, 1, 2, 16, torch.float32, torch.device("cuda"))
    cos, sin = torch_path._rope_tables(16, 10000.0, 8, "cpu", torch.float32)
    q = torch.zeros(1, 5, 32, device="cuda")
    with pytest.raises(AssertionError):  # 5 new rows do not fit max_length 4
        kv_cache.rope_append(q, q.clone(), q.clone(), cos.cuda(), sin.cuda(),
                             torch.zeros(1, 5, dtype=torch.long, device="cuda"), cache.sliced[0])
