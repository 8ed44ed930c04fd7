"""rd_beam_topk_static, the entry point that allocates nothing: through the C ABI, against
rd_beam_topk (the entry point it is a variant of) on the same inputs, bit for bit -- two calls in
a row, the second with a smaller input (the built-in scratch keeps the first call's contents) --
and its size limit."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _call(entry, logits, lpb, beams, want_log_probs, workspace):
    """One beam-search iteration through `entry`; workspace None selects the static form."""
    from recurrent_drafting_amd import _hip

    B, W, V = logits.shape
    t = beams.shape[2]
    dev = logits.device
    x = logits.reshape(B * W, V)
    new_lpb = torch.empty((B, W), dtype=torch.float32, device=dev)
    tok = torch.empty((B, W), dtype=torch.long, device=dev)
    par = torch.empty((B, W), dtype=torch.long, device=dev)
    new_beams = torch.empty((B, W, t + 1), dtype=torch.long, device=dev)
    logp = torch.empty((B, W, V), dtype=torch.float32, device=dev) if want_log_probs else None
    head = (_hip.ptr(x), _hip.dtype_code(x.dtype), x.stride(0), 0, B, W, V, _hip.ptr(lpb), 50, -50000.0,
            _hip.ptr(beams), t, _hip.ptr(new_lpb), _hip.ptr(tok), _hip.ptr(par), _hip.ptr(new_beams),
            _hip.ptr(logp), V)
    lib = _hip.lib()
    # device memory the driver has free, right around the call alone (the outputs above were
    # allocated before; torch's own counters would not see a hipMalloc made inside the library)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    if workspace is None:
        rc = lib.rd_beam_topk_static(*head, 0, _hip.stream())
    else:
        rc = lib.rd_beam_topk(*head, _hip.ptr(workspace), workspace.numel(), 0, _hip.stream())
    torch.cuda.synchronize()
    _call.freed_or_taken = free_before - torch.cuda.mem_get_info()[0]
    return rc, (new_lpb, tok, par, new_beams, logp)


def _inputs(B, W, V, t, dtype, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    logits = (torch.randn(B, W, V, device="cuda", generator=g) * 1.7).to(dtype)
    lpb = -torch.rand(B, W, device="cuda", generator=g) * 4
    beams = torch.randint(0, V, (B, W, t), device="cuda", generator=g)
    return logits, lpb, beams


def test_static_entry_point_matches_the_workspace_form_on_two_calls_in_a_row():
    from recurrent_drafting_amd import _hip

    lib = _hip.lib()
    # the larger call first: the smaller one then runs over scratch that still holds its lists
    for (B, W, V, t, dtype, want), seed in zip(
            [(8, 45, 32000, 3, torch.bfloat16, False), (3, 7, 4000, 2, torch.float32, True)], (11, 12)):
        logits, lpb, beams = _inputs(B, W, V, t, dtype, seed)
        ws = torch.empty(lib.rd_beam_topk_workspace_bytes(B, W), dtype=torch.uint8, device="cuda")
        rc, want_out = _call("workspace", logits, lpb, beams, want, ws)
        assert rc == 0
        rc, _ = _call("static", logits, lpb, beams, want, None)  # (the first call looks up the scratch's address)
        assert rc == 0, lib.rd_last_error().decode()
        deltas = []
        for _ in range(3):
            rc, got = _call("static", logits, lpb, beams, want, None)
            assert rc == 0, lib.rd_last_error().decode()
            deltas.append(_call.freed_or_taken)
        # an allocation made by the entry point would show in every call (the driver's own bookkeeping
        # may move the figure once in a while)
        assert min(deltas) <= 0, f"the driver's free device memory shrank across every call: {deltas}"
        for g, w in zip(got, want_out):
            assert (g is None) == (w is None)
            if g is not None:
                assert torch.equal(g, w)


def test_static_entry_point_rejects_what_its_scratch_cannot_hold():
    from recurrent_drafting_amd import _hip

    lib = _hip.lib()
    B, W, V = 70, 64, 64  # 4480 beam rows > 4096
    logits, lpb, beams = _inputs(B, W, V, 1, torch.float32, 1)
    rc, _ = _call("static", logits, lpb, beams, False, None)
    assert rc == -2  # RD_ELIMIT
    assert b"built-in scratch" in lib.rd_last_error()
    # the workspace form takes the same call
    ws = torch.empty(lib.rd_beam_topk_workspace_bytes(B, W), dtype=torch.uint8, device="cuda")
    rc, _ = _call("workspace", logits, lpb, beams, False, ws)
    assert rc == 0
