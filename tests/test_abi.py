"""The C-ABI library loads on a machine without a GPU and exports every symbol the header declares."""
import ctypes
import os
import re

from conftest import ROOT


def _declared():
    names = []
    inc = os.path.join(ROOT, "include")
    for f in sorted(os.listdir(inc)):
        if f.endswith(".h"):
            text = open(os.path.join(inc, f)).read()
            names += re.findall(r"RD_API\s+[\w\s\*]+?\b(rd_\w+)\s*\(", text)
    return names


def test_header_declares_entry_points():
    names = _declared()
    assert "rd_version" in names and "rd_tree_build" in names and len(names) == len(set(names))


def test_library_exports_every_declared_symbol():
    from recurrent_drafting_amd import _hip

    assert os.path.exists(_hip.library_path()), "build with python ml-recurrent-drafter_amd/build_hip.py"
    handle = ctypes.CDLL(_hip.library_path())
    for name in _declared():
        assert hasattr(handle, name), f"{name} declared in include/ but not exported"
    lib = _hip.lib()
    assert lib.rd_version() == _hip.ABI_VERSION
    header = open(os.path.join(ROOT, "include", "redrafter_hip.h")).read()
    assert int(re.search(r"#define RD_ABI_VERSION (\d+)", header).group(1)) == _hip.ABI_VERSION
    # every bound prototype is a declared symbol and vice versa
    assert sorted(_hip._PROTOTYPES) == sorted(_declared())


def test_argument_errors_are_reported_without_a_gpu():
    from recurrent_drafting_amd import _hip

    lib = _hip.lib()
    rc = lib.rd_tree_build(None, 0, 45, 5, None, None, None, None, None, None, None, None, None, None, 0, None)
    assert rc == -1 and b"positive" in lib.rd_last_error()
    rc = lib.rd_tree_build(None, 8, 2000, 5, None, None, None, None, None, None, None, None, None, None, 0, None)
    assert rc == -2
    assert lib.rd_tree_workspace_bytes(8, 45, 5) >= 8 * 45 * 5 * 12


def test_cpu_tensors_are_refused():
    import pytest
    import torch

    from recurrent_drafting_amd import tree_attention

    with pytest.raises(RuntimeError, match="GPU"):
        tree_attention.pack(torch.zeros((1, 2, 3), dtype=torch.long), torch.ones((1, 2), dtype=torch.long))


def test_host_side_checks_of_the_attention_and_probe_entry_points():
    """What the library decides on the host, before any GPU call: which shapes the one-kernel
    RoPE + attention entry point takes, the size of the attention workspace (closed form), and the
    argument errors of entry points whose checks come first (no kernel is launched here)."""
    from recurrent_drafting_amd import _hip

    lib = _hip.lib()
    BF16, F16, F32 = _hip.RD_BF16, _hip.RD_F16, _hip.RD_F32
    ok = lib.rd_rope_verify_attention_eligible
    assert ok(BF16, 32, 128, 168) == 1 and ok(BF16, 128, 128, 256) == 1 and ok(BF16, 1, 128, 1) == 1
    assert ok(F16, 32, 128, 168) == 0 and ok(F32, 32, 128, 168) == 0      # bf16 only
    assert ok(BF16, 32, 64, 168) == 0 and ok(BF16, 32, 256, 168) == 0     # head_dim 128 only
    assert ok(BF16, 129, 128, 168) == 0                                   # the arrival counters are laid out for 128 heads
    assert ok(BF16, 32, 128, 257) == 0 and ok(BF16, 32, 128, 0) == 0      # a prompt goes through the two kernels

    def align(x):
        return (x + 255) // 256 * 256

    for batch, heads, n_q, kv, d in [(8, 32, 168, 2716, 128), (1, 1, 1, 1, 128), (3, 5, 40, 512, 128), (2, 8, 300, 513, 64)]:
        slots = batch * heads * ((kv + 511) // 512)
        assert lib.rd_attention_workspace_bytes(batch, heads, n_q, kv, d) == align(slots * n_q * d * 4) + align(slots * n_q * 2 * 4)
    assert lib.rd_attention_workspace_bytes(0, 32, 168, 2716, 128) == 0

    # rd_verify_attention: sizes, head grouping, head_dim, null pointers
    nulls = [None] * 8
    assert lib.rd_verify_attention(*nulls, BF16, 0, 32, 32, 168, 700, 128, 1.0, None, None, None, 0, 0, None, None) == -1
    assert b"bad sizes" in lib.rd_last_error()
    assert lib.rd_verify_attention(*nulls, BF16, 8, 32, 5, 168, 700, 128, 1.0, None, None, None, 0, 0, None, None) == -1
    assert b"multiple" in lib.rd_last_error()
    assert lib.rd_verify_attention(*nulls, BF16, 8, 32, 32, 168, 700, 512, 1.0, None, None, None, 0, 0, None, None) == -2
    assert lib.rd_verify_attention(*nulls, BF16, 8, 32, 32, 168, 700, 128, 1.0, None, None, None, 0, 0, None, None) == -1
    assert b"null" in lib.rd_last_error()

    # rd_beam_topk_static: what the built-in scratch cannot hold is refused before the scratch is looked up
    args = [None, BF16, 0, 0]
    rest = [32000, None, 50, 0.0, None, 0, None, None, None, None, None, 0, 0, None]
    assert lib.rd_beam_topk_static(*args, 0, 45, *rest) == -1
    assert lib.rd_beam_topk_static(*args, 128, 45, *rest) == -2 and b"workspace" in lib.rd_last_error()  # 5760 rows > 4096
    assert lib.rd_beam_topk_static(*args, 8, 65, *rest) == -2                                            # width > 64
