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
    assert lib.rd_version() >= 100
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
