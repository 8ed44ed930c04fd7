import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_PARENT = os.path.join(ROOT, "ml-recurrent-drafter_amd")
for p in (ROOT, PKG_PARENT):
    if p not in sys.path:
        sys.path.insert(0, p)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")
    # the suite speaks for the library built from this tree, never for another build
    override = os.environ.get("RD_HIP_LIBRARY")
    in_tree = os.path.join(PKG_PARENT, "recurrent_drafting_amd", "libredrafter_hip.so")
    if override and os.path.realpath(override) != os.path.realpath(in_tree):
        raise pytest.UsageError(
            f"RD_HIP_LIBRARY={override} points the package at another build of the library; "
            "unset it to run the tests")


@pytest.fixture(scope="session")
def literals():
    with open(os.path.join(GOLDEN, "reference_literals.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def ref_vectors():
    with open(os.path.join(GOLDEN, "reference_vectors.json")) as f:
        return json.load(f)
