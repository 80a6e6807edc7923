import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def kvm():
    """The ctypes binding of the C ABI (loads the in-tree libkvmove.so)."""
    from distserve_amd import cabi

    return cabi


@pytest.fixture(scope="session")
def kvm_explore():
    """The same binding over the exploration build (-DKVM_EXPLORE: every kernel flavour and
    the knobs that select them).  A library of its own: its registry and options are not the
    product's."""
    from distserve_amd import cabi

    path = os.path.join(ROOT, "tests", "lib_explore", "libkvmove.so")
    assert os.path.exists(path), "tests/lib_explore/libkvmove.so is not built: python distserve_amd/csrc/build.py"
    return cabi.Binding(path)


@pytest.fixture()
def fresh_registry(kvm):
    kvm.reset()
    yield kvm
    kvm.reset()
