import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import __graft_entry__ as entry  # noqa: E402

entry.load_package()  # registers the package directory as `effect_torch_amd`


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950) device")


@pytest.fixture(scope="session")
def et():
    """The product package (``effect-torch_amd``), loaded as ``effect_torch_amd``.

    Loads the in-tree HIP library; builds it only if nothing is built yet."""
    package = entry.load_package()
    from effect_torch_amd import _native
    if not os.path.exists(_native.LIB_PATH):
        entry.build()
    _native.lib()
    return package


@pytest.fixture(scope="session")
def device(et):
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    assert et.is_available(), "a GPU is visible but it is not gfx950"
    return torch.device("cuda:0")
