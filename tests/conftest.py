import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden():
    import json
    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def hip():
    """The ctypes binding of the native library; importing it fails if the library is not built."""
    import __graft_entry__ as entry
    return entry.load_package().itexhip


@pytest.fixture(scope="session")
def dev():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def _tile_shape_choice_restored():
    """A test that forced a tile shape (hip.force_tile_shape) does not leave it forced for the next one."""
    yield
    pkg = sys.modules.get("itex_amd")
    if pkg is not None and hasattr(pkg, "itexhip"):
        pkg.itexhip.force_tile_shape(-1, -1)
