import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950); run with -m gpu")


@pytest.fixture(scope="session")
def kats():
    with open(os.path.join(ROOT, "tests", "golden", "reference_kats.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (numpy twin + C library).  Test infrastructure only."""
    from oracle import ggml_oracle
    ggml_oracle.lib()  # builds libggml_oracle.so with gcc if it is missing
    return ggml_oracle


@pytest.fixture(scope="session")
def gpu():
    """torch + the initialised HIP library; fails (not skips) if either is unusable."""
    import torch
    assert torch.cuda.is_available(), "GPU tests need a visible MI355X"
    from gomlx_amd import _lib
    _lib.init(0)
    return torch
