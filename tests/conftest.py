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


def pytest_terminal_summary(terminalreporter):
    """Margins of the GPU parity tests: per test, the worst max-norm error and the worst per-element error scaled by
    rms(want) over all comparisons it made."""
    mod = sys.modules.get("tests.test_parity_gpu") or sys.modules.get("test_parity_gpu")
    margins = getattr(mod, "MARGINS", None)
    if not margins:
        return
    terminalreporter.write_line("parity margins: test, max|d|/max|want|, max|d|/rms(want)")
    for name, (a, b) in sorted(margins.items(), key=lambda kv: -kv[1][1])[:25]:
        terminalreporter.write_line(f"  {name:64s} {a:9.2e} {b:9.2e}")
    try:
        out = os.path.join(ROOT, "gpurun_out")
        os.makedirs(out, exist_ok=True)
        with open(os.path.join(out, "parity_margins.json"), "w") as f:
            json.dump({k: {"max_norm": v[0], "rms_scaled": v[1]} for k, v in margins.items()}, f, indent=1)
    except OSError:
        pass
