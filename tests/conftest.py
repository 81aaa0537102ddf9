"""Shared test configuration.

``gpu`` marks the parity tests that need an MI355X; everything else runs on the
CPU.  The oracle under ``oracle/`` is importable from tests only.
"""

import sys
from pathlib import Path

import pytest

REPO_ROOT = Path(__file__).resolve().parent.parent
for path in (REPO_ROOT, REPO_ROOT / "oracle"):
    if str(path) not in sys.path:
        sys.path.insert(0, str(path))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950) GPU")


@pytest.fixture(scope="session")
def gpu_device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")
    from turbo_dllm_amd import chunked_linear_ce_native as native

    native.verify_device(0)  # raises if the HIP library is missing or the arch is wrong
    return torch.device("cuda:0")


@pytest.fixture
def set_panel_budget():
    """Returns a function that bounds the backward's staging panel (bytes) for the
    rest of the test, through the package's context-local option."""
    import contextlib

    from turbo_dllm_amd import options

    with contextlib.ExitStack() as stack:
        yield lambda nbytes: stack.enter_context(options.panel_budget(int(nbytes)))
