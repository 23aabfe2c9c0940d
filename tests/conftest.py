import sys
from pathlib import Path

import pytest

REPO = Path(__file__).resolve().parent.parent
if str(REPO) not in sys.path:
    sys.path.insert(0, str(REPO))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box only)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (built on first use with gcc; test infrastructure only)."""
    import oracle as _oracle
    _oracle.lib()
    return _oracle


@pytest.fixture(scope="session")
def ops():
    """The product path: torch device tensors -> C ABI -> HIP kernels.  No fallback."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from anygpu_amd import ops as _ops, capi
    capi.load()
    return _ops
