import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def rt():
    """The product runtime on cuda:0; GPU tests only."""
    import torch

    from docc_amd import runtime

    assert torch.cuda.is_available(), "GPU test selected but no GPU is visible"
    runtime.init(0)
    return runtime
