import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def hip_lib():
    """The loaded C-ABI library; built first only if no built library is present."""
    from quick_ssm_amd import _lib

    if not _lib.is_built():
        from quick_ssm_amd import build as builder

        builder.build(verbose=False)
    return _lib.load()


@pytest.fixture(scope="session")
def gpu(hip_lib):
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda", 0)
