import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 GPU and the built libnpamd.so")


@pytest.fixture(scope="session")
def oracle_lib():
    import oracle

    oracle.build()
    return oracle


@pytest.fixture(scope="session")
def gpu():
    """Device handle for GPU tests; fails (not skips) if the HIP library is missing on a GPU box."""
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from neuropress_amd import _lib

    _lib.load()  # raises RuntimeError: a GPU box without the kernel library is an error
    return torch.device("cuda:0")
