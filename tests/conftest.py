import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def ref():
    """The CPU oracle (oracle/liboxq_oracle.so), built on demand."""
    import oracle
    oracle.load()
    return oracle


@pytest.fixture(scope="session")
def hip():
    """The HIP library through its Python binding; fails loudly if it is not built."""
    import torch
    from oxillama_amd import quant
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible")
    quant.init(0)
    return quant
