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


@pytest.fixture
def tuning():
    """Setter for the launch-shape knobs of oxq_tuning.h; every knob a test touched is back at its
    default (0; fusion: 1) when the test ends, pass or fail."""
    from oxillama_amd import capi
    lib = capi.load()
    touched = set()

    def set_knob(name, value):
        touched.add(name)
        assert getattr(lib, "oxq_set_" + name)(value) == capi.OK

    yield set_knob
    for name in touched:
        getattr(lib, "oxq_set_" + name)(1 if name == "ffn_fusion" else 0)


@pytest.fixture(scope="session")
def hip():
    """The HIP library through its Python binding; fails loudly if it is not built."""
    import torch
    from oxillama_amd import quant
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible")
    quant.init(0)
    return quant
