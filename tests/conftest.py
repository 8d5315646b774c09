import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (MI355X); run with -m gpu")


@pytest.fixture(scope="session")
def device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    return torch.device("cuda:0")


@pytest.fixture
def tuning():
    """``tuning(ARTAB_SMALL=0)``: route overrides of the loaded library (artab_tuning_set) for the
    duration of one test; the state found before the test is restored afterwards."""
    from ar_nanotabpfn_amd import _lib

    saved = {}

    def set_overrides(**overrides):
        for key in overrides:
            saved.setdefault(key, _lib.tuning.get(key))
        _lib.tuning.set(**overrides)

    yield set_overrides
    _lib.tuning.set(**saved)
