import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def cuda():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")


_KNOB_DEFAULTS = {"no_pipe": 0, "bm": 0, "no_split": 0, "no_xcd_order": 0, "bound": -1, "stream": -1, "stream_even": -1, "stream_dyn": -1, "stream_solo": 0, "sparse_pair": 0, "wave_rows": 0, "short_keys": -1, "sparse_order": 1}


@pytest.fixture
def tuning():
    """Setter for the library's tuning knobs (pa_set_tuning); every knob is back at its default after the test."""
    from paraattention_amd import _lib

    yield _lib.set_tuning
    for name, val in _KNOB_DEFAULTS.items():
        _lib.set_tuning(name, val)
