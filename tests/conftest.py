import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (run on the MI355X box)")


@pytest.fixture(autouse=True)
def _deterministic_backward():
    """Parity tests compare gradients bit for bit, which is what the plan-based backward
    delivers; the default mode would run the first backward on a new pattern statelessly
    (atomics, rounding order not fixed).  Tests of that policy switch the mode themselves."""
    from numml_amd import _binding
    old = _binding.backward_mode()
    _binding.set_backward_mode("eager")
    yield
    _binding.set_backward_mode(old)


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    return torch.device("cuda:0")
