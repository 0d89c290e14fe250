import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "mini-sglang-mlx_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU (run on the MI355X box)")


@pytest.fixture(scope="session")
def gpu():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no ROCm GPU visible")
    return torch.device("cuda:0")


_KNOBS = range(10)  # MSGL_TUNE_* of include/msgl_paged_attention.h


def _reset_knobs():
    from mini_sglang_amd_kernel import _lib

    if os.path.exists(_lib.LIB_PATH):
        for knob in _KNOBS:
            _lib.set_tuning(knob, 0)


@pytest.fixture(autouse=True)
def _knobs_back_to_default():
    """No test can leak a benchmarking knob into the next one, however it ends."""
    yield
    _reset_knobs()


@pytest.fixture
def tuning():
    """``tuning(knob, value)`` sets a benchmarking knob of the library for the rest of the test;
    every knob is back at its default when the test is over."""
    from mini_sglang_amd_kernel import _lib

    def set_knob(knob, value):
        _lib.set_tuning(knob, value)

    yield set_knob
    _reset_knobs()
