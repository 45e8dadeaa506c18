"""Shared fixtures.  Tests marked `gpu` need an MI355X and the built HIP library; everything else
runs on the CPU (oracle pins, host logic, C-ABI symbol checks)."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture
def rng():
    return np.random.default_rng(0)


def f16(a):
    """fp32 -> fp16 with IEEE round-to-nearest-even (what the device conversion does)."""
    return np.asarray(a, dtype=np.float32).astype(np.float16)


@pytest.fixture(autouse=True)
def _default_tuning_after_gpu_tests(request):
    """The tuning hooks of the library are process-global: whatever a GPU test forced (and however it
    ended) the next test starts from the default plans."""
    yield
    if request.node.get_closest_marker("gpu") is None:
        return
    from axono_amd import _lib

    l = _lib.load()
    l.axhip_gqa_decode_tune(0, 0)
    l.axhip_linear_f16_tune(0, 0, 0, 0)
    l.axhip_prefill_attention_tune(-1)
