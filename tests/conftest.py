import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "state-space-models-neuron_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def goldens():
    import numpy as np
    return np.load(os.path.join(ROOT, "tests", "golden", "hf_goldens.npz"))


@pytest.fixture(scope="session")
def lib():
    """The C-ABI library; GPU tests fail (not skip) when it is missing."""
    from mamba2 import _lib
    return _lib.load()


def rel_rms_err(got, ref):
    """max |got - ref| / RMS(ref): the bf16 acceptance metric (tolerance 2e-2)."""
    import torch
    ref = ref.double()
    got = got.double().to(ref.device)
    rms = ref.pow(2).mean().sqrt().clamp_min(1e-30)
    return ((got - ref).abs().max() / rms).item()


def rel_err(got, ref):
    """fp32 acceptance metric: max |got - ref| / max |ref|  (tolerance 1e-4)."""
    ref = ref.double()
    got = got.double().to(ref.device)
    return ((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30)).item()
