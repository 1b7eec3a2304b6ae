import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.oracle import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def golden():
    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as fh:
        return json.load(fh)


@pytest.fixture(scope="session")
def hip():
    """The HIP backend on device 0.  Fails loudly when the extension is not built."""
    import eddl_amd
    return eddl_amd.Backend(0)


def tensor_of(entry):
    return np.asarray(entry["data"], dtype=np.float32).reshape(entry["shape"])


def eddl_allclose(ref, out, atol, rtol=0.0):
    """The reference's own comparison, |a-b| <= atol + rtol*|b| with equal NaNs
    (src/hardware/cpu/cpu_comparison.cpp:146-170)."""
    ref = np.asarray(ref, np.float32)
    out = np.asarray(out, np.float32)
    both_nan = np.isnan(ref) & np.isnan(out)
    close = np.abs(ref - out) <= (atol + rtol * np.abs(out))
    return bool(np.all(close | both_nan))
