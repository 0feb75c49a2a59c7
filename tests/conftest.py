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
def golden():
    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def orc():
    from oracle import cpu_oracle
    cpu_oracle.lib()
    return cpu_oracle


@pytest.fixture(scope="session")
def device():
    """The HipDevice under test; a missing library or GPU is an error for a gpu test, never a skip to CPU."""
    from neureka_amd import HipDevice
    dev = HipDevice.get(0)
    # every buffer is handed out filled with 0xFF bytes (NaN) for the whole session: an operation that relied on the
    # contents of a fresh drain, which the pool does not define, would show in its own test
    dev.configurePool(poison=True)
    print(f"[device] {dev!r}", flush=True)
    yield dev


DTYPES = {"f32": np.float32, "f64": np.float64}
