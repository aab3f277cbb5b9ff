import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def vectors():
    with open(os.path.join(GOLDEN, "reference_vectors.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def n22():
    return np.fromfile(os.path.join(GOLDEN, "n22_mt19937_seed1_6000.f32"), np.float32)


@pytest.fixture(scope="session")
def oracle():
    import oracle as o
    return o.lib


@pytest.fixture(scope="session")
def ref():
    import oracle as o
    if o.ref is None:
        pytest.skip("compiled reference (oracle/_ref) not built on this machine")
    return o.ref
