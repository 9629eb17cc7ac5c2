import importlib
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
    config.addinivalue_line("markers", "gpu: needs a HIP device (run on the MI355X box)")


@pytest.fixture(scope="session")
def pkg():
    return importlib.import_module("turboquant-pytorch_amd")


@pytest.fixture(scope="session")
def oracle():
    from oracle import tq_oracle
    tq_oracle._load()
    return tq_oracle


@pytest.fixture(scope="session")
def golden():
    """Outputs of the upstream reference on seeded inputs (written by tests/golden/make_fixtures.py)."""
    out = {name: np.load(os.path.join(GOLDEN, name + ".npz")) for name in
           ("codebooks", "rotations", "mse_roundtrip", "config1", "v3", "odd_dims")}
    with open(os.path.join(GOLDEN, "fixtures.json")) as f:
        out["json"] = json.load(f)
    return out
