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
    """Tensor literals transcribed from the reference's own unit tests."""
    with open(os.path.join(ROOT, "tests", "golden", "reference_literals.json")) as f:
        raw = json.load(f)

    def get(rel, test, name, dtype=np.float32):
        return np.array(raw[rel][test][name]["data"], dtype=dtype)

    return get
