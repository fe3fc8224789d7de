import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

FIXTURES = os.path.join(ROOT, "tests", "golden", "reference_fixtures")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def load_fixture(kind, name):
    """Whitespace-separated float text file copied from the reference's tests/{input,output}."""
    with open(os.path.join(FIXTURES, kind, name)) as f:
        return np.array(f.read().split(), dtype=np.float64).astype(np.float32)


@pytest.fixture(scope="session")
def oracle():
    from oracle import cct_oracle
    cct_oracle.lib()
    return cct_oracle
