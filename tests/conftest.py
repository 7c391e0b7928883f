import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def load_txt(path):
    """Reference text tensor: first line '# (shape)', then one value per line."""
    import numpy as np
    with open(path) as f:
        first = f.readline().strip()
        shape = tuple(int(s) for s in first.lstrip("# (").rstrip(")").split(",") if s.strip())
        vals = np.array([float(l) for l in f if l.strip()], np.float64)
    return vals.reshape(shape)


@pytest.fixture(scope="session")
def golden_dir():
    return GOLDEN
