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


FP32_RTOL = 1e-4   # parity bar for fp32 (relative to the tensor's largest magnitude)
BF16_RTOL = 1e-2   # parity bar for 16-bit storage


def assert_close(actual, expected, rtol, what=""):
    import numpy as np
    a = np.asarray(actual, np.float64).reshape(-1)
    b = np.asarray(expected, np.float64).reshape(-1)
    assert a.shape == b.shape, (what, a.shape, b.shape)
    assert np.all(np.isfinite(a)), what
    scale = max(float(np.abs(b).max()), 1e-30)
    err = float(np.abs(a - b).max()) / scale
    assert err <= rtol, "%s: relative error %.3e > %.1e" % (what, err, rtol)
    return err


def bf16_round(x):
    """Round an fp32 array to the nearest bf16 value (ties to even), returned as fp32."""
    import numpy as np
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return r.astype(np.uint32).view(np.float32).reshape(np.shape(x))


class Dev:
    """Thin test helper over the CudaDnn mirror: numpy in, handles out."""

    def __init__(self):
        from mycaffe_amd.cudadnn import CudaDnn
        self.cuda = CudaDnn(0)
        self.handles = []

    def put(self, arr, half=False):
        import numpy as np
        h = self.cuda.AllocMemory(np.asarray(arr, np.float32), bHalfSize=half)
        self.handles.append(h)
        return h

    def zeros(self, n, half=False):
        h = self.cuda.AllocMemory(int(n), bHalfSize=half)
        self.handles.append(h)
        return h

    def get(self, h, shape=None):
        a = self.cuda.GetMemoryFloat(h)
        return a.reshape(shape) if shape is not None else a

    def close(self):
        for h in self.handles:
            try:
                self.cuda.FreeMemory(h)
            except Exception:
                pass
        self.handles = []
        self.cuda.Dispose()


@pytest.fixture()
def dev():
    d = Dev()
    yield d
    d.close()
