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


def load_golden(name):
    """Returns {case: {array_name: ndarray}} from tests/golden/<name>.npz."""
    out = {}
    with np.load(os.path.join(GOLDEN, name + ".npz")) as z:
        for key in z.files:
            case, arr = key.split("/")
            out.setdefault(case, {})[arr] = z[key]
    return out


def rel_err(y, ref, floor_frac=1.0):
    """max|y-ref| / max(|ref|, floor_frac*rms(ref)).

    y is a weighted mean of zero-mean values and crosses zero, so a pointwise relative error
    needs a floor; with floor_frac=1 this is the usual allclose(rtol, atol=rtol*rms) test.
    floor_frac=1e-2 is the stricter variant, reported but only gated where stated."""
    y = np.asarray(y, np.float64)
    ref = np.asarray(ref, np.float64)
    floor = floor_frac * np.sqrt(np.mean(ref * ref)) + 1e-300
    return float(np.max(np.abs(y - ref) / np.maximum(np.abs(ref), floor)))


@pytest.fixture
def force():
    """force(name, value): sets a tuning / testing switch of the library (vrwkv_set_option) until the test ends."""
    import vision_rwkv_amd as ops
    saved = {}

    def _set(name, value=1):
        saved.setdefault(name, ops.get_option(name))
        ops.set_option(name, value)

    yield _set
    for name, value in saved.items():
        ops.set_option(name, value)
