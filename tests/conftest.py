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
    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as handle:
        return json.load(handle)


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as module

    module.load()
    return module


@pytest.fixture(scope="session")
def hip():
    """The HIP backend mirror; fails (does not skip) when the library or the device is missing."""
    from spiraltorch_amd import hip as module

    module.init()
    return module


def assert_close(actual, expected, rel, abs_tol, what=""):
    """Elementwise |a - e| <= abs_tol + rel*|e| — the parity bar (f32: rel 1e-4 / abs 1e-5)."""
    a = np.asarray(actual, dtype=np.float64).ravel()
    e = np.asarray(expected, dtype=np.float64).ravel()
    assert a.shape == e.shape, f"{what}: shape {a.shape} vs {e.shape}"
    assert np.isfinite(a).all(), f"{what}: non-finite values in the result"
    err = np.abs(a - e)
    bound = abs_tol + rel * np.abs(e)
    worst = int(np.argmax(err - bound))
    if os.environ.get("ST_PRINT_MARGINS") and a.size:  # how much of each bar a run uses: `pytest -s` with this set
        used = float(np.max(err / np.maximum(bound, 1e-300))) if np.all(bound > 0) else float("nan")
        print(f"\n[margin] {used:8.3f} of the bar  {what}  ({a.size} values)", flush=True)
    assert (err <= bound).all(), (
        f"{what}: {int((err > bound).sum())} of {a.size} elements out of tolerance; worst at {worst}: "
        f"actual {a[worst]!r} expected {e[worst]!r} |diff| {err[worst]:.3e} bound {bound[worst]:.3e}")


F32_REL, F32_ABS = 1e-4, 1e-5
BF16_REL = 2e-2
