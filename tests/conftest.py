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
def device():
    import floneum_amd as fa
    return fa.Device.default()


def rel_l2(y, ref):
    y = np.asarray(y, np.float64)
    ref = np.asarray(ref, np.float64)
    return float(np.linalg.norm(y - ref) / max(np.linalg.norm(ref), 1e-300))


def max_abs(y, ref):
    return float(np.max(np.abs(np.asarray(y, np.float64) - np.asarray(ref, np.float64)))) if np.size(y) else 0.0


# tolerances of the parity gate: 16-bit inputs max-abs 2e-3 and relative L2 1e-3; f32 inputs relative L2 1e-5
TOL_16 = dict(max_abs=2e-3, rel_l2=1e-3)
TOL_F32 = dict(rel_l2=1e-5, max_abs=2e-5)


def assert_parity(y, ref, tol, what=""):
    assert not np.isnan(np.asarray(y, np.float64)).any(), f"{what}: NaN in output"
    ra, ma = rel_l2(y, ref), max_abs(y, ref)
    assert ra <= tol["rel_l2"], f"{what}: rel-L2 {ra:.3e} > {tol['rel_l2']:.1e} (max-abs {ma:.3e})"
    assert ma <= tol["max_abs"], f"{what}: max-abs {ma:.3e} > {tol['max_abs']:.1e} (rel-L2 {ra:.3e})"
    return ra, ma
