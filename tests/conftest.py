import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 GPU (runs the HIP kernels through the C ABI)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (checker only)."""
    from oracle import oracle as O

    O.lib()
    return O


@pytest.fixture(scope="session")
def ctx():
    """One context on GPU 0 for the whole session.  Fails (does not skip) when the
    library or the device is missing: GPU tests never pass on a fallback."""
    import wick_amd as W

    c = W.RocmContext(0)
    yield c
    c.close()


def rel_l2(a, b) -> float:
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))


def assert_f32_parity(got, ref, what=""):
    """The contract for f32 outputs: rel-L2 <= 1e-5 and max-abs <= 1e-4 x output RMS."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    r = rel_l2(got, ref)
    rms = float(np.sqrt(np.mean(ref * ref)))
    mx = float(np.abs(got - ref).max()) if got.size else 0.0
    assert r <= 1e-5, f"{what}: rel-L2 {r:.3e} > 1e-5"
    assert mx <= 1e-4 * rms + 1e-30, f"{what}: max-abs {mx:.3e} > 1e-4 * rms ({rms:.3e})"
