import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def pkg():
    return entry.load_package()


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (test infrastructure)."""
    return entry.load_oracle()


@pytest.fixture(scope="session")
def gpu(pkg):
    g = pkg.HipGpu(0)
    yield g
    g.close()


def peak_err(got, want) -> float:
    """max|got - want| / max|want| — the reference's GEMV metric
    (crates/ojas-cuda/tests/conformance.rs:817-823)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return float(np.max(np.abs(got - want)) / max(np.max(np.abs(want)), 1e-30))


def rms_errs(got, want):
    """(max|d| / rms(want), rms(d) / rms(want)) — the reference's GEMM metric
    (crates/ojas-cuda/tests/prefill_gemm_q.rs:247-260)."""
    got = np.asarray(got, np.float64).ravel()
    want = np.asarray(want, np.float64).ravel()
    assert np.all(np.isfinite(got)), "non-finite output"
    rms = max(float(np.sqrt(np.mean(want * want))), 1e-30)
    d = got - want
    return float(np.max(np.abs(d)) / rms), float(np.sqrt(np.mean(d * d)) / rms)
