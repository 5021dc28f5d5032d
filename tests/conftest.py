import os
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parents[1]
for p in (str(ROOT), str(ROOT / "oracle"), str(ROOT / "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (runs through the PJRT C API of the built plugin)")


@pytest.fixture(scope="session")
def client():
    """The plugin's PJRT client.  No fallback: a missing library or device is an error, not a skip."""
    from jax_mps_amd import pjrt
    return pjrt.get_client()


def rel_err(got: np.ndarray, want: np.ndarray) -> float:
    """max |got - want| / max |want| over finite entries; NaN/inf positions must agree exactly."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    fin = np.isfinite(want)
    if not np.array_equal(np.isnan(got), np.isnan(want)):
        return float("inf")
    if not np.array_equal(got[~fin & ~np.isnan(want)], want[~fin & ~np.isnan(want)]):
        return float("inf")
    if not fin.any():
        return 0.0
    scale = max(float(np.abs(want[fin]).max()), 1e-30)
    return float(np.abs(got[fin] - want[fin]).max()) / scale


def closeness(got: np.ndarray, want: np.ndarray, rtol: float = 1e-5, atol: float = 1e-5) -> float:
    """The reference's elementwise rule (tests/test_ops.py:91-105: assert_allclose(atol=1e-5, rtol=1e-5)) as a
    number: max over elements of |got - want| / (atol + rtol * |want|); <= 1 passes.  NaN and infinite
    positions must agree exactly."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    if not np.array_equal(np.isnan(got), np.isnan(want)):
        return float("inf")
    fin = np.isfinite(want)
    if not np.array_equal(got[~fin & ~np.isnan(want)], want[~fin & ~np.isnan(want)]):
        return float("inf")
    if not fin.any():
        return 0.0
    return float((np.abs(got[fin] - want[fin]) / (atol + rtol * np.abs(want[fin]))).max())
