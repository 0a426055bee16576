import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")
for p in (ROOT, GOLDEN):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def close_either(got, want, eps):
    """The reference's comparison rule (src/tensor/data.rs:63-102, CompPolicy::Either):
    every element passes if |x-y| < eps OR |x-y|/|y| < eps."""
    got = np.asarray(got, np.float64).ravel()
    want = np.asarray(want, np.float64).ravel()
    assert got.shape == want.shape, (got.shape, want.shape)
    diff = np.abs(got - want)
    both_inf = np.isinf(got) & np.isinf(want) & (np.sign(got) == np.sign(want))
    with np.errstate(divide="ignore", invalid="ignore"):
        rel = np.where(np.abs(want) == 0, diff, diff / np.abs(want))
    ok = both_inf | (diff < eps) | (rel < eps)
    return bool(ok.all()), float(np.nanmax(np.where(both_inf, 0, diff))) if diff.size else 0.0


def max_abs_rel(got, want):
    """max over elements of |x-y| / max(|y|, floor) with floor = 1e-2 * max|y| (the
    'max-abs-rel' figure quoted for 16-bit outputs)."""
    got = np.asarray(got, np.float64).ravel()
    want = np.asarray(want, np.float64).ravel()
    floor = 1e-2 * max(float(np.max(np.abs(want))), 1e-30)
    return float(np.max(np.abs(got - want) / np.maximum(np.abs(want), floor)))


def max_err_rel_to_max(got, want):
    """max|x-y| / max|y|: the error relative to the tensor's magnitude.  Used for results that
    pass through many 16-bit roundings (whole-decoder logits), where elements near zero carry an
    absolute error set by the large ones."""
    got = np.asarray(got, np.float64).ravel()
    want = np.asarray(want, np.float64).ravel()
    return float(np.max(np.abs(got - want)) / max(float(np.max(np.abs(want))), 1e-30))


@pytest.fixture(scope="session")
def golden_dir():
    return GOLDEN
