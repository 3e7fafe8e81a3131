"""Shared pytest plumbing: the `gpu` marker, import paths, and seeded input makers."""
import importlib
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (checker only)."""
    import w4a32_oracle

    w4a32_oracle.lib()
    return w4a32_oracle


@pytest.fixture(scope="session")
def pkg():
    """The product package (its directory name has a hyphen, hence import_module)."""
    return importlib.import_module("mllm-advanced_amd")


def make_weights(n, k, seed=0, std=0.02):
    return (np.random.default_rng(seed).standard_normal((n, k)) * std).astype(np.float32)


def make_acts(m, k, seed=1, outlier_frac=0.0):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, k)).astype(np.float32)
    if outlier_frac > 0:
        cnt = max(1, int(np.ceil(outlier_frac * m)))
        rows = rng.permutation(m)[:cnt]
        x[rows] *= 20.0
    return x


def max_abs_rel(y, ref):
    """max |y - ref| / max |ref|: the tolerance metric used for f32 outputs."""
    ref = np.asarray(ref, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    denom = max(float(np.abs(ref).max()), 1e-30)
    return float(np.abs(y - ref).max() / denom)
