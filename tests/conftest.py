import importlib
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

# the reference's shape grid (B, N, L, K), testing/test.cpp:50-59
REFERENCE_SHAPES = [
    (3, 5, 4, 2),
    (12, 8, 8, 4),
    (127, 254, 513, 4),
    (12, 8, 32, 16),
    (17, 12, 63, 44),
    (127, 254, 513, 73),
    (127, 254, 513, 80),
    (1, 32, 4_000_000, 4),
]


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def load_package():
    """The package directory has a hyphen in its name, so it is imported by string."""
    return importlib.import_module("ecml23-sparse_amd")


@pytest.fixture(scope="session")
def pkg():
    return load_package()


def reference_law_inputs(B, N, L, K, seed=42):
    """Inputs drawn the way the reference's randomised tests draw them
    (testing/test_case_templates.h:52-69,113-114): uniform[-1,1] features and weights, column ids
    uniform WITH replacement, out_grad = max(0, uniform[-1,1]) (about half exact zeros)."""
    rng = np.random.default_rng(seed)
    x = rng.uniform(-1, 1, (B, N)).astype(np.float32)
    lookup = rng.integers(0, N, (L, K), dtype=np.int64).astype(np.int32)
    w = rng.uniform(-1, 1, (L, K)).astype(np.float32)
    g = np.maximum(rng.uniform(-1, 1, (B, L)), 0).astype(np.float32)
    return x, lookup, w, g


def rel_err(a, ref):
    """max|a-ref| / max|ref| — the relative gate used for every parity check."""
    a = np.asarray(a, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    denom = np.abs(ref).max()
    return float(np.abs(a - ref).max() / (denom if denom > 0 else 1.0))
