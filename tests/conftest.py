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
def oracle():
    """The CPU oracle (test infrastructure; builds libls_oracle.so on first use)."""
    from oracle import oracle as _oracle
    return _oracle


@pytest.fixture
def rng():
    return np.random.default_rng(0)


def assert_codes_close(got, want, max_frac=1e-3, what="int8 codes"):
    """int8 activations: at most +-1 code on at most 0.1 % of the elements."""
    got = np.asarray(got).astype(np.int32)
    want = np.asarray(want).astype(np.int32)
    assert got.shape == want.shape, (got.shape, want.shape)
    diff = np.abs(got - want)
    assert diff.max(initial=0) <= 1, "%s: max code difference %d" % (what, diff.max())
    frac = float((diff != 0).mean()) if diff.size else 0.0
    assert frac <= max_frac, "%s: %.4f%% of elements differ (limit %.4f%%)" % (
        what, 100 * frac, 100 * max_frac)
    return frac
