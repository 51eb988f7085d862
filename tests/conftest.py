import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    """Known-answer vectors of the reference's own unit tests (tests/golden/reference_vectors.json)."""
    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
        return json.load(f)


class Case(object):
    """One TEST_F of the reference: its arrays, size_t scalars and expectations."""

    def __init__(self, data, rel, name):
        f = data[rel]
        t = f["tests"][name]
        self.arrays = dict(f["globals"])
        self.arrays.update(t["arrays"])
        self.scalars = t["scalars"]
        self.expect = t["expect"]

    def check(self, got, var=None, closed_form=None):
        """Assert every expectation on `var` (default: all) against the flat array `got`.
        EXPECT_NEAR keeps its tolerance; EXPECT_FLOAT_EQ is 4 ulp of fp32."""
        import numpy as np
        flat = np.asarray(got, dtype=np.float64).ravel()
        n = 0
        for v, idx, value, tol in self.expect:
            if var is not None and v != var:
                continue
            if isinstance(value, str):
                value = closed_form(idx)
            if tol is None:
                tol = 4 * np.spacing(np.float32(abs(value))) if value != 0 else 1e-30
            assert abs(flat[idx] - value) <= tol, "%s[%d]: got %r want %r (tol %g)" % (v, idx, flat[idx], value, tol)
            n += 1
        assert n > 0
        return n


@pytest.fixture(scope="session")
def case(golden):
    return lambda rel, name: Case(golden, rel, name)
