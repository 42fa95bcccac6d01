import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def vectors():
    """The reference's golden vectors (tests/vectors.sexp converted by tests/golden/make_vectors.py)."""
    with open(os.path.join(ROOT, "tests", "golden", "vectors.json")) as f:
        data = json.load(f)

    def of(kind):
        out = [v for v in data if v["kind"] == kind]
        assert out, f"no test vectors of kind {kind}"
        return out

    return of
