import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
TESTS = os.path.dirname(os.path.abspath(__file__))
if TESTS not in sys.path:  # (test modules share helpers)
    sys.path.insert(1, TESTS)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def vectors():
    """The reference's own golden vectors (tests/golden/extract_fixtures.py wrote them)."""
    import json
    with open(os.path.join(ROOT, "tests", "golden", "frink_quant_vectors.json")) as f:
        return json.load(f)
