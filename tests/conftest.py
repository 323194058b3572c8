import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden():
    import json
    with open(os.path.join(GOLDEN, "reference_goldens.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def golden_dir():
    return GOLDEN


@pytest.fixture(autouse=True)
def plans_at_the_first_product(monkeypatch):
    """The library builds its SpMM and SpMV plans when a matrix is multiplied for the second time; the tests
    multiply once, so they ask for the plan at once (the tests of that rule take the switch away again)."""
    monkeypatch.setenv("COMET_HIP_PLAN_AT_ONCE", "1")
