import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "small_batch: runs with the library's default handling of small batches")


@pytest.fixture(autouse=True)
def _one_pass_sums_unless_asked(request, monkeypatch):
    """By default the library spreads a small batch over slices of the trees and adds the slices' sums, which
    rounds differently from the CPU evaluator's single pass (within the 1e-9 bar). Most GPU tests compare sums
    bit for bit, so they switch that off; tests marked small_batch keep the default."""
    if "small_batch" not in request.keywords:
        monkeypatch.setenv("CATBOOST_AMD_SMALL_BATCH", "0")


@pytest.fixture(scope="session")
def golden_dir():
    return GOLDEN
