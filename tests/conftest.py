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
    config.addinivalue_line("markers", "both_batch_modes: runs twice, with the one-pass sums that most tests ask for and "
                                       "with the library's default handling of small batches (what a production caller gets)")


def pytest_generate_tests(metafunc):
    if metafunc.definition.get_closest_marker("both_batch_modes"):
        metafunc.fixturenames.append("batch_mode")
        metafunc.parametrize("batch_mode", ["one_pass", "default"])


@pytest.fixture(autouse=True)
def _one_pass_sums_unless_asked(request, monkeypatch):
    """By default the library spreads a small batch over slices of the trees and adds the slices' sums, which
    rounds differently from the CPU evaluator's single pass (within the 1e-9 bar). Most GPU tests compare sums
    bit for bit, so they switch that off; tests marked small_batch keep the default, and tests marked
    both_batch_modes (those that compare within the bar: goldens of the reference's tests, its unit-test
    models, the workloads through the host entry points) run both ways. The library reads its kernel switches
    only in a process that sets CATBOOST_AMD_TEST_SWITCHES=1, which every test does."""
    monkeypatch.setenv("CATBOOST_AMD_TEST_SWITCHES", "1")
    callspec = getattr(request.node, "callspec", None)
    mode = callspec.params.get("batch_mode") if callspec is not None else None
    if mode == "default":
        return
    if "small_batch" not in request.keywords:
        monkeypatch.setenv("CATBOOST_AMD_SMALL_BATCH", "0")


@pytest.fixture(scope="session")
def golden_dir():
    return GOLDEN
