import os
import sys
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _has_gpu():
    return os.path.exists("/dev/kfd")


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this container")
    for it in items:
        if "gpu" in it.keywords:
            it.add_marker(skip)


def pytest_terminal_summary(terminalreporter):
    """The margins of every parity check of the run (tests/helpers.py assert_parity), worst first."""
    try:
        from helpers import MARGINS
    except Exception:
        return
    if not MARGINS:
        return
    terminalreporter.write_sep("-", "parity margins: %d checks, worst 25 by share of the effective budget" % len(MARGINS))
    for what, d, rel, mx, budget in sorted(MARGINS, key=lambda r: -r[1] / r[4])[:25]:
        terminalreporter.write_line("%-60s max-abs %.3e  rel %.3e  max|ref| %.5f  %5.1f %% of budget %.2e" % (what, d, rel, mx, 100 * d / budget, budget))
