import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_ROOT = os.path.join(ROOT, "sinabs-exodus_amd")
for p in (ROOT, PKG_ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden_dir():
    return os.path.join(ROOT, "tests", "golden")


def pytest_terminal_summary(terminalreporter):
    """Gradient assertions that used a scaled tolerance: their worst error in units of the stated
    tolerance (rtol 1e-4 / atol 1e-5), so that the scaling hides nothing."""
    try:
        from _util import SCALED_TOLERANCE_REPORT as report
    except ImportError:
        return
    if not report:
        return
    tr = terminalreporter
    tr.write_sep("-", "assertions judged with a scaled tolerance: worst error in units of rtol 1e-4 / atol 1e-5")
    rows = sorted(report.items(), key=lambda kv: -kv[1][0])
    for what, (stated, used, rtol, atol) in rows[:40]:
        tr.write_line(f"{stated:10.3g} x stated   ({used:.3g} x the rtol {rtol:g} / atol {atol:.3g} it was judged with)   {what}")
    if len(rows) > 40:
        tr.write_line(f"... and {len(rows) - 40} more, all below {rows[40][1][0]:.3g} x stated")
