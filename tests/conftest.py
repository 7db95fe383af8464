import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.lib()
    return o


def pytest_terminal_summary(terminalreporter):
    """How much of each dot comparison passed only through the absolute floor (or, for f8 results,
    with a code other than the oracle's): the comparisons with the largest shares, so that the
    tolerance actually used shows in the log of every run."""
    try:
        from tests.gpu_util import FLOOR_LOG
    except Exception:
        return
    if not FLOOR_LOG:
        return
    rows = sorted(FLOOR_LOG, key=lambda r: -(r[2] / max(r[3], 1)))
    shown = [r for r in rows if r[2] > 0][:25]
    tr = terminalreporter
    tr.write_sep("-", "parity: %d dot comparisons, %d leaned on the floor / differ in code" % (len(rows), len([r for r in rows if r[2]])))
    for what, kind, n, total in shown:
        tr.write_line("  %6.3f%%  %7d of %-9d %s: %s" % (100.0 * n / max(total, 1), n, total, kind, what))
