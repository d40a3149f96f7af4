import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_terminal_summary(terminalreporter):
    """Measured parity errors of the session (max|got-ref| / max|ref| per tensor), so that a
    drift inside the tolerance is visible in the run's output."""
    from tests import util
    if not util.MEASURED:
        return
    terminalreporter.write_sep("-", "measured parity errors: max|got - oracle| / max|oracle|")
    labels = []
    for label, _ in util.MEASURED:
        if label not in labels:
            labels.append(label)
    for label in labels:
        cells = ["%s %.2e" % (name, err) for (lab, name), err in util.MEASURED.items() if lab == label]
        terminalreporter.write_line("%-34s %s" % (label, "  ".join(cells)))
