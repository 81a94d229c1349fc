import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden_dir():
    return os.path.join(ROOT, "tests", "golden")


def pytest_terminal_summary(terminalreporter):
    """What the element-wise comparisons of tests/parity.py measured in this session (exempt shares and
    worst entries per tensor): printed, and also written to the file that the environment variable
    P2_PARITY_REPORT names, if it is set."""
    from tests import parity
    if not parity.MEASURED:
        return
    text = parity.measured_report()
    terminalreporter.write_sep("-", "parity: measured over this session")
    terminalreporter.write_line(text)
    out = os.environ.get("P2_PARITY_REPORT")
    if out:
        with open(out, "w") as f:
            f.write(text + "\n")
