import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests"), os.path.join(ROOT, "ins-conv_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def orc():
    from oracle import oracle

    oracle.lib()
    return oracle


def pytest_terminal_summary(terminalreporter):
    """The float errors the parity checks observed (tests/parity.py), one line per check."""
    import parity

    if parity.REPORT:
        terminalreporter.section("parity report (tolerance 1e-5 + 1e-4*|ref| per element)")
        for line in parity.REPORT:
            terminalreporter.write_line(line)
