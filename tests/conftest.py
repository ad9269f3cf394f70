import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests"), os.path.join(ROOT, "ins-conv_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


@pytest.fixture(autouse=True)
def layer_by_layer_module_path():
    """A whole-network Sequential hands its frames to the network executor by itself.  The tests compare
    that executor with the layer-by-layer module path (one C call per layer through the reference's
    operator names), so here the switch is off unless a test turns it on (`auto_compile` fixture)."""
    import sparseconvnet as scn

    prev = scn.set_auto_compile(False)
    yield
    scn.set_auto_compile(prev)


@pytest.fixture
def auto_compile(layer_by_layer_module_path):
    import sparseconvnet as scn

    scn.set_auto_compile(True)
    yield
    scn.set_auto_compile(False)


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
