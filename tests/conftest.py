import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
if os.path.dirname(os.path.abspath(__file__)) not in sys.path:
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """A fresh checkout has no native libraries: compile them once (hipcc cross-compiles without a GPU).
    Libraries that are there are used as they are."""
    import __graft_entry__
    __graft_entry__.ensure_built()


@pytest.fixture(scope="session")
def hk():
    """The product package (ctypes harness over libhk_rowwise.so)."""
    import helpers
    return helpers.load_package()


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")


def pytest_terminal_summary(terminalreporter):
    """The strictly element-relative error of every comparison against the oracle, worst case per test file and
    quantity (helpers.assert_close)."""
    import helpers
    if not helpers.STRICT_LOG:
        return
    tr = terminalreporter
    tr.section("strict relative error |a - e| / |e| over elements with |e| >= %.0e rms(e)" % helpers.STRICT_FLOOR)
    tr.write_line("ordinary: the same over elements with |e| >= %.1f rms(e), held to the dtype's own tolerance"
                  % helpers.ORDINARY_FLOOR)
    tr.write_line("%-34s %-22s %-5s %11s %9s %11s %9s %11s %6s" % ("test file", "quantity", "dtype", "ordinary", "bound",
                                                                   "strict", "bound", "gate", "calls"))
    for (f, what, dt), (strict, bound, gate, n, ordinary, obound) in sorted(helpers.STRICT_LOG.items()):
        tr.write_line("%-34s %-22s %-5s %11.3e %9.1e %11.3e %9.1e %11.3e %6d" % (f, what[:22], dt, ordinary, obound,
                                                                                 strict, bound, gate, n))
