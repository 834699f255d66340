import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def pytest_terminal_summary(terminalreporter):
    """The measured error of every parity assertion, worst case per label, with the bound it was held to; also
    written to the file PMESH_PARITY_REPORT names."""
    import util
    worst = {}
    for what, e, tol in util.MEASURED:
        if what not in worst or e > worst[what][0]:
            worst[what] = (e, tol)
    if not worst:
        return
    lines = ["%-72s %.3e  (bound %.1e)" % (w[:72], e, tol) for w, (e, tol) in sorted(worst.items())]
    terminalreporter.write_sep("-", "measured parity errors (worst per label)")
    for l in lines:
        terminalreporter.write_line(l)
    path = os.environ.get("PMESH_PARITY_REPORT")
    if path:
        with open(path, "w") as fh:
            fh.write("\n".join(lines) + "\n")


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from picassoplus_amd import _lib
    _lib.load()                      # fail loudly if the HIP library is missing
    return torch.device("cuda:0")


@pytest.fixture
def native_options(monkeypatch):
    """Set PMESH_* switches for one test: the library reads them once, so it is told to read them again, and once
    more when the test is over."""
    from picassoplus_amd import _lib

    def set_options(**env):
        for k, v in env.items():
            monkeypatch.setenv(k, v)
        _lib.reload_options()

    yield set_options
    monkeypatch.undo()
    _lib.reload_options()
