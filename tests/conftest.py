import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def hip_lib():
    """The C-ABI library, loaded once; GPU tests call through it."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from matchattention_amd import _cabi
    return _cabi.load()


def pytest_terminal_summary(terminalreporter):
    """Worst measured error per label of every tests.util.check_err call, with its bound."""
    from tests import util
    if not util.MEASURED:
        return
    worst = {}
    for label, err, tol in util.MEASURED:
        if label not in worst or err / tol > worst[label][0] / worst[label][1]:
            worst[label] = (err, tol)
    terminalreporter.write_sep("-", "measured errors (max|a-b| / max|b|), worst per label")
    for label in sorted(worst):
        err, tol = worst[label]
        terminalreporter.write_line(f"{label:60s} {err:9.3e}  bound {tol:.1e}  ({err / tol:5.2f} x)")
