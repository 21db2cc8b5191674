import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle_mod():
    from oracle import oracle
    oracle.lib()
    return oracle


@pytest.fixture(scope="session")
def gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from svox_amd.csrc import _abi
    _abi.load_library()  # raises if the HIP library is not built: GPU tests never fall back
    return torch.device("cuda:0")


def pytest_terminal_summary(terminalreporter):
    """How close to the gradient gate the kernels ran: the worst error of every test that compared a gradient."""
    try:
        from util import GATE_LOG
    except ImportError:
        return
    if not GATE_LOG:
        return
    worst = {}
    for label, err, limit, slack in GATE_LOG:
        key = (label, limit, slack)
        worst[key] = max(worst.get(key, 0.0), err)
    tr = terminalreporter
    tr.write_sep("-", "gradient gate: worst relative error per test (limit; * = order slack of the oracle taken off)")
    for (label, limit, slack), err in sorted(worst.items(), key=lambda kv: -kv[1] / kv[0][1])[:30]:
        tr.write_line(f"  {err:9.3e} of {limit:.0e}{'*' if slack else ' '} {label}")
