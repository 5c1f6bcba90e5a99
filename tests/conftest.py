import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def lib():
    from flex_attention_tpu_amd import _lib
    return _lib.load()


@pytest.fixture(autouse=True)
def _name_the_test(request):
    import helpers
    helpers.CURRENT = request.node.name
    yield


def pytest_terminal_summary(terminalreporter):
    """Strict figures of every oracle comparison of the run, worst max-abs per test and tensor."""
    import helpers
    if not helpers.REPORT:
        return
    worst = {}
    for test, name, ref_max, ma, rl, ratio in helpers.REPORT:
        base = name.replace(" chain", "").replace(" whole", "")
        key = (test, base.split("[")[0].split(" ")[-1] + ("(whole)" if " whole" in name else "") + ("(chain)" if " chain" in name else ""))
        if key not in worst or ma > worst[key][1]:
            worst[key] = (ref_max, ma, rl, ratio)
    tr = terminalreporter
    tr.write_sep("-", "parity figures (worst per test and tensor): max|ref|, max-abs, rel-L2, error / bound")
    for (test, name), (ref_max, ma, rl, ratio) in worst.items():
        tr.write_line(f"{test:60s} {name:14s} max|ref|={ref_max:9.3f} max_abs={ma:.3e} rel_l2={rl:.3e} err/bound={ratio:.2f}")
