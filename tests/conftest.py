import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_terminal_summary(terminalreporter):
    """Largest error of every 16-bit parity check, in ulps of the output type (tests/tolerance.py)."""
    from tests import tolerance

    if not tolerance.RECORDS:
        return
    worst = {}
    for label, ulps, err, floor in tolerance.RECORDS:
        kind = label.split(" ")[0]
        if kind not in worst or ulps > worst[kind][1]:
            worst[kind] = (label, ulps, err, floor)
    terminalreporter.write_line(f"16-bit parity checks against the fp32 anchor: {len(tolerance.RECORDS)} (rtol 1.6e-2 + floor)")
    for kind in sorted(worst):
        label, ulps, err, floor = worst[kind]
        terminalreporter.write_line(f"  worst {kind}: {ulps:.2f} ulp, |err| {err:.3g}, floor {floor:.3g}  [{label}]")


@pytest.fixture(autouse=True)
def _reset_dynamo():
    torch._dynamo.reset()
    yield
    torch._dynamo.reset()


@pytest.fixture(scope="session")
def device():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")
