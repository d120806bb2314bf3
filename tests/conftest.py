import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "expert-kit_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.lib()
    return o


@pytest.fixture(scope="session")
def ek():
    """The ek_hip package with libek_hip.so loaded (fails loudly if it is not built)."""
    import ek_hip
    ek_hip.load()
    return ek_hip


@pytest.fixture(scope="session")
def cuda(ek):
    import torch
    assert torch.cuda.is_available(), "gpu-marked test started without a GPU"
    assert ek.load().ek_device_count() >= 1
    return torch.device("cuda:0")


def pytest_terminal_summary(terminalreporter):
    """The parity gates' plain figures (`-q` drops test output, not this)."""
    import parity_report
    for line in parity_report.summary_lines():
        terminalreporter.write_line(line)
    parity_report.dump_if_asked()
