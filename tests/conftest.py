import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def cuda():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


# Parity figures that tests want seen even in a quiet run (label differences under the strict gap rule,
# iteration counts): collected here and printed as one block after the test summary.
_PARITY_LINES = []


@pytest.fixture
def parity_report():
    def add(line: str) -> None:
        print(line, flush=True)
        _PARITY_LINES.append(line)

    return add


def pytest_terminal_summary(terminalreporter):
    if _PARITY_LINES:
        terminalreporter.section("parity figures (product vs CPU oracle)")
        for line in _PARITY_LINES:
            terminalreporter.write_line(line)
