import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden_cpu():
    from oracle import bsmxfix
    return bsmxfix.load(os.path.join(ROOT, "tests", "golden", "golden_cpu.bin"))


@pytest.fixture(scope="session")
def golden_gpu():
    from oracle import bsmxfix
    return bsmxfix.load(os.path.join(ROOT, "tests", "golden", "golden_gpu.bin"))
