import os
import random
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(autouse=True)
def _seed_everything():
    # same discipline as the reference's test/conftest.py:225-245: every test starts from a fixed seed
    random.seed(95051)
    np.random.seed(95051)
    torch.manual_seed(95051)
    yield


MEASURED = []  # (what, measured, bound): margins the GPU parity tests report in the terminal summary


def pytest_terminal_summary(terminalreporter):
    if MEASURED:
        terminalreporter.write_line("measured parity margins (relative L2 error against the fp32 oracle):")
        for what, value, bound in MEASURED:
            terminalreporter.write_line(f"  {what}: {value:.3e} (bound {bound:g})")
