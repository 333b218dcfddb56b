import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


# With log-prob outputs the top-k layer takes its fused step only from a few hundred rows on (below that the kernel
# sequence is faster); the tests want the fused step at every batch size. Tests of the default say so themselves.
os.environ.setdefault("FT_SAMPLING_FUSED_LOGPROBS_MIN_ROWS", "0")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")
