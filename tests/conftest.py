import os
import sys

import pytest

# Every launch made through the Python operators in the tests is followed by a read of the scheduler's status word: a
# schedule the device refused (or a wait of the chained backward that ran out) raises instead of returning zeros.
os.environ.setdefault("SBA_DEBUG_CHECK", "1")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_PARENT = os.path.join(ROOT, "stickbreaking-attention_amd")
for p in (ROOT, PKG_PARENT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gpu_device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")
