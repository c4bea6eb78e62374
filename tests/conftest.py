import os
import sys
from pathlib import Path

import pytest

# The GPU tests own the box they run on: opt in to the one-kernel per-tensor dynamic quantization, as a
# caller with the GPU to itself would (tests of the default switch it off themselves).
os.environ.setdefault("DRISS_TORCH_RESIDENT", "1")

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu_device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")
