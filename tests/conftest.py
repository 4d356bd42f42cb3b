import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (run on the MI355X box)")


@pytest.fixture(autouse=True)
def _global_state():
    # mirrors the reference's tests/conftest.py:6-9, without moving the default
    # device: every test here places its tensors explicitly
    from triturus_amd.utils import set_tf32_enabled

    set_tf32_enabled(False)
    torch.manual_seed(42)


@pytest.fixture
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    return torch.device("cuda", 0)
