import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def dev():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def bf16_tensor(x_f32_np, device):
    """numpy float32 holding bf16-representable values -> torch bf16 tensor on device (exact)."""
    import torch

    return torch.from_numpy(np.ascontiguousarray(x_f32_np)).to(torch.bfloat16).to(device)


def fp8_tensor(q_u8_np, device):
    import torch

    return torch.from_numpy(np.ascontiguousarray(q_u8_np)).to(device).view(torch.float8_e4m3fn)


def u8(t):
    import torch

    return t.contiguous().view(torch.uint8).cpu().numpy()
