import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (run on the MI355X box)")


@pytest.fixture(scope="session")
def built_lib():
    """Path of libunirl_hip.so; builds it only when nothing has been built yet."""
    from unirl_amd import _native

    if not _native.LIB_PATH.exists():
        from unirl_amd.build import build

        build(verbose=False)
    return _native.LIB_PATH


@pytest.fixture(scope="session")
def dev(built_lib):
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no HIP device visible")
    return torch.device("cuda", 0)


def rel_err(a, b, floor=0.0):
    """max |a-b| / max(|b|, floor) over all elements, in float64."""
    import torch

    a = torch.as_tensor(a).double().cpu()
    b = torch.as_tensor(b).double().cpu()
    return float(((a - b).abs() / b.abs().clamp_min(floor if floor > 0 else 1e-300)).max())
