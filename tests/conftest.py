import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def row_rel_err(got, want):
    """Attention error norm of every GPU test: for each row of the last dim (one query of one head), the largest
    |got - want| divided by the largest |want| of that same row; the result is the worst row."""
    got, want = got.float(), want.float()
    return ((got - want).abs().amax(-1) / want.abs().amax(-1).clamp_min(1e-30)).max().item()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def dev():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import diffsynth_engine_amd as dsa

    rc = dsa._lib.load().dsx_check_device()
    assert rc == 0, dsa._lib.strerror(rc)
    return torch.device("cuda:0")
