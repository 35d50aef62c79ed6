import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    import __graft_entry__
    __graft_entry__.ensure_built()          # compiles only when the tree holds no library yet


def rel_err(got, ref):
    """max|got - ref| / max|ref| and the relative L2 error, both as floats."""
    import torch
    got = got.detach().double().cpu()
    ref = ref.detach().double().cpu()
    diff = (got - ref)
    return (diff.abs().max() / ref.abs().max().clamp_min(1e-30)).item(), \
        (diff.norm() / ref.norm().clamp_min(1e-30)).item()


@pytest.fixture(scope="session")
def gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")
