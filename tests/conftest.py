import sys
from pathlib import Path

import pytest

REPO = Path(__file__).resolve().parents[1]
for p in (REPO, REPO / "kernel-align_amd"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def sampler():
    """SamplerBackend on cuda:0; fails loudly if the HIP library is not built."""
    import torch
    from rl_engine.kernels.sampling import SamplerBackend

    assert torch.cuda.is_available(), "gpu tests need a GPU"
    return SamplerBackend().to("cuda")
