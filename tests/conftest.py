import os
import sys

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if REPO not in sys.path:
    sys.path.insert(0, REPO)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """A fresh checkout has no binaries: build them once (library, list helper, oracle, C driver).
    When they are there they are used as they are."""
    if not os.path.exists(os.path.join(REPO, "fairscale_amd", "csrc", "libfsadam.so")):
        import __graft_entry__

        __graft_entry__.build()


@pytest.fixture(scope="session")
def oracle():
    from oracle import adam_oracle

    adam_oracle.build()
    return adam_oracle


@pytest.fixture(scope="session")
def cuda_device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU in this process")
    return torch.device("cuda", 0)
