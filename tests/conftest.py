import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle module, with its C library built on demand."""
    from oracle import attn_oracle, build_oracle

    if not os.path.exists(attn_oracle.C_LIB_PATH):
        build_oracle.build_oracle()
    return attn_oracle


@pytest.fixture(scope="session")
def gpu():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from flex_block_attn_amd import _lib

    _lib.load()  # fails loudly if the HIP library has not been built
    return torch.device("cuda:0")
